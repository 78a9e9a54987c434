"""mode="kernel": integer weights read straight from HBM by the gfx950 kernels.

API mirror of llmquant/quantizers/kernel.py (KernelQuantLinear, pad_activation,
KERNEL_MAX_ROWS), with one storage change: 4-bit weights live in HBM as the nibble-packed
bytes the file format holds -- [N, G, gs/2] uint8 -- instead of one code per int8 byte, so
a decode step streams half the bytes. `qweight` still hands back the canonical int8
[N, G, gs] tensor for anything that wants the reference's view of the layer.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from llmquant.core.observers import group_view, pad_to_group
from llmquant.core.scheme import QuantizationScheme
from llmquant.hip.build import load_extension
from llmquant.packing.packing import pack_int4, unpack_int4
from llmquant.quantizers.real import quantize_weight

#: up to this many activation rows the GEMV kernel runs; above it the weight is dequantized
#: once and a dense matmul takes over
KERNEL_MAX_ROWS = 4
#: ... except that up to this many rows of a 16-bit activation go to the fused GEMM, which reads
#: the codes once and builds no dense weight (the measured crossover with dequantize + matmul).
#: In its one-launch form (a workgroup owns whole weight rows) at every row count: since the activation
#: reaches the matrix core through LDS that form is the faster one on every shape measured (Llama-3.2-1B and
#: Llama-3-8B layers, lm_head), by 5-40 %; the form that splits the reduction axis across workgroups (two
#: launches) stays available through the extension (`split=True`).
FUSED_GEMM_MAX_ROWS = 64
FUSED_GEMM_WHOLE_ROWS = FUSED_GEMM_MAX_ROWS
#: ... and from this many rows on it is also faster than the GEMV kernel, which multiplies its rows
#: as int8 digit planes and slows down with each row (14336 x 4096 int4, graph replay: GEMV 9.6 /
#: 13.0 / 14.8 / 21.0 us for 1-4 rows, the fused GEMM 13.4-14.3 us for any of them)
FUSED_GEMM_MIN_ROWS = 3
FUSED_GEMM_SPLIT_GROUPS = 1 << 30   # (no row is long enough for the split form to win)


#: Prompt-sized bf16 / fp16 activations: the tiled fused GEMM (128 x 256 or 64 x 128 output tiles, no dense weight) up
#: to this many rows where its estimated time is within 5 % of the estimate for dequantize + the BLAS library's matmul
#: (beyond 1024 rows the library's 1.2-1.4 PFLOP/s kernels win by more than the dequantize pass costs)
TILED_GEMM_MAX_ROWS = 1024


def _tile_plan_cost(rows: int, out_features: int, groups: int, narrow: bool, int4: bool) -> float:
    """Microseconds of the tiled GEMM's launch for one tile shape: the plan and the cost figures of
    csrc/wq_gemm_a16_tile.hip (plan_for, plan_cost), which chooses the cheaper shape itself."""
    tile_m, tile_n = (64, 128) if narrow else (128, 256)
    tiles = -(-rows // tile_m) * -(-out_features // tile_n)
    splits = max(1, min(256 // tiles, groups // 4)) if tiles < 160 else 1
    per_split = -(-groups // splits)
    splits = -(-groups // per_split)
    fixed = 6.0 if narrow else 8.0
    per_group = (0.75 if int4 else 1.0) if narrow else (1.93 if int4 else 2.1)
    cost = -(-(tiles * splits) // 256) * (fixed + per_split * per_group)
    if splits > 1:
        cost += 3.0 + splits * rows * out_features * 8.0 / 9.0e6
    return cost


def tiled_gemm_cost(rows: int, out_features: int, groups: int, bits: int = 8, prepared: bool = False) -> float:
    """Estimated microseconds of llmq_wq_gemm_a16_tile (within a tenth of the measured launches, 128-2048 rows on
    weights of 2048-28672 rows): rounds of 256 workgroups, each a fixed part plus a time per group, the partial sums'
    way through memory where the reduction axis is cut, and 3.5 us for the activation's preparation unless the rows
    arrive prepared (llmq_add_rmsnorm_prepared, the gate|up epilogue)."""
    launch = min(_tile_plan_cost(rows, out_features, groups, narrow, bits == 4) for narrow in (False, True))
    return launch + (0.0 if prepared else 3.5)


def dense_branch_cost(rows: int, out_features: int, groups: int, bits: int = 8) -> float:
    """Estimated microseconds of dequantize + the BLAS library's matmul: 16 us of fixed cost (two launches, the
    library's dispatch), the dequantize pass at 4 TB/s (codes in, 16-bit values out), the matmul at 1.5 PFLOP/s
    (less below 400 rows and on reduction axes beyond 4096). Fitted to the same measurements; the library's kernels vary
    more with shape than this."""
    weights = out_features * groups * 128
    matmul = 2.0 * rows * weights / 1.5e9 / min(1.0, rows / 400) * (1.0 + max(0, groups * 128 - 4096) / 32768)
    return 16.0 + weights * (bits / 8 + 2) / 4.0e6 + matmul


def tiled_gemm_pays(rows: int, out_features: int, groups: int, bits: int = 8, prepared: bool = False) -> bool:
    """Whether the tiled fused GEMM is the branch for this many activation rows. Up to 128 rows: wide or long
    weights, and mid-sized ones (the fused GEMM for a few dozen rows keeps the narrow short ones). Beyond: where its
    estimated time is within 5 % of dequantize + matmul's (a tie goes to the branch that builds no dense weight).
    Measured, M x N x K int4, tiled / dense us: 512 x 16384 x 2048 46 / 54, 640 x 16384 x 2048 77 / 59 (320 tiles:
    a second round), 512 x 28672 x 4096 143 / 164, 640 x 4096 x 14336 102 / 120, 1024 x 14336 x 4096 149 / 122;
    int8: 512 x 3072 x 2048 24.2 / 24.9, 192 x 3072 x 2048 17.1 / 24.4, 1024 x 3072 x 2048 33.0 / 28.7,
    136 x 512 x 2048 12.6 / 13.8."""
    if not FUSED_GEMM_MAX_ROWS < rows <= TILED_GEMM_MAX_ROWS:
        return False
    if rows <= FUSED_GEMM_SLAB_MAX_ROWS:
        # one tile of rows on a mid-sized weight (Llama-3-8B's q|k|v, 6144 x 4096 int8, M = 65-128: 24.8-27.1 us
        # against 32.7-36.0 for dequantize + matmul); smaller weights take the fused GEMM for a few dozen rows twice
        return out_features >= 8192 or groups >= 64 or out_features * groups > FUSED_GEMM_SLAB_MAX_GROUP_ROWS
    return (tiled_gemm_cost(rows, out_features, groups, bits, prepared)
            <= 1.05 * dense_branch_cost(rows, out_features, groups, bits))


#: Narrow, short weights (N * groups up to 4096 x 32: q|k|v and o_proj of the 1B and 8B models) keep the fused GEMM up
#: to this many rows, 64 at a time: two launches of it beat both dequantize + matmul and the tiled GEMM there
#: (3072 x 2048 int8, M = 128: 14.1 us against 21.7 and 21.2; 4096 x 4096: 24.4 against 32.0 and 27.4).
FUSED_GEMM_SLAB_MAX_ROWS = 128
FUSED_GEMM_SLAB_MAX_GROUP_ROWS = 4096 * 32


def fused_gemm_takes(rows: int, out_features: int, groups: int) -> bool:
    """Whether this many rows of a 16-bit activation go to the fused GEMM for a few dozen rows."""
    if FUSED_GEMM_MIN_ROWS <= rows <= FUSED_GEMM_MAX_ROWS:
        return True
    return (FUSED_GEMM_MAX_ROWS < rows <= FUSED_GEMM_SLAB_MAX_ROWS and not tiled_gemm_pays(rows, out_features, groups)
            and out_features * groups <= FUSED_GEMM_SLAB_MAX_GROUP_ROWS)


def fused_gemm_splits(rows: int, groups: int) -> bool:
    """Which form of the fused GEMM is faster for this many activation rows and groups per weight row: the
    whole-rows form (False) at every row count, the split form only from FUSED_GEMM_SPLIT_GROUPS groups a row."""
    return groups >= FUSED_GEMM_SPLIT_GROUPS


def pad_activation(flat: torch.Tensor, args) -> torch.Tensor:
    """Zero-pad an activation into the same groups its weight was cut into (per head when the
    reduction axis carries heads)."""
    if not args.head_dim:
        return pad_to_group(flat, args.group_size)
    *lead, k = flat.shape
    heads = flat.reshape(*lead, k // args.head_dim, args.head_dim)
    return pad_to_group(heads, args.group_size).flatten(-2)


class KernelQuantLinear(nn.Module):
    """Linear over a canonical quantized weight: [N, groups, group_size] codes with padding
    and head splits already applied, plus fp32 scales [scale_rows, groups]."""

    def __init__(self, qweight, wscale, bias, scheme: QuantizationScheme, in_features: int):
        super().__init__()
        bits = scheme.weights.num_bits
        if qweight.dtype == torch.uint8:
            if bits != 4:
                raise ValueError("a uint8 (nibble-packed) weight needs a 4-bit scheme")
            stored = qweight.contiguous()
            group_size = stored.shape[2] * 2
        elif bits == 4:
            stored = pack_int4(qweight)
            group_size = qweight.shape[2]
        else:
            stored = qweight.contiguous()
            group_size = qweight.shape[2]
        self.register_buffer("qdata", stored)      # what the kernel reads
        self.register_buffer("wscale", wscale.contiguous())  # [scale_rows, groups] fp32
        self.bias = bias
        self.scheme = scheme
        self.out_features = stored.shape[0]
        self.in_features = in_features                       # the layer's real width
        self.padded_in_features = stored.shape[1] * group_size  # the canonical, padded one
        self.out_group = scheme.weights.out_group or 0
        self._packed = stored.dtype == torch.uint8
        self._needs_padding = self.in_features != self.padded_in_features
        self._weight_args = scheme.weights
        # head-aligned groups (o_proj: heads of 64 in groups of 128): real elements per group
        head_dim = scheme.weights.head_dim
        self._head_keep = (head_dim if head_dim and head_dim < group_size
                           and self.in_features == stored.shape[1] * head_dim else 0)
        # int8 activations: the integer GEMM (real-mode arithmetic, bit for bit) serves every M.
        # The reference's kernel mode ignores the activation scheme (kernel.py:97-103); here it
        # is honoured when the geometry allows (one activation group per weight group of 128).
        act = scheme.input_activations
        self._int8_act = (act is not None and act.num_bits == 8 and act.strategy == "group"
                          and act.group_size == group_size == 128)
        #: int8 activations: True keeps RealQuantLinear's fp32 roundings bit for bit; False takes the tiled
        #: integer GEMM that folds a group in with one rounding fewer (same integer sums, agrees to ~1e-7
        #: relative) and runs up to twice as fast on prompt-sized activations
        self.a8_exact = True
        # the fused GEMM's reach (it needs groups of 128)
        self._fused_max_rows = FUSED_GEMM_MAX_ROWS if group_size == 128 else 0
        # looked up once: a decode step runs ~113 of these modules
        self._ext = load_extension()
        self._gemv = self._ext.wq_gemv

    # the loaded extension is a module object, which copy and pickle refuse: a copy (copy.deepcopy(model),
    # torch.save of the module) carries everything else and looks the extension up again
    def __getstate__(self):
        state = dict(self.__dict__)
        state.pop("_ext", None)
        state.pop("_gemv", None)
        return state

    def __setstate__(self, state):
        super().__setstate__(state)
        self._ext = load_extension()
        self._gemv = self._ext.wq_gemv

    @classmethod
    def from_linear(cls, linear: nn.Linear, scheme: QuantizationScheme):
        if scheme.weights is None:
            raise ValueError("the kernel path needs a weight scheme; bf16 weights stay nn.Linear")
        args = scheme.weights
        codes, scale = quantize_weight(linear.weight.detach(), args)
        canonical = group_view(codes, args.group_size, args.head_dim).contiguous()
        scales = scale.reshape(-1, canonical.shape[1]).contiguous().float()
        return cls(canonical, scales, linear.bias, scheme, linear.in_features)

    @property
    def qweight(self) -> torch.Tensor:
        """Canonical int8 codes [N, groups, group_size] (unpacked on demand for 4-bit)."""
        return unpack_int4(self.qdata) if self._packed else self.qdata

    @property
    def _broadcast_scale(self) -> torch.Tensor:
        """[N, groups, 1] fp32: every row's scales, tiles expanded."""
        repeat = self.out_features // self.wscale.shape[0]
        return self.wscale.repeat_interleave(repeat, dim=0).unsqueeze(-1)

    # ---- state_dict in the reference's terms -----------------------------------------------------------
    # The reference registers `qweight` ([N, groups, gs] int8), `wscale` and `_broadcast_scale` ([N, groups, 1])
    # as persistent buffers (llmquant/quantizers/kernel.py:36-54). state_dict() here writes those three keys
    # with those shapes and dtypes (4-bit codes unpacked to one per int8 byte), and load_state_dict() takes
    # either that form or this module's own stored form (`qdata`, nibble-packed for 4 bits), so a kernel-mode
    # state_dict moves between the two implementations in both directions.
    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        stored = destination.pop(prefix + "qdata")
        wscale = destination.pop(prefix + "wscale")
        destination[prefix + "qweight"] = unpack_int4(stored) if self._packed else stored
        destination[prefix + "wscale"] = wscale
        broadcast = self._broadcast_scale
        destination[prefix + "_broadcast_scale"] = broadcast if keep_vars else broadcast.detach()

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        theirs = state_dict.pop(prefix + "qweight", None)
        if theirs is not None and prefix + "qdata" not in state_dict:
            if self._packed and theirs.dtype == torch.int8:
                theirs = pack_int4(theirs)
            state_dict[prefix + "qdata"] = theirs
        state_dict.pop(prefix + "_broadcast_scale", None)  # derived from wscale on demand
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)

    def _dequantized_weight(self, dtype, real_width: bool = False):
        """[out, padded_in] in the activation dtype, rebuilt per call and never cached: one kernel
        pass (the reference multiplies and casts in PyTorch, kernel.py:68-79). With `real_width`
        and head-aligned groups the zero padding is dropped: [out, in_features]."""
        group_size = self.padded_in_features // self.qdata.shape[1]
        if group_size % 8 == 0:
            keep = self._head_keep if real_width else 0
            return self._ext.dequant_weight(self.qdata, self.wscale, self.out_group, keep, dtype)
        return (self.qweight * self._broadcast_scale).to(dtype).reshape(self.out_features, -1)

    def _dense(self, rows, real_width: bool = False):
        """rows @ W.T on the dense branch. bf16 / fp16: one extension call (dequantize pass, then the BLAS
        library's matmul with its plan kept per shape: same bits as `@`, half the host time)."""
        group_size = self.padded_in_features // self.qdata.shape[1]
        if rows.dtype in (torch.bfloat16, torch.float16) and group_size % 8 == 0:
            keep = self._head_keep if real_width else 0
            return self._ext.wq_dense_linear(rows.contiguous(), self.qdata, self.wscale, self.out_group, keep)
        return rows @ self._dequantized_weight(rows.dtype, real_width).T

    def forward(self, x):
        rows = x.reshape(-1, x.shape[-1])
        # (heads padded to groups: above 64 rows the dense branch on the real width reads half the codes)
        fused = (self._fused_max_rows > 0 and fused_gemm_takes(rows.shape[0], self.out_features, self.qdata.shape[1])
                 and (rows.shape[0] <= self._fused_max_rows or not self._head_keep)
                 and rows.dtype in (torch.bfloat16, torch.float16) and not self._int8_act)
        tiled = (self._fused_max_rows > 0 and rows.dtype in (torch.bfloat16, torch.float16) and not self._int8_act
                 and tiled_gemm_pays(rows.shape[0], self.out_features, self.qdata.shape[1],
                                     4 if self.qdata.dtype == torch.uint8 else 8))
        if rows.shape[0] > KERNEL_MAX_ROWS and not self._int8_act and self._head_keep and not fused and not tiled:
            # dense branch on the real width: neither the activation nor the weight is padded
            out = self._dense(rows, real_width=True)
            if self.bias is not None:
                out = out + self.bias.to(out.dtype)
            return out.reshape(*x.shape[:-1], self.out_features).to(x.dtype)
        if self._needs_padding:
            rows = pad_activation(rows, self._weight_args)
        if self._int8_act:
            if (self.a8_exact and rows.dtype in (torch.bfloat16, torch.float16) and x.dtype == rows.dtype
                    and self._ext.wq_gemm_a8_takes_groups(rows.shape[0], self.out_features, self.qdata.shape[1])):
                # few output tiles, long rows: the group-parallel kernel, with the codes written in its operand order
                # by the quantizer (the same codes and scales, the same result bit for bit)
                codes, act_scale = self._ext.quant_act_codes_tiled(rows.contiguous(),
                                                                   4 if self.qdata.dtype == torch.uint8 else 8)
                out = self._ext.wq_gemm_a8_tiled(codes, act_scale, rows.shape[0], self.qdata, self.wscale, self.bias,
                                                 self.out_group, x.dtype)
                return out.reshape(*x.shape[:-1], self.out_features)
            codes, act_scale = self._ext.quant_group_codes(rows, 8, 128, False)
            out = self._ext.wq_gemm_a8(codes, act_scale, self.qdata, self.wscale, self.bias, self.out_group,
                                       x.dtype, self.a8_exact)
            return out.reshape(*x.shape[:-1], self.out_features)
        if fused:
            out = self._ext.wq_gemm_a16(rows, self.qdata, self.wscale, self.out_group,
                                        fused_gemm_splits(rows.shape[0], self.qdata.shape[1]))
        elif rows.shape[0] <= KERNEL_MAX_ROWS:
            out = self._gemv(rows, self.qdata, self.wscale, self.out_group)
        elif tiled:
            out = self._ext.wq_gemm_a16_tile(rows, self.qdata, self.wscale, self.out_group)
        else:
            out = self._dense(rows)
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out.reshape(*x.shape[:-1], self.out_features).to(x.dtype)

    def extra_repr(self):
        a = self.scheme.input_activations
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"w{self.scheme.weights.num_bits}a{a.num_bits if a else 16}, "
                f"group_size={self.scheme.weights.group_size}")
