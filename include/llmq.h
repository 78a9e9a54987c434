/*
 * llmq.h -- C ABI of libllmq_hip.so, the gfx950 (MI355X) kernels behind llm-quant's
 * `mode="kernel"` path.
 *
 * Every entry point
 *   - takes plain device pointers, sizes and a stream; no torch or HIP C++ types,
 *   - launches on the given stream and returns without synchronising or reading back,
 *     so a caller may record it into a HIP graph,
 *   - allocates nothing (callers own inputs, outputs and workspaces),
 *   - returns 0 on success, otherwise a hipError_t value (1 = invalid argument); the text
 *     for the most recent failure on the calling thread is llmq_last_error().
 *
 * The reference (pjh5672/llm-quant) binds its kernels as a torch extension in
 * llmquant/cuda/csrc/fake_quant.cpp:21-51; the functions below are what that binding's
 * four ops reduce to once tensor checks and allocation are peeled off, plus the ops the
 * reference still runs as PyTorch chains (activation quant, W4A8 GEMM, KV-cache quant and
 * decode attention).
 */
#ifndef LLMQ_H
#define LLMQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A hipStream_t, passed as an opaque pointer so this header needs no HIP include. */
typedef void* llmq_stream_t;

/* Element type of activations / outputs. Values are stable: they are part of the ABI. */
enum llmq_dtype { LLMQ_F32 = 0, LLMQ_F16 = 1, LLMQ_BF16 = 2 };

/* Weight storage. INT8: one code per byte, [N, G, gs]. INT4_PACKED: two codes per byte,
 * [N, G, gs/2], each code biased by +8, even k in the low nibble -- the bytes
 * llmquant/packing/packing.py:20-33 writes to disk. */
enum llmq_wformat { LLMQ_W_INT8 = 8, LLMQ_W_INT4_PACKED = 4 };

#define LLMQ_GEMV_MAX_ROWS 4

int llmq_abi_version(void);
const char* llmq_last_error(void);

/* Fused symmetric RTN quantize-dequantize over contiguous groups of the last axis.
 * Replaces fake_quant_group (llmquant/cuda/csrc/fake_quant.cu:88-139), bit-exact with
 * fake_quantize (llmquant/core/quant_ops.py:26-37):
 *   scale = max(amax(|x|)/qmax, 1e-8); q = clamp(rint(x/scale), -qmax-1, qmax); out = q*scale
 * x, out: n_groups*group_size elements of `dtype`; scale_or_null: n_groups fp32 or NULL.
 * num_bits in [2, 8]. */
int llmq_fake_quant_group(const void* x, void* out, float* scale_or_null, int64_t n_groups,
                          int group_size, int num_bits, int dtype, llmq_stream_t stream);

/* Same arithmetic, but emits the integer codes instead of the dequantized values:
 * codes int8 [n_groups*group_size] (pack4 == 0) or nibble-packed uint8
 * [n_groups*group_size/2] (pack4 != 0, num_bits <= 4), scale fp32 [n_groups].
 * This is compute_scale + quantize (llmquant/core/observers.py:74-98,
 * llmquant/core/quant_ops.py:13-19) as one pass: the activation quantizer of the A8 path
 * (llmquant/quantizers/real.py:89-90). */
int llmq_quant_group_codes(const void* x, void* codes, float* scale, int64_t n_groups,
                           int group_size, int num_bits, int pack4, int dtype,
                           llmq_stream_t stream);

/* Weight-only quantized GEMV, out[m, n] = sum_g wscale[sr(n), g] * sum_{k in g} x[m, k]*q[n, g, k]
 * with sr(n) = n / out_group when out_group > 0, else n. fp32 accumulation, result cast
 * to `dtype`. Replaces wq_gemv (llmquant/cuda/csrc/wq_gemv.cu:134-185).
 * x: [M, G*gs] `dtype`; qweight: see llmq_wformat; wscale: fp32 [scale_rows, G];
 * out: [M, N] `dtype`. Any M >= 0 (rows are processed LLMQ_GEMV_MAX_ROWS at a time).
 * gs must be a multiple of 4 (int8) or 8 (packed int4). */
int llmq_wq_gemv(const void* x, const void* qweight, const float* wscale, void* out, int M,
                 int N, int G, int gs, int out_group, int wformat, int dtype,
                 llmq_stream_t stream);

/* Many small GEMVs in one launch: the routed experts of a Mixture-of-Experts layer. Replaces
 * wq_gemv_batched (llmquant/cuda/csrc/wq_gemv_batched.cu:39-186). qweight is [E, N, G, gs] (or
 * packed [E, N, G, gs/2]), wscale [E, scale_rows, G]. Plan entry b (three device int32 arrays of
 * n_blocks entries, built by the caller on the device and never read by the host) says: rows
 * block_row0[b] .. +block_rows[b]-1 of x [n_rows, G*gs] go through expert block_expert[b]; an entry
 * with block_rows <= 0 is skipped, one that points outside x or the expert stack is ignored. A run
 * holds at most llmq_wq_gemv_batched_max_rows() rows, and runs do not overlap (so at most n_rows
 * entries hold rows: the launch is sized for that many). out: [n_rows, N]; rows no entry covers are
 * left untouched. Each row's arithmetic is llmq_wq_gemv's. */
int llmq_wq_gemv_batched_max_rows(void);
int llmq_wq_gemv_batched(const void* x, const void* qweight, const float* wscale, void* out,
                         const int32_t* block_expert, const int32_t* block_row0,
                         const int32_t* block_rows, int n_blocks, int n_rows, int n_experts, int N,
                         int G, int gs, int out_group, int wformat, int dtype, llmq_stream_t stream);

/* The routing plan llmq_wq_gemv_batched takes, in one launch: what KernelQuantExperts._plan
 * (llmquant/quantizers/kernel.py:176-214) computes with a stable argsort, scatter_add, cumsum and
 * arange arithmetic in PyTorch, same integers. expert_of_row: [n_rows] expert of every (token, slot)
 * row (top_k_index flattened; an id outside [0, n_experts) is counted with the nearest valid one).
 * order: [n_rows], order[i] = index of the i-th row when the rows are sorted by expert, equal experts
 * in their original order. Every expert gets B = llmq_route_plan_blocks_per_expert(n_rows, limit) =
 * max(1, ceil(n_rows / limit)) entries: block_expert / block_row0 / block_rows are [n_experts * B],
 * entry e * B + b = (e, first[e] + b * limit, clamp(count[e] - b * limit, 0, limit)). One workgroup;
 * llmq_route_plan_supported says whether the sizes fit it (up to 8192 rows, 1024 experts). */
int llmq_route_plan_blocks_per_expert(int n_rows, int limit);
int llmq_route_plan_supported(int n_rows, int n_experts);
int llmq_route_plan(const int64_t* expert_of_row, int n_rows, int n_experts, int limit, int64_t* order,
                    int32_t* block_expert, int32_t* block_row0, int32_t* block_rows, llmq_stream_t stream);

/* llmq_wq_gemv_batched for the two projections of a gated Mixture-of-Experts block with the
 * PyTorch steps around them folded in (KernelQuantExperts.forward, llmquant/quantizers/kernel.py:
 * 221-253, runs them as separate kernels). Group size 128, one scale row per weight row.
 *   x_row_stride  elements between the rows of x; 0: every row is x[0] (one token routed to several
 *                 experts: `hidden_states[tokens_per_row]` without the gather)
 *   act_pair != 0 qweight is [experts, 2I, G, gs] (gate rows, then up rows) and out is [n_rows, I]
 *                 = dtype(dtype(silu(dtype(gate))) * dtype(up)): `act_fn(gate) * up` for SiLU
 * Every row must be covered by the plan (out is written, not accumulated). */
int llmq_wq_gemv_batched_fused(const void* x, int64_t x_row_stride, const void* qweight,
                               const float* wscale, void* out, const int32_t* block_expert,
                               const int32_t* block_row0, const int32_t* block_rows, int n_blocks,
                               int n_rows, int n_experts, int N, int G, int wformat, int dtype,
                               int act_pair, llmq_stream_t stream);

/* The end of KernelQuantExperts.forward (kernel.py:247-252) in one launch:
 *   final[t, :] = sum over the rows i routed from token t of dtype(rows_out[i, :] * weights[order[i]])
 * accumulated in `dtype` (every addition rounded, as index_add_ on a `dtype` tensor does) in the
 * order of the sorted rows, i.e. by ascending expert: one of the orders the reference's atomic
 * index_add_ may take, and the same one on every run. rows_out: [n_rows, width]; order: [n_rows]
 * from llmq_route_plan (order[i] = token * top_k + slot); weights: [n_tokens * top_k] `dtype`;
 * final: [n_tokens, width], written in full (tokens nobody routed get zeros). */
int llmq_moe_combine(const void* rows_out, const int64_t* order, const void* weights, void* final_out,
                     int n_rows, int top_k, int n_tokens, int width, int dtype, llmq_stream_t stream);

/* The decode-step form of llmq_wq_gemv (M = 1, group size 128): the same product with the
 * elementwise operations that surround a Linear in a Llama decoder layer folded in, so that a
 * layer is five launches instead of ~40. There is no counterpart in the reference, which leaves
 * these operations to PyTorch (transformers' LlamaDecoderLayer); each is computed with the same
 * rounding points as the PyTorch form:
 *   prologue LLMQ_PRO_RMSNORM   x' = w * dtype(x * rsqrt(mean(x^2) + eps))     (LlamaRMSNorm)
 *            LLMQ_PRO_SILU_MUL  x is [gate | up], x' = dtype(dtype(silu(gate)) * up)   (LlamaMLP)
 *   in_head_dim > 0             x is [G * in_head_dim]; group g multiplies head g zero-padded to
 *                               128, i.e. pad_activation (llmquant/quantizers/kernel.py:17-25)
 *   residual != NULL            out = dtype(residual + dtype(y))
 * x, norm_weight, residual, out all have element type `dtype`. */
enum llmq_prologue { LLMQ_PRO_NONE = 0, LLMQ_PRO_RMSNORM = 1, LLMQ_PRO_SILU_MUL = 2,
                     LLMQ_PRO_ATTN_MERGE = 3 /* only through llmq_wq_gemv_attn_merge */ };
int llmq_wq_gemv_fused(const void* x, const void* qweight, const float* wscale, void* out, int N,
                       int G, int out_group, int wformat, int dtype, int prologue,
                       const void* norm_weight, float eps, int in_head_dim,
                       const void* residual_or_null, llmq_stream_t stream);

/* llmq_wq_gemv_fused for the gate|up weight of a gated MLP with the activation folded into the
 * store: qweight is [2 * intermediate, G, gs] (gate rows, then up rows: transformers' fused
 * gate_up_proj, or gate_proj over up_proj), out is [intermediate] with
 *   out[i] = dtype(dtype(silu(dtype(y[i]))) * dtype(y[intermediate + i]))
 * which is LLMQ_PRO_SILU_MUL applied to the [gate | up] output of the plain GEMV (LlamaMLP), so the
 * GEMV that follows (down_proj) takes it with no prologue. A row tile multiplies eight gate rows
 * and their eight up rows; `intermediate` must be a multiple of 8. prologue: LLMQ_PRO_NONE or
 * LLMQ_PRO_RMSNORM. One scale row per weight row. No counterpart in the reference. */
int llmq_wq_gemv_gate_up_silu(const void* x, const void* qweight, const float* wscale, void* out,
                              int intermediate, int G, int wformat, int dtype, int prologue,
                              const void* norm_weight, float eps, llmq_stream_t stream);

/* The dense form of a quantized weight, out[n, g*keep + k] = (dtype)(code[n,g,k] * wscale[sr(n),g])
 * for k < keep_per_group <= gs: the matrix KernelQuantLinear builds per forward when more rows
 * arrive than the GEMV takes (`_dequantized_weight`, llmquant/quantizers/kernel.py:68-79), in one
 * pass. keep_per_group < gs drops the zero padding of head-aligned groups, giving the layer's real
 * input width. out: [N, G*keep_per_group] `dtype`. gs a multiple of 8. */
int llmq_dequant_weight(const void* qweight, const float* wscale, void* out, int N, int G, int gs,
                        int keep_per_group, int out_group, int wformat, int dtype,
                        llmq_stream_t stream);

/* Integer GEMM with per-group scales on both operands (the A8 branch of
 * RealQuantLinear.forward, llmquant/quantizers/real.py:76-103):
 *   out[m, n] = sum over g, in order, of  float(sum_k a[m,g,k]*q[n,g,k]) * sw[sr(n), g] * sx[m, g]
 * each group's term rounded to fp32 after every multiply and added sequentially, then
 * bias (fp32, nullable) added and the sum cast to `dtype`. gs must be 128.
 * a: int8 [M, G*128]; sx: fp32 [M, G]; qweight/wscale as for llmq_wq_gemv. G <= 2^17 (rows of up
 * to 2^24 codes). */
int llmq_wq_gemm_a8(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                    const float* bias_or_null, void* out, int M, int N, int G, int gs,
                    int out_group, int wformat, int dtype, llmq_stream_t stream);

/* llmq_wq_gemm_a8 with the activation codes in operand order, for the shapes where it runs its group-parallel
 * kernel (few output tiles, long rows; llmq_wq_gemm_a8_takes_groups(M, N, G) != 0 says where this call is the
 * faster one; LLMQ_A8_FORM in the environment pins the answer): the same result bit for bit, without the pass that turns activation rows into matrix-core operand
 * layout inside the kernel (128 x 4096 x 14336 int4: 38 -> 31 us). llmq_quant_act_codes_tiled is llmq_quant_group_codes
 * (int8 codes, groups of 128, the same arithmetic: scales [M, K / 128] equal) writing the codes where the kernel's
 * waves read them: blocks of 32 rows x one group, [ceil(M / 32)][K / 128][4096] bytes, inside a block [k-step 0..3]
 * [row % 32 + 32 * (k / 64)][16], and for packed int4 weights (wformat 4) every eight bytes as even k then odd k;
 * `codes`: llmq_act_codes_tiled_bytes(M, K) bytes, 16-byte aligned; x: LLMQ_BF16 or LLMQ_F16 [M, K] contiguous.
 * llmq_wq_gemm_a8_tiled takes any shape (arguments as for llmq_wq_gemm_a8, `codes_tiled` made for the same wformat).
 * No counterpart in the reference, whose real mode keeps the codes inside RealQuantLinear.forward
 * (llmquant/quantizers/real.py:76-88). */
size_t llmq_act_codes_tiled_bytes(int M, int K);
int llmq_quant_act_codes_tiled(const void* x, void* codes, float* scale, int M, int K, int wformat, int dtype,
                               llmq_stream_t stream);
int llmq_wq_gemm_a8_tiled(const void* codes_tiled, const float* sx, const void* qweight, const float* wscale,
                          const float* bias_or_null, void* out, int M, int N, int G, int gs, int out_group,
                          int wformat, int dtype, llmq_stream_t stream);
int llmq_wq_gemm_a8_takes_groups(int M, int N, int G);

/* The same GEMM in its fast form: the same exact integer group sums, folded into the total as
 * fma((float)isum * sw, sx, total) (one instruction and one rounding fewer than RealQuantLinear's
 * ((float)isum * sw) * sx followed by an add, llmquant/quantizers/real.py:94-99). Where the output has too few
 * tiles to fill the chip the reduction axis is split across workgroups (fp32 partial tiles added in a fixed
 * order by a second launch). Agrees with llmq_wq_gemm_a8 to fp32 rounding (rel-L2 ~1e-7), not bit for bit.
 * Arguments as for llmq_wq_gemm_a8 plus `sx_groups`: G for sx [M, G], or 1 for one activation scale per token,
 * sx [M] (the scale then leaves the sum over groups: two instructions per output and group instead of
 * three); and `workspace`: llmq_wq_gemm_a8_fast_workspace_bytes(M, N, G) bytes (0 where nothing is split: then
 * it may be null), 16-byte aligned, contents irrelevant before and after (the activation in operand order and
 * the partial tiles); calls that share a workspace must not overlap. */
size_t llmq_wq_gemm_a8_fast_workspace_bytes(int M, int N, int G);
int llmq_wq_gemm_a8_fast(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                         const float* bias_or_null, void* out, void* workspace, size_t workspace_bytes, int M,
                         int N, int G, int sx_groups, int gs, int out_group, int wformat, int dtype,
                         llmq_stream_t stream);

/* Weight-only GEMM for more rows than the GEMV takes, without the dense copy of the weight that
 * KernelQuantLinear builds per forward for M > KERNEL_MAX_ROWS (`_dequantized_weight` + matmul,
 * llmquant/quantizers/kernel.py:68-79, 88-91):
 *   out[m, n] = sum over g of  wscale[sr(n), g] * sum_k x[m, g*128 + k] * code[n, g, k]
 * in the form of RealQuantLinear's weight-only branch (llmquant/quantizers/real.py:84-91), fp32
 * accumulation on the matrix cores, cast to `dtype`. x, out: LLMQ_F16 or LLMQ_BF16, [M, G*128] and
 * [M, N]; qweight/wscale as for llmq_wq_gemv; gs must be 128. Any M: rows are taken 64 at a time and
 * every slab streams the weight once, so this pays up to a few dozen rows. */
int llmq_wq_gemm_a16(const void* x, const void* qweight, const float* wscale, void* out, int M, int N,
                     int G, int gs, int out_group, int wformat, int dtype, llmq_stream_t stream);

/* The same GEMM with the reduction axis split across workgroups (128 weight rows x 4 groups each):
 * every workgroup copies only its slice of x into LDS, so the bytes the CUs pull in stay close to
 * the codes' own whatever M, and the launch has N/128 * ceil(G/4) workgroups whatever the shape. The
 * slices' fp32 sums go through `workspace` (llmq_wq_gemm_a16_workspace_bytes(M, N, G) bytes, 16-byte
 * aligned, contents irrelevant before and after) and a second launch adds them in a fixed order; with
 * G <= 4 there is one slice, no workspace and no second launch. Same arguments and result form as
 * llmq_wq_gemm_a16 otherwise. Calls that share a workspace must not overlap. No counterpart in the
 * reference. */
size_t llmq_wq_gemm_a16_workspace_bytes(int M, int N, int G);
int llmq_wq_gemm_a16_split(const void* x, const void* qweight, const float* wscale, void* out,
                           void* workspace, size_t workspace_bytes, int M, int N, int G, int gs,
                           int out_group, int wformat, int dtype, llmq_stream_t stream);

/* The same GEMM for prompt-sized activations (M in the hundreds and thousands), the reference's M > 4 branch
 * (dequantize the whole weight to the activation dtype, then the BLAS library: llmquant/quantizers/kernel.py:
 * 68-79, 88-91) without the dense weight: 128 x 256 output tiles (64 x 128 where the output has few of those; the
 * cheaper plan by an estimate of both, LLMQ_A16_TILE=wide / narrow in the environment pins one), 16-bit matrix
 * cores, codes turned into operands in registers, the reduction axis split across workgroups (fp32 partial tiles,
 * added in a fixed order by a second launch) when the output has too few tiles to occupy the chip. Same sum as
 * llmq_wq_gemm_a16: products exact, fp32 accumulation, one scale per group.
 * x, out: LLMQ_BF16 or LLMQ_F16, 16-byte aligned; gs must be 128. `workspace`: llmq_wq_gemm_a16_tile_workspace_bytes
 * (M, N, G) bytes, 16-byte aligned, contents irrelevant before and after (it holds the activation in operand
 * order, its per-group sums, and the partial tiles). Calls that share a workspace must not overlap. */
size_t llmq_wq_gemm_a16_tile_workspace_bytes(int M, int N, int G);
int llmq_wq_gemm_a16_tile(const void* x, const void* qweight, const float* wscale, void* out, void* workspace,
                          size_t workspace_bytes, int M, int N, int G, int gs, int out_group, int wformat,
                          int dtype, llmq_stream_t stream);

/* gate_proj | up_proj and the activation between them and down_proj in one launch, for the prompt pass of a gated
 * MLP (transformers' LlamaMLP: down_proj(act_fn(gate_proj(x)) * up_proj(x)), each Linear on the reference's
 * M > 4 branch, llmquant/quantizers/kernel.py:68-79,88-91): `qweight` is gate_proj's I rows followed by up_proj's
 * I rows ([2 I, G, gs], wscale [2 I (or tiles of out_group), G]); a workgroup multiplies 128 gate rows and the
 * 128 up rows that belong to them, rounds both results to bfloat16 as the two Linears would, and writes
 * silu(gate) * up (rounded where `act_fn(gate) * up` on bfloat16 tensors rounds) for its 128 x 128 block directly as
 * the prepared activation of the next GEMM: into the first llmq_wq_gemm_a16_tile_prepared_bytes(M, I / 128) bytes
 * of `next_workspace`, which is then the workspace of llmq_wq_gemm_a16_tile_prepared on down_proj's weight
 * (N, G = I / 128). The bits are those of llmq_wq_gemm_a16_tile + llmq_silu_mul_rows + llmq_wq_gemm_a16_tile.
 * I must be a multiple of 128; the reduction axis is never split (use it where ceil(M / 128) * I / 128 workgroups
 * fill the chip). `workspace`: at least llmq_wq_gemm_a16_tile_prepared_bytes(M, G) bytes. */
size_t llmq_wq_gemm_a16_tile_prepared_bytes(int M, int G);
int llmq_wq_gemm_a16_tile_gate_up_silu(const void* x, const void* qweight, const float* wscale, void* workspace,
                                       size_t workspace_bytes, void* next_workspace, size_t next_workspace_bytes,
                                       int M, int I, int G, int gs, int out_group, int wformat, int dtype,
                                       llmq_stream_t stream);
/* llmq_wq_gemm_a16_tile_gate_up_silu on an activation that is already in `workspace` in prepared form (left there
 * by llmq_add_rmsnorm_prepared): no x. */
int llmq_wq_gemm_a16_tile_gate_up_silu_prepared(const void* qweight, const float* wscale, void* workspace,
                                                size_t workspace_bytes, void* next_workspace,
                                                size_t next_workspace_bytes, int M, int I, int G, int gs, int out_group,
                                                int wformat, int dtype, llmq_stream_t stream);
/* llmq_add_rmsnorm (below) whose normed rows are written in the tiled GEMM's prepared form into the first
 * llmq_wq_gemm_a16_tile_prepared_bytes(rows, hidden / 128) bytes of `workspace` instead of as a tensor: what
 * llmq_wq_gemm_a16_tile would make of that tensor, bit for bit, without the tensor and without the preparation
 * launch; `workspace` is then the workspace of llmq_wq_gemm_a16_tile_prepared (q|k|v) or
 * llmq_wq_gemm_a16_tile_gate_up_silu_prepared with M = rows, G = hidden / 128. LLMQ_BF16 or LLMQ_F16; hidden a multiple
 * of 128; delta_or_null and sum_out_or_null as in llmq_add_rmsnorm. No counterpart in the reference (transformers'
 * LlamaRMSNorm.forward followed by the Linear's M > 4 branch, llmquant/quantizers/kernel.py:68-79). */
int llmq_add_rmsnorm_prepared(const void* x, const void* delta_or_null, const void* weight, void* sum_out_or_null,
                              void* workspace, size_t workspace_bytes, int rows, int hidden, float eps, int dtype,
                              llmq_stream_t stream);
/* llmq_wq_gemm_a16_tile on an activation that is already in `workspace` in prepared form (left there by
 * llmq_wq_gemm_a16_tile_gate_up_silu or llmq_add_rmsnorm_prepared): no x. workspace_bytes as for
 * llmq_wq_gemm_a16_tile. */
int llmq_wq_gemm_a16_tile_prepared(const void* qweight, const float* wscale, void* out, void* workspace,
                                   size_t workspace_bytes, int M, int N, int G, int gs, int out_group, int wformat,
                                   int dtype, llmq_stream_t stream);

/* The elementwise pieces of a prompt pass, one launch each, with the rounding points of the PyTorch
 * sequences they replace (the same ones the decode kernels use). dtype: LLMQ_F32 / F16 / BF16; all
 * tensors 16-byte aligned. No counterpart in the reference, which leaves these to transformers
 * (LlamaRMSNorm.forward, apply_rotary_pos_emb, LlamaMLP.forward: ~20 PyTorch kernels per layer).
 *   llmq_rmsnorm   out[r, :] = weight * (dtype)(x[r, :] * rsqrt(mean(x[r, :]^2) + eps)), fp32 inside;
 *                  hidden a multiple of 8 (4 for fp32). llmq_add_rmsnorm: the same on (dtype)(x + delta),
 *                  which is also written to sum_out (the residual add in front of a norm); delta and
 *                  sum_out both NULL make it llmq_rmsnorm
 *   llmq_rope_qk   q [tokens, q_heads * head_dim] and k [tokens, kv_heads * head_dim] (row strides in
 *                  elements) rotated by cos / sin [tokens, head_dim] into contiguous q_out / k_out:
 *                  (dtype)((dtype)(x * cos) + (dtype)(rotate_half(x) * sin)); head_dim a multiple of 16
 *                  (8 for fp32)
 *   llmq_silu_mul  out = (dtype)((dtype)silu(gate) * up) over `count` elements; _rows: gate and up as
 *                  [rows, width] with row strides in elements (two column blocks of one projection's output),
 *                  out contiguous [rows, width] */
int llmq_rmsnorm(const void* x, const void* weight, void* out, int rows, int hidden, float eps, int dtype,
                 llmq_stream_t stream);
int llmq_add_rmsnorm(const void* x, const void* delta_or_null, const void* weight, void* sum_out_or_null,
                     void* out, int rows, int hidden, float eps, int dtype, llmq_stream_t stream);
int llmq_rope_qk(const void* q, const void* k, const void* cos_rows, const void* sin_rows, void* q_out,
                 void* k_out, int tokens, int q_heads, int kv_heads, int head_dim, int64_t q_row_stride,
                 int64_t k_row_stride, int dtype, llmq_stream_t stream);
int llmq_silu_mul(const void* gate, const void* up, void* out, int64_t count, int dtype, llmq_stream_t stream);
int llmq_silu_mul_rows(const void* gate, const void* up, void* out, int64_t rows, int width,
                       int64_t gate_row_stride, int64_t up_row_stride, int dtype, llmq_stream_t stream);

/* KV cache, one layer. Codes are [kv_heads, t_max, head_dim] int8 (bits == 8) or
 * [kv_heads, t_max, head_dim/2] nibble-packed uint8 (bits == 4); scales are fp32
 * [kv_heads, t_max]: one scale per token per head, which is what FakeQuantCache's
 * group-128 rule gives for head_dim <= 128 (llmquant/quantizers/fake.py:39-55).
 *
 * llmq_kv_append quantizes `n_new` tokens of K and V ([kv_heads, n_new, head_dim] `dtype`,
 * token stride given in elements so a [heads, T, D] view of a larger tensor works) and
 * writes them at positions *pos_dev .. *pos_dev + n_new - 1, where pos_dev is a device
 * int32 (read by the kernel, never by the host). When dq_k / dq_v are non-NULL the
 * dequantized values (dtype)(q*scale) are also written there ([kv_heads, n_new, head_dim]),
 * which is what FakeQuantCache.update hands back to attention during prefill. */
int llmq_kv_append(const void* k_new, const void* v_new, int64_t head_stride,
                   int64_t token_stride, void* k_codes, void* v_codes, float* k_scale,
                   float* v_scale, void* dq_k_or_null, void* dq_v_or_null,
                   const int32_t* pos_dev, int n_new, int kv_heads, int head_dim, int t_max,
                   int bits, int dtype, llmq_stream_t stream);

/* The prompt pass's RoPE and append in one launch: equivalent to llmq_rope_qk on q and k followed
 * by llmq_kv_append of the rotated k and of v, bit for bit (the rotated key is rounded to `dtype`
 * before it is quantized, as the tensor between the two launches would be). q / k / v: [tokens,
 * heads, head_dim] with the given element strides between tokens (column blocks of one q|k|v
 * projection output work); cos_rows / sin_rows: [tokens, head_dim]; q_out: [tokens, q_heads,
 * head_dim]; dq_k / dq_v: [kv_heads, tokens, head_dim] or both NULL. head_dim 64 or 128. No
 * counterpart in the reference, which runs apply_rotary_pos_emb and FakeQuantCache.update as
 * PyTorch chains (llmquant/quantizers/fake.py:39-55). */
int llmq_rope_kv_append(const void* q, const void* k, const void* v, int64_t q_row_stride,
                        int64_t k_row_stride, int64_t v_row_stride, const void* cos_rows,
                        const void* sin_rows, void* q_out, void* k_codes, void* v_codes, float* k_scale,
                        float* v_scale, void* dq_k_or_null, void* dq_v_or_null, const int32_t* pos_dev,
                        int tokens, int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                        int dtype, llmq_stream_t stream);

/* Dequantize positions 0 .. n_tokens-1 of one layer's cache to [kv_heads, n_tokens, head_dim]
 * `dtype`: (dtype)(code * scale), the tensor FakeQuantCache.update returns
 * (llmquant/quantizers/fake.py:52-55) when attention is not run by the fused decode kernel. */
int llmq_kv_dequant(const void* codes, const float* scale, void* out, int kv_heads, int head_dim,
                    int t_max, int n_tokens, int bits, int dtype, llmq_stream_t stream);

/* Single-token grouped-query attention over the quantized cache: for each query head h
 * (kv head h / (q_heads/kv_heads)), softmax(q_h . K^T * sm_scale) V over tokens
 * 0 .. *len_dev - 1, with K and V dequantized on read as (dtype)(code*scale) to keep the
 * rounding point of FakeQuantCache. Scores and softmax in fp32.
 * q: [q_heads, head_dim] `dtype`; out: [q_heads, head_dim] `dtype`.
 * head_dim 64 or 128; q_heads / kv_heads in {1, 2, 4, 8}.
 * workspace: at least llmq_kv_decode_workspace_floats(q_heads, head_dim, t_max) floats, zeroed once
 * by the caller before first use (it holds arrival counters that each launch leaves at zero);
 * launches that share a workspace must not overlap. There is no counterpart kernel in the
 * reference: it runs HF attention over the dequantized bf16 cache (llmquant/quantizers/fake.py:39-55). */
size_t llmq_kv_decode_workspace_floats(int q_heads, int head_dim, int t_max);
int llmq_kv_decode_attention(const void* q, const void* k_codes, const void* v_codes,
                             const float* k_scale, const float* v_scale, void* out,
                             float* workspace, const int32_t* len_dev, float sm_scale,
                             int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                             int dtype, llmq_stream_t stream);

/* llmq_kv_decode_attention for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without the workspace,
 * same kernel, same result bit for bit. It has no counterpart in the reference. The partial records and
 * arrival counters live in a device array inside the library, 4.3 MB on every GPU the library runs on,
 * held until the process ends. Limits: q_heads <= 128 (more is an error that names the limit; head_dim and
 * t_max as for llmq_kv_decode_attention). Calls no hipMalloc / hipFree and no allocating routine. Every
 * call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams) race; calls on one
 * stream, and calls on different GPUs, are fine. Each call clears the counters first with a one-workgroup
 * fill kernel (not a memset node, so the call can be captured). The FIRST call on a device looks the array's
 * address up (hipGetDevice, hipGetSymbolAddress: they may load the code object) and must be made outside
 * stream capture; every later call on that device launches two kernels and nothing else. */
int llmq_kv_decode_attention_static(const void* q, const void* k_codes, const void* v_codes,
                                    const float* k_scale, const float* v_scale, void* out,
                                    const int32_t* len_dev, float sm_scale, int q_heads, int kv_heads,
                                    int head_dim, int t_max, int bits, int dtype, llmq_stream_t stream);

/* One decode step of attention for one layer in a single launch: RoPE on the new token's query
 * and key (transformers' apply_rotary_pos_emb, same rounding points), quantize-and-append of its
 * key and value at position *pos_dev, then attention over tokens 0 .. *pos_dev. Equivalent to
 * RoPE in PyTorch + llmq_kv_append + llmq_kv_decode_attention; no counterpart in the reference.
 * qkv: [(q_heads + 2*kv_heads) * head_dim] `dtype`, query heads first, then key heads, then value
 * heads (the concatenated outputs of q_proj, k_proj, v_proj). cos_table / sin_table:
 * [positions, head_dim] `dtype` as LlamaRotaryEmbedding produces them. out: [q_heads * head_dim].
 * One workgroup per query head, no workspace; meant for contexts up to a few thousand tokens. */
int llmq_kv_rope_append_attend(const void* qkv, const void* cos_table, const void* sin_table,
                               void* k_codes, void* v_codes, float* k_scale, float* v_scale, void* out,
                               const int32_t* pos_dev, float sm_scale, int q_heads, int kv_heads,
                               int head_dim, int t_max, int bits, int dtype, llmq_stream_t stream);

/* The same decode step with the tokens of every head spread over n_splits workgroups (256 CUs are
 * filled by 32 heads x 8 splits; one workgroup per head leaves 7/8 of the chip idle and is bound by
 * the dequantization arithmetic). Instead of the attention output it writes, per (head, split), a
 * record [max, sum, 0, 0, weighted output[head_dim]] of fp32 (scores in log2 units) into
 * `partials`, llmq_kv_attend_partials_floats(...) floats, 16-byte aligned. The records are merged
 * by llmq_kv_attend_merge (out: [q_heads * head_dim] `dtype`), or for free by the GEMV that
 * consumes the attention output: llmq_wq_gemv_attn_merge is llmq_wq_gemv_fused whose activation is
 * dtype(merge(partials)) (o_proj of a decoder layer; in_head_dim / residual as there).
 * With n_splits >= 32 (or >= 8 and t_max >= 2048; heads of 128: >= 8 at any t_max) and q_heads / kv_heads a multiple of 4 a workgroup takes four query heads of
 * a kv head together, so every cache row is read and dequantized once for the four (long caches:
 * the step is bound by that arithmetic); the records and their layout are the same. When in
 * addition t_max >= 2048 (heads of 128: at any t_max), the four heads' scores and weighted values are computed on the int8 matrix
 * core with the cache's codes as operands (the query in three base-256 digits, the softmax weights
 * times the value scales in two): exact integer sums of code * scale, without the rounding of the
 * dequantized K and V to `dtype` that the other forms make as the reference's cache does; the
 * output agrees with them to ~1e-3 relative.
 * bits == 16 (this entry point only; dtype fp16 / bf16): an UNQUANTIZED cache, k_codes / v_codes holding
 * [kv_heads, t_max, head_dim] values of `dtype` (the rotated key and the value as they are; scales written
 * as 1): the 16-bit baseline's cache under the same step, one query head per workgroup. */
size_t llmq_kv_attend_partials_floats(int q_heads, int head_dim, int n_splits);
int llmq_kv_rope_append_attend_split(const void* qkv, const void* cos_table, const void* sin_table,
                                     void* k_codes, void* v_codes, float* k_scale, float* v_scale,
                                     float* partials, const int32_t* pos_dev, float sm_scale,
                                     int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                                     int n_splits, int dtype, llmq_stream_t stream);
int llmq_kv_attend_merge(const float* partials, void* out, int q_heads, int head_dim, int n_splits,
                         int dtype, llmq_stream_t stream);
int llmq_wq_gemv_attn_merge(const float* partials, int n_splits, int head_dim, const void* qweight,
                            const float* wscale, void* out, int N, int G, int out_group, int wformat,
                            int dtype, int in_head_dim, const void* residual_or_null,
                            llmq_stream_t stream);

/* The same decode-step GEMV over an UNQUANTIZED fp16 / bf16 weight [N, K] (row-major), one activation row:
 *   out[n] = sum_k x'[k] * weight[n, k], fp32 accumulation,
 * with llmq_wq_gemv_fused's RMSNorm prologue and residual epilogue, llmq_wq_gemv_gate_up_silu's store
 * (pair_half > 0: weight is gate rows over up rows, N = 2 * pair_half, out [pair_half] = act(gate) * up) and
 * llmq_wq_gemv_attn_merge's prologue (LLMQ_PRO_ATTN_MERGE: x is the split attention's records, attn_splits per
 * head of attn_head_dim), each with the same rounding points. It has no counterpart among the reference's
 * kernels: it is what lets the 16-bit baseline run through the same five-launch decode step as the quantized
 * model, as the reference times both sides under one runtime (llmquant/eval/verify.py:44-47).
 * K a multiple of 8, at most 28672; pointers 16-byte aligned; dtype LLMQ_F16 or LLMQ_BF16. */
int llmq_dense_gemv_fused(const void* x, const void* weight, void* out, int N, int K, int dtype, int prologue,
                          const void* norm_weight, float eps, const void* residual, int pair_half,
                          int attn_splits, int attn_head_dim, llmq_stream_t stream);

/* Index of the first maximum of a row of n elements, written to *out_index on the device: the
 * greedy sampler of the decode loop (the reference calls logits.argmax(-1),
 * llmquant/runtime/graph_decode.py:131). */
int llmq_argmax_row(const void* x, int n, int64_t* out_index, int dtype, llmq_stream_t stream);
/* The same, plus the bookkeeping the decode loop does after it in three more PyTorch kernels
 * (llmquant/runtime/graph_decode.py:131-140): when non-NULL, *token = the index (next step's input),
 * *step64 += 1 (the position fed to the rotary table) and *step32 += 1 (the cache's write position). */
int llmq_argmax_advance(const void* x, int n, int64_t* out_index, int64_t* token_or_null,
                        int64_t* step64_or_null, int32_t* step32_or_null, int dtype,
                        llmq_stream_t stream);
/* Causal grouped-query attention of a prompt: out[i, h, :] = softmax over j <= i of (scale * q[i, h, :] .
 * k[h / (q_heads / kv_heads), j, :]) times v, what the reference's prompt pass gets from transformers'
 * attention on the rotated queries and the K / V its FakeQuantCache returns (llmquant/quantizers/fake.py:39-55;
 * the reference has no kernel of its own for it). q: [tokens, q_heads, head_dim]; k, v: [kv_heads, tokens,
 * head_dim] (the dequantized cache values, as llmq_rope_kv_append hands them back); out: [tokens, q_heads,
 * head_dim]. float16 or bfloat16, head_dim 64 or 128, 16-byte aligned, scale > 0; fp32 accumulation,
 * probabilities rounded to `dtype` before they meet v. */
int llmq_prefill_attention(const void* q, const void* k, const void* v, void* out, int tokens, int q_heads,
                           int kv_heads, int head_dim, float scale, int dtype, llmq_stream_t stream);

/* llmq_argmax_advance over 32 workgroups instead of one (the workgroup that finishes last picks among the
 * slices' first maxima: the same index), and, when embed_or_null is given, the next step's embedding lookup
 * as well: hidden_out[0 .. hidden_dim) = embed[index * hidden_dim ..], what the reference's loop does with
 * model.embed_tokens on the token it feeds back (llmquant/runtime/graph_decode.py:131-140). `workspace`:
 * llmq_argmax_workspace_bytes() bytes, 16-byte aligned, zero before the first call; every call leaves it
 * ready for the next; calls that share it must not overlap. x must be 16-byte aligned. */
size_t llmq_argmax_workspace_bytes(void);
int llmq_argmax_advance_embed(const void* x, int n, int64_t* out_index, int64_t* token_or_null,
                              int64_t* step64_or_null, int32_t* step32_or_null, const void* embed_or_null,
                              void* hidden_out_or_null, int hidden_dim, void* workspace, int dtype,
                              llmq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMQ_H */
