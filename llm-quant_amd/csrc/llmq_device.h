// Device-side helpers shared by the gfx950 kernels: element conversion with the rounding
// the parity contract fixes (round-to-nearest-even everywhere), 128-bit vector access,
// wave64 reductions, and the host-side error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/llmq.h"

namespace llmq {

constexpr int kWave = 64;
constexpr float kScaleEps = 1e-8f;  // SCALE_EPS, llmquant/core/observers.py:5

struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

// ---- scalar conversions -----------------------------------------------------------------
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(f16_t v) { return static_cast<float>(v.v); }
__device__ __forceinline__ float to_float(bf16_t v) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(v.bits) << 16);
}

// fp32 -> bf16, round-to-nearest-even: gfx950 converts in hardware (v_cvt_pk_bf16_f32, two
// values per instruction), which the compiler selects for these casts.
__device__ __forceinline__ uint16_t bf16_bits_rne(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
__device__ __forceinline__ uint32_t bf16_pair_rne(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
// fp32 -> fp16, round-to-nearest-even (v_cvt_f16_f32). The empty asm keeps the compiler from
// folding a preceding multiply into v_fma_mixlo_f16, which adds +0 and so turns a -0 product
// into +0.
__device__ __forceinline__ _Float16 f16_rne(float f) {
  asm volatile("" : "+v"(f));
  return static_cast<_Float16>(f);
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) { return f16_t{f16_rne(f)}; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bf16_t{bf16_bits_rne(f)};
}

// The value after a round trip through storage type T (what a tensor of that dtype would hold).
template <typename T> __device__ __forceinline__ float round_through(float v);
template <> __device__ __forceinline__ float round_through<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_through<bf16_t>(float v) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(bf16_bits_rne(v)) << 16);
}
template <> __device__ __forceinline__ float round_through<f16_t>(float v) {
  return static_cast<float>(f16_rne(v));
}

// ---- 128-bit access ---------------------------------------------------------------------
struct alignas(16) u32x4 { uint32_t x, y, z, w; };
struct alignas(8) u32x2 { uint32_t x, y; };

__device__ __forceinline__ u32x4 load16(const void* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
__device__ __forceinline__ void store16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }

// A 16-byte packet of T, unpacked to fp32 and back.
template <typename T> struct Pack;
template <> struct Pack<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(u32x4 r, float* f) {
    f[0] = __builtin_bit_cast(float, r.x); f[1] = __builtin_bit_cast(float, r.y);
    f[2] = __builtin_bit_cast(float, r.z); f[3] = __builtin_bit_cast(float, r.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    return u32x4{__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]),
                 __builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3])};
  }
};
template <> struct Pack<bf16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[i] = bf16_pair_rne(f[2 * i], f[2 * i + 1]);
    }
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};
template <> struct Pack<f16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w[i] & 0xffffu)));
      f[2 * i + 1] = static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w[i] >> 16)));
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint16_t lo = __builtin_bit_cast(uint16_t, f16_rne(f[2 * i]));
      const uint16_t hi = __builtin_bit_cast(uint16_t, f16_rne(f[2 * i + 1]));
      w[i] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
    }
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};

// ---- wave64 reductions ------------------------------------------------------------------
// Lane exchanges inside a row of 16 lanes are DPP modifiers on an ordinary ALU instruction (a
// few cycles); __shfl_xor compiles to ds_bpermute, a round trip through the LDS unit of ~100
// cycles, and a butterfly is a chain of them. Rows are combined through v_readlane.
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <-> 7 - i within each 8
constexpr int kDppMirror = 0x140;      // lane i <-> 15 - i within each 16
constexpr int kDppRor4 = 0x124;        // lane i <- lane (i + 4) % 16 of its row of 16
constexpr int kDppRor8 = 0x128;        // lane i <- lane (i + 8) % 16 of its row of 16
template <int CTRL> __device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int CTRL> __device__ __forceinline__ int dpp(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Maximum over each aligned group of WIDTH lanes (a power of two), in every lane of the group.
// The mirror steps pair whole sub-groups that already agree, so after log2(WIDTH) steps all agree.
template <int WIDTH> __device__ __forceinline__ float group_max(float v) {
  if constexpr (WIDTH >= 2) v = fmaxf(v, dpp<kDppXor1>(v));
  if constexpr (WIDTH >= 4) v = fmaxf(v, dpp<kDppXor2>(v));
  if constexpr (WIDTH >= 8) v = fmaxf(v, dpp<kDppHalfMirror>(v));
  if constexpr (WIDTH >= 16) v = fmaxf(v, dpp<kDppMirror>(v));
  if constexpr (WIDTH == 32) {
    const float lo = fmaxf(lane_value(v, 0), lane_value(v, 16)), hi = fmaxf(lane_value(v, 32), lane_value(v, 48));
    v = (threadIdx.x & 32) ? hi : lo;
  }
  if constexpr (WIDTH == 64) {
    v = fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
  }
  return v;
}
// Sum over each row of 16 lanes, in every lane of the row (fixed order).
template <typename V> __device__ __forceinline__ V row16_sum(V v) {
  v += dpp<kDppXor1>(v);
  v += dpp<kDppXor2>(v);
  v += dpp<kDppHalfMirror>(v);
  v += dpp<kDppMirror>(v);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

// ---- the quantizer, one element ------------------------------------------------------------
// compute_scale (llmquant/core/observers.py:94-98): true IEEE division, then the eps floor.
__device__ __forceinline__ float scale_from_amax(float amax, float qmax) {
  return fmaxf(amax / qmax, kScaleEps);
}
// quantize (llmquant/core/quant_ops.py:13-19): divide, round half to even, clamp.
__device__ __forceinline__ float quant_code(float v, float scale, float qmin, float qmax) {
  return fminf(fmaxf(rintf(v / scale), qmin), qmax);
}

// Split attention: the records of one query head, n_splits x [max, sum, 0, 0, weighted output[head_dim]]
// (a four-float header keeps the output 16-byte aligned) with scores in log2 units, merged for the
// eight output elements d0 .. d0+7: sum_s w_s o_s[d] / sum_s w_s l_s, w_s = 2^(m_s - max m). A split
// that saw no token has m = -inf and contributes nothing. Records are read eight at a time with
// all loads issued before any is used (a loop that waits for each record costs a memory round
// trip per split); further batches rescale the running sums like online softmax.
constexpr int kAttnRecordHeader = 4;
struct NoHook {
  __device__ __forceinline__ void operator()() const {}
};
// `after_first_loads` runs once, between the first batch's loads and their first use: the place for
// a caller's own loads that have more slack than these.
template <typename Hook = NoHook>
__device__ __forceinline__ void merge_partials8(const float* rec, int n_splits, int head_dim, int d0, float* f,
                                                Hook after_first_loads = Hook()) {
  const int stride = head_dim + kAttnRecordHeader;
  float mm = -INFINITY, ll = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = 0.0f;
  for (int s0 = 0; s0 < n_splits; s0 += 8) {
    float m_s[8], l_s[8];
    u32x4 lo[8], hi[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float* r = rec + min(s0 + j, n_splits - 1) * stride;  // clamped: loaded, then weighted by zero
      m_s[j] = r[0];
      l_s[j] = r[1];
      lo[j] = load16(r + kAttnRecordHeader + d0);
      hi[j] = load16(r + kAttnRecordHeader + d0 + 4);
    }
    if (s0 == 0) after_first_loads();
    float m_new = mm;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (s0 + j < n_splits) m_new = fmaxf(m_new, m_s[j]);
    }
    const float corr = mm == -INFINITY ? 0.0f : exp2f(mm - m_new);
    ll *= corr;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] *= corr;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float a = (s0 + j < n_splits && m_s[j] != -INFINITY) ? exp2f(m_s[j] - m_new) : 0.0f;
      ll += l_s[j] * a;
      const uint32_t w[8] = {lo[j].x, lo[j].y, lo[j].z, lo[j].w, hi[j].x, hi[j].y, hi[j].z, hi[j].w};
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] += __builtin_bit_cast(float, w[e]) * a;
    }
    mm = m_new;
  }
  const float inv = ll > 0.0f ? 1.0f / ll : 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] *= inv;
}

// ---- codes as 16-bit matrix-core operands without a conversion instruction -------------------------------
// A 4-bit code is stored with a bias of 8 (n = code + 8, 0..15); placed in the mantissa of 16.0 it IS the value
// 16 + n in bf16 (0x4180 | n << 3) and in fp16 (0x4c00 | n << 6), two codes per AND-OR. An 8-bit code with its
// sign bit flipped is b = code + 128 (0..255): fp16 holds 256 + b as 0x5c00 | b << 2 (a byte permute and a
// shift-OR per two codes); bf16 has seven mantissa bits, so there b goes through v_cvt_f32_ubyte, whose upper
// half is the bf16 value. What the matrix core then sums is x (code + kBias); kBias sum x comes out again per
// group (the products are exact in fp32 either way). Operand element order: the eight codes of a 32-bit word of
// int4 (two of int8) as (0, 4, 1, 5, 2, 6, 3, 7): the other operand's 16-byte chunks must be in the same
// order (interleave_halves), which a sum over k does not mind.
__device__ __forceinline__ uint32_t and_or(uint32_t value, uint32_t mask_scalar, uint32_t bits) {
  // (value & mask) | bits in one instruction; the compiler leaves it as two. One operand of a VOP3 may come
  // from a scalar register on this chip, so the mask is scalar and the bits sit in a vector register.
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(value), "s"(mask_scalar), "v"(bits));
  return d;
}
// (x0 x1)(x2 x3)(x4 x5)(x6 x7) -> (x0 x4)(x1 x5)(x2 x6)(x3 x7), 16-bit elements
__device__ __forceinline__ u32x4 interleave_halves(const u32x4 v) {
  u32x4 o;
  o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
  return o;
}
template <typename T, int BITS> struct BiasedCodes;
template <> struct BiasedCodes<bf16_t, 4> {
  static constexpr float kBias = 24.0f;
  static constexpr uint32_t kMagic = 0x41804180u;   // keep it in a vector register: asm volatile("" : "+v"(magic))
  // raw: the lane's codes of a group; step: which eight of them
  static __device__ __forceinline__ u32x4 operand(const uint32_t* raw, int step, uint32_t magic) {
    const uint32_t w = raw[step];
    return u32x4{and_or(w << 3, 0x00780078u, magic), and_or(w >> 1, 0x00780078u, magic),
                 and_or(w >> 5, 0x00780078u, magic), and_or(w >> 9, 0x00780078u, magic)};
  }
};
template <> struct BiasedCodes<f16_t, 4> {
  static constexpr float kBias = 24.0f;
  static constexpr uint32_t kMagic = 0x4c004c00u;
  static __device__ __forceinline__ u32x4 operand(const uint32_t* raw, int step, uint32_t magic) {
    const uint32_t w = raw[step];
    return u32x4{and_or(w << 6, 0x03c003c0u, magic), and_or(w << 2, 0x03c003c0u, magic),
                 and_or(w >> 2, 0x03c003c0u, magic), and_or(w >> 6, 0x03c003c0u, magic)};
  }
};
template <> struct BiasedCodes<bf16_t, 8> {
  static constexpr float kBias = 128.0f;
  static constexpr uint32_t kMagic = 0u;
  static __device__ __forceinline__ u32x4 operand(const uint32_t* raw, int step, uint32_t) {
    const uint32_t w0 = raw[2 * step] ^ 0x80808080u, w1 = raw[2 * step + 1] ^ 0x80808080u;   // codes 0..3, 4..7
    uint32_t out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = static_cast<float>((w0 >> (8 * i)) & 0xffu), hi = static_cast<float>((w1 >> (8 * i)) & 0xffu);
      // integers below 256: the upper half of the float is the bf16 value, exactly
      out[i] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x07060302u);
    }
    return u32x4{out[0], out[1], out[2], out[3]};
  }
};
template <> struct BiasedCodes<f16_t, 8> {
  static constexpr float kBias = 384.0f;
  static constexpr uint32_t kMagic = 0x5c005c00u;
  static __device__ __forceinline__ u32x4 operand(const uint32_t* raw, int step, uint32_t magic) {
    const uint32_t w0 = raw[2 * step] ^ 0x80808080u, w1 = raw[2 * step + 1] ^ 0x80808080u;
    // byte i of w0 into the low half, byte i of w1 into the high half, zeros above each
    return u32x4{(__builtin_amdgcn_perm(w1, w0, 0x0c040c00u) << 2) | magic, (__builtin_amdgcn_perm(w1, w0, 0x0c050c01u) << 2) | magic,
                 (__builtin_amdgcn_perm(w1, w0, 0x0c060c02u) << 2) | magic, (__builtin_amdgcn_perm(w1, w0, 0x0c070c03u) << 2) | magic};
  }
};

}  // namespace llmq

// ---- host-side error plumbing -----------------------------------------------------------------
namespace llmq_host {
void set_error(const char* fmt, ...);
int fail_invalid(const char* fmt, ...);   // records the text, returns hipErrorInvalidValue
int check_launch(const char* what);       // hipGetLastError() -> 0 or the error, text recorded

bool gemv_force_alu();
// The integer GEMM's kernel with its scale epilogue in three (or, one activation scale per token, two)
// vector instructions per output and group instead of real mode's four (wq_gemm_a8.hip).
int gemm_a8_relaxed(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                    const float* bias_or_null, void* out, int M, int N, int G, bool token_scale, int out_group,
                    int wformat, int dtype, hipStream_t stream);
// The exact integer GEMM with a tile's groups computed eight at a time and added in order (wq_gemm_a8_groups.hip).
bool gemm_a8_groups_supported(int M, int N, int G);
// (tiled_a: the activation codes are in operand order, as llmq_quant_act_codes_tiled writes them)
int gemm_a8_groups(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                   const float* bias_or_null, void* out, int M, int N, int G, int out_group, int wformat, int dtype,
                   hipStream_t stream, bool tiled_a = false);
// Matrix-core GEMV (wq_gemv_mfma.hip): whether it can take a problem, and its launch.
bool gemv_mfma_supported(const void* x, const void* qw, const float* ws, int M, int G, int gs,
                         int wformat);
int gemv_mfma_launch(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                     int out_group, int wformat, int dtype, hipStream_t stream);
int gemv_mfma_launch_fused(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                           int out_group, int wformat, int dtype, int prologue, const void* norm_weight,
                           float eps, int in_head_dim, const void* residual, hipStream_t stream,
                           int attn_splits = 0, int attn_head_dim = 0, int pair_half = 0);
// Batched form (a plan of expert / row runs read on the device): see llmq_wq_gemv_batched.
bool gemv_batched_mfma_supported(const void* x, const void* qw, const float* ws, int G, int gs, int wformat);
int gemv_batched_mfma_launch(const void* x, const void* qw, const float* ws, void* out, const int32_t* block_expert,
                             const int32_t* block_row0, const int32_t* block_rows, int n_blocks, int n_rows,
                             int n_experts, int N, int G, int out_group, int wformat, int dtype,
                             hipStream_t stream, int64_t x_row_stride = -1, int pair_half = 0);
}  // namespace llmq_host
