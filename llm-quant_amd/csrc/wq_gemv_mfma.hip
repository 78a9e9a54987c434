// Weight-only quantized GEMV on the int8 matrix core (v_mfma_i32_16x16x64_i8), gfx950.
//
//   out[m, n] = sum_g wscale[sr(n), g] * sum_{k in g} x[m, k] * q[n, g, k]        (group = 128)
//
// Decode reads every weight once and does two flops per code, so the kernel is judged by
// how close it gets to streaming the codes at HBM rate. Converting codes to floats on the
// vector ALU costs 2-3 instructions per code, which at 8 TB/s is more than the ALU has.
// Here the codes go to the matrix core as they are:
//
//   * int8 codes are MFMA operand bytes straight out of the 128-bit load: no conversion.
//   * packed int4: `w & 0x0f0f0f0f` and `(w >> 4) & 0x0f0f0f0f` are the even-k and odd-k
//     codes (+8) as bytes: three ALU instructions per eight codes. The +8 comes back out
//     as -8 * sum_k xdigit[k], a per-group constant that rides in as the MFMA's C operand.
//   * the activation is made an integer once per workgroup: per (row, group) a power-of-two
//     scale 2^-sh brings the group's abs-max into [2^21, 2^22), x*2^sh is rounded to an
//     integer and split into three signed base-256 digits. Scaling by a power of two is
//     exact and a bf16/fp16 element within 2^13 / 2^10 of its group's abs-max is carried
//     without any rounding; smaller ones round at 2^-22 of the abs-max, i.e. at fp32
//     resolution. The integer dot products are exact; the only fp32 roundings left are
//     the per-group scale multiply and the sum over groups.
//
// MFMA mapping. One instruction multiplies a 16 x 64 A tile by a 64 x 16 B tile. B holds
// 16 weight rows (lane l: row l%16, sixteen consecutive code bytes of k-block l/16), so a
// 128-bit load per lane IS the operand and a wave-load covers 16 rows x 64 contiguous
// bytes. A holds the activation digits, row i = 4*digit + m (m < 4 activation rows), read
// from LDS once per workgroup and kept in registers. The int32 result has lane l holding
// weight row l%16 and A rows 4*(l/16)..+3, i.e. lane block q = l/16 owns digit q for
// m = 0..3: digits are recombined by scaling block q with 256^q in fp32.
//
// Work split: a workgroup owns 16 weight rows at a time and all of K; wave w owns groups
// 4w..4w+3 (so K = 2048 -> 4 waves, 8192 -> 16 waves; longer rows: waves that each take
// several such chunks: 5..8 waves). Per row tile a wave issues 8 (int8)
// or 4 (int4) 128-bit loads per lane plus one 128-bit load of its four scales, the next
// tile's loads being issued before the current tile's epilogue. Partial sums meet in LDS.
#include "llmq_device.h"

namespace {

using namespace llmq;

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kGroup = 128;
constexpr int kGW = 4;       // groups per wave
constexpr int kDigits = 3;
constexpr int kTileRows = 16;
constexpr int kPlanePad = 16;

struct MfmaArgs {
  const void* x;
  const uint8_t* qw;
  const float* ws;
  void* out;
  int N, G, out_group;
  int n_tiles;
  int row_bytes;  // bytes of one weight row
  // what happens to x before it is multiplied (M == 1 only) and to y after; see llmq_wq_gemv_fused
  int prologue;              // LLMQ_PRO_*
  const void* norm_weight;   // [K] for LLMQ_PRO_RMSNORM
  float eps;
  int in_head_dim;           // > 0: x is [G * in_head_dim]; group g takes head g, zero-padded to 128
  const void* residual;      // [N] or null: out = residual + y, both rounded like the model dtype
  // > 0: the weight is gate rows [0, pair_half) over up rows [pair_half, 2 * pair_half); a row tile
  // is eight gate rows and the eight up rows that go with them, n_tiles = pair_half / 8, and out is
  // [pair_half]: act(gate) * up as the SiLU prologue would compute it from the two outputs
  int pair_half;
  int64_t x_row_stride;      // elements between activation rows; < 0: the rows are packed (the row's width)
  int attn_splits;           // LLMQ_PRO_ATTN_MERGE: x is the split-attention records, this many per head
  int attn_head_dim;         // ... of heads this wide
  int tile_rows;             // 16, or 8: lanes 8..15 of a tile then repeat rows 0..7 (loaded, multiplied, never stored)
};

template <typename T> __device__ __forceinline__ void load8(const T* p, float* f) {
  if constexpr (Pack<T>::N == 8) {
    Pack<T>::unpack(load16(p), f);
  } else {
    Pack<T>::unpack(load16(p), f);
    Pack<T>::unpack(load16(p + 4), f + 4);
  }
}

// LDS carve-up, shared by host (size) and device (offsets).
struct LdsLayout {
  int plane;     // bytes of one digit plane of one activation row
  int dig_off, red_off, cx_off, csum_off, part_off, total;
  __host__ __device__ LdsLayout(int M, int G, int wk, bool need_csum) {
    plane = G * kGroup + kPlanePad;
    dig_off = 0;
    red_off = (kDigits * M * plane + 15) & ~15;
    cx_off = red_off + 64;
    csum_off = cx_off + M * G * 4;
    part_off = csum_off + (need_csum ? kDigits * M * G * 4 : 0);
    part_off = (part_off + 15) & ~15;
    total = part_off + 2 * wk * kDigits * M * kTileRows * 4;
  }
};

template <typename T>
__device__ __forceinline__ T finish(float total, const void* residual, int64_t n) {
  if (residual == nullptr) return from_float<T>(total);
  // hidden = residual + linear(x): the Linear's output is rounded to the model dtype first
  return from_float<T>(to_float(static_cast<const T*>(residual)[n]) + round_through<T>(total));
}

// Weight row that lane j (0..15) of a row tile multiplies; rows past the end are clamped (loaded,
// never stored).
__device__ __forceinline__ int tile_row(const MfmaArgs& a, int tile, int j) {
  if (a.pair_half > 0) return tile * 8 + (j & 7) + (j >= 8 ? a.pair_half : 0);
  return min(tile * a.tile_rows + (j & (a.tile_rows - 1)), a.N - 1);
}

// Stores row j's result of a tile. Every lane of a 16-lane row must call it (the paired form moves
// data between lanes); `owner` marks the lanes whose `total` is the finished sum.
template <typename T>
__device__ __forceinline__ void store_row(const MfmaArgs& a, T* __restrict__ out, int tile, int j, float total,
                                          bool owner) {
  if (a.pair_half > 0) {
    const float up = dpp<kDppRor8>(total);  // lane j < 8 <- lane j + 8: the up row of gate row j
    if (owner && j < 8) {
      // exactly the SiLU prologue on the two rounded outputs
      const float g = round_through<T>(total), u = round_through<T>(up);
      const float silu = g / (1.0f + expf(-g));
      out[tile * 8 + j] = from_float<T>(round_through<T>(silu) * u);
    }
    return;
  }
  const int n = tile * a.tile_rows + j;
  if (owner && j < a.tile_rows && n < a.N) out[n] = finish<T>(total, a.residual, n);
}

struct Prologue {
  int kind;
  const void* norm_weight;
  float eps;
  int in_head_dim;
  int attn_splits = 0;
  int attn_head_dim = 0;
  int64_t x_row_stride = -1;  // elements between rows of x; < 0: packed
};

// The activation as integers, whole workgroup, into LDS: per (row m, group g) the digits of
// rint(x * 2^sh) in three planes laid out so a lane's MFMA operand is 16 contiguous bytes,
// the group's 2^-sh in cxs[m*G + g] and (int4 only) the digit sums in csum[(q*M + m)*G + g].
// Every thread of the block must call it; the caller synchronises afterwards.
// Only rows m < m_valid are staged; what LDS holds for the others is left as it was, which is
// harmless because the caller never stores their results (integer products cannot trap).
// MERGE compiles in the split-attention merge (LLMQ_PRO_ATTN_MERGE); it needs ~80 more registers
// while staging, so only the kernels launched for that prologue carry it.
// How the activation is cut into items of 8 elements, 16 consecutive ones to a group. Heads of at
// most 64 values under int8 weights: the group's upper half is padding that the multiply skips, so
// 8 items cover a group.
template <bool HALF> struct StageGeometry {
  int real_per_group, lg, items, k_real;
  int64_t row_stride;
  __device__ __forceinline__ StageGeometry(int G, const Prologue& pro, int m_valid) {
    real_per_group = pro.in_head_dim > 0 ? pro.in_head_dim : kGroup;
    lg = HALF ? 3 : 4;
    items = (m_valid * G) << lg;
    k_real = G * real_per_group;
    row_stride = pro.x_row_stride >= 0 ? pro.x_row_stride : k_real;
  }
};
template <int M> struct StageItem {
  bool active, real;
  int tq, mg, m, g;
  int64_t src;  // first of the item's 8 elements in x
  template <bool HALF>
  __device__ __forceinline__ StageItem(const StageGeometry<HALF>& geo, int item, int G, int m_valid) {
    active = item < geo.items;
    tq = item & ((1 << geo.lg) - 1);
    mg = active ? item >> geo.lg : 0;  // m * G + g
    m = M == 1 ? 0 : mg / G;
    g = mg - m * G;
    // beyond real_per_group: the zero padding of a head group
    real = active && tq * 8 < geo.real_per_group && m < m_valid;
    src = m * geo.row_stride + g * geo.real_per_group + tq * 8;
  }
};

// What a thread's first item reads from memory, requested at the very top of a kernel: the
// activation heads the kernel's longest dependency chain (load -> digits -> LDS -> barrier ->
// operand fragments -> multiply), while the weight loads that are issued next have slack.
struct StageFirst {
  float x[8];  // the item's elements (the gate half under LLMQ_PRO_SILU_MUL)
  float w[8];  // RMSNorm weights, or the up half
};
template <typename T, int M, bool HALF = false>
__device__ __forceinline__ StageFirst stage_first(const T* __restrict__ x, const int G, const Prologue& pro,
                                                  const int m_valid = M) {
  StageFirst r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r.x[e] = r.w[e] = 0.0f;
  if (pro.kind == LLMQ_PRO_ATTN_MERGE) return r;  // its records are read where they are merged
  const StageGeometry<HALF> geo(G, pro, m_valid);
  const StageItem<M> it(geo, threadIdx.x, G, m_valid);
  if (it.real) {
    load8<T>(x + it.src, r.x);
    if (pro.kind == LLMQ_PRO_RMSNORM) load8<T>(static_cast<const T*>(pro.norm_weight) + it.src, r.w);
    if (pro.kind == LLMQ_PRO_SILU_MUL) load8<T>(x + geo.k_real + it.src, r.w);
  }
  return r;
}

// `after_first_loads`: called by every thread once, as soon as its first item's loads from memory
// are requested when those are requested here (the merge prologue), else at the top.
template <typename T, int BITS, int M, bool MERGE = false, bool HALF = false, typename Hook = NoHook>
__device__ __forceinline__ void stage_activation(const T* __restrict__ x, const int G, const LdsLayout& L,
                                                 int8_t* dig, float* cxs, int* csum, const Prologue pro,
                                                 float* red, const StageFirst& first, const int m_valid = M,
                                                 Hook after_first_loads = Hook()) {
  const int tid = threadIdx.x;
  static_assert(!HALF || BITS == 8, "only int8 rows have a whole multiply step of padding per group");
  const StageGeometry<HALF> geo(G, pro, m_valid);
  const int items = geo.items, k_real = geo.k_real;

  bool hook_pending = true;
  if (!(MERGE && pro.kind == LLMQ_PRO_ATTN_MERGE)) {
    after_first_loads();
    hook_pending = false;
  }
  // RMSNorm (transformers' LlamaRMSNorm.forward): variance of the whole row in fp32 first
  // (a prologue excludes head padding and M > 1, so item i covers elements 8i .. 8i+7 of the row)
  float inv_rms = 0.0f;
  if (pro.kind == LLMQ_PRO_RMSNORM) {
    float ss = 0.0f;
    if (tid * 8 < k_real) {
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(first.x[e], first.x[e], ss);
    }
    for (int i = (tid + blockDim.x) * 8; i < k_real; i += blockDim.x * 8) {
      float f[8];
      load8<T>(x + i, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
    }
    ss = wave_sum(ss);
    if ((tid & (kWave - 1)) == 0) red[tid / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < static_cast<int>(blockDim.x) / kWave; ++w) total += red[w];
    inv_rms = rsqrtf(total / static_cast<float>(k_real) + pro.eps);
  }

  for (int base = 0; base < items; base += blockDim.x) {
    const StageItem<M> it(geo, base + tid, G, m_valid);
    const bool active = it.active;
    const int tq = it.tq, mg = it.mg, m = it.m, g = it.g;
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = 0.0f;
    if (it.real) {
      const int64_t src = it.src;
      bool merged = false;
      if constexpr (MERGE) {
        if (pro.kind == LLMQ_PRO_ATTN_MERGE) {
          // x holds the partial records of split attention; elements src .. src+7 lie in one head
          const int hd = pro.attn_head_dim;
          const int head = static_cast<int>(src) / hd, d0 = static_cast<int>(src) - head * hd;
          const bool fire = hook_pending;
          hook_pending = false;
          merge_partials8(reinterpret_cast<const float*>(x) +
                              static_cast<int64_t>(head) * pro.attn_splits * (hd + kAttnRecordHeader),
                          pro.attn_splits, hd, d0, f, [&] {
                            if (fire) after_first_loads();
                          });
#pragma unroll
          for (int e = 0; e < 8; ++e) f[e] = round_through<T>(f[e]);
          merged = true;
        }
      }
      if (merged) {
      } else if (base == 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = first.x[e];
      } else {
        load8<T>(x + src, f);
      }
      if (pro.kind == LLMQ_PRO_RMSNORM) {
        float w[8];
        if (base == 0) {
#pragma unroll
          for (int e = 0; e < 8; ++e) w[e] = first.w[e];
        } else {
          load8<T>(static_cast<const T*>(pro.norm_weight) + src, w);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = round_through<T>(w[e] * round_through<T>(f[e] * inv_rms));
      } else if (pro.kind == LLMQ_PRO_SILU_MUL) {
        // x holds gate then up: act_fn(gate) * up with both results rounded to the model dtype
        float up[8];
        if (base == 0) {
#pragma unroll
          for (int e = 0; e < 8; ++e) up[e] = first.w[e];
        } else {
          load8<T>(x + k_real + src, up);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float silu = f[e] / (1.0f + expf(-f[e]));
          f[e] = round_through<T>(round_through<T>(silu) * up[e]);
        }
      }
    }
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(f[e]));
    amax = group_max<8>(amax);
    if constexpr (!HALF) amax = fmaxf(amax, dpp<kDppMirror>(amax));
    const int ebits = static_cast<int>((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xffu);
    const int sh = 148 - ebits;  // amax * 2^sh in [2^21, 2^22)
    // xi = x * 2^sh as an integer of three signed base-256 digits d0 + 256 d1 + 65536 d2. With
    // t1 = (xi + 128) >> 8 and t2 = (t1 + 128) >> 8 the digits are the low bytes of xi, t1, t2, and
    // t2 = (xi + 128 + 32768) >> 16: d0 is byte 0 of xi, d1 byte 1 of xi + 0x80, d2 byte 2 of
    // xi + 0x8080. (A group of zeros gives xi = 0 without a special case.)
    uint32_t y[kDigits][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t xi = static_cast<uint32_t>(static_cast<int>(rintf(ldexpf(f[e], sh))));
      y[0][e] = xi;
      y[1][e] = xi + 0x80u;
      y[2][e] = xi + 0x8080u;
    }
    // int8: bytes in element order. int4: even elements first (they meet the low nibbles), odd
    // elements second.
    uint32_t packed[kDigits][2];
    int dsum[kDigits] = {};
#pragma unroll
    for (int q = 0; q < kDigits; ++q) {
      // byte q of each of a, b: -> (a.q, b.q, 0, 0)
      const uint32_t pick = 0x0c0c0000u | (static_cast<uint32_t>(4 + q) << 8) | static_cast<uint32_t>(q);
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int e0 = BITS == 8 ? 4 * h : h, step = BITS == 8 ? 1 : 2;
        const uint32_t lo = __builtin_amdgcn_perm(y[q][e0 + step], y[q][e0], pick);
        const uint32_t hi = __builtin_amdgcn_perm(y[q][e0 + 3 * step], y[q][e0 + 2 * step], pick);
        packed[q][h] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        if constexpr (BITS == 4) dsum[q] = __builtin_amdgcn_sdot4(static_cast<int>(packed[q][h]), 0x01010101, dsum[q], false);
      }
    }
    if (active) {
#pragma unroll
      for (int q = 0; q < kDigits; ++q) {
        int8_t* plane = dig + (q * M + m) * L.plane + g * kGroup;
        if constexpr (BITS == 8) {
          *reinterpret_cast<u32x2*>(plane + tq * 8) = u32x2{packed[q][0], packed[q][1]};
        } else {
          // element k = 32*kb + 2*t + p lives at  p*64 + kb*16 + t
          const int kb = tq >> 2, t0 = (tq & 3) * 4;
          *reinterpret_cast<uint32_t*>(plane + kb * 16 + t0) = packed[q][0];
          *reinterpret_cast<uint32_t*>(plane + 64 + kb * 16 + t0) = packed[q][1];
        }
      }
    }
    if constexpr (BITS == 4) {
#pragma unroll
      for (int q = 0; q < kDigits; ++q) {
        const int s = row16_sum(dsum[q]);
        if (active && tq == 0) csum[(q * M + m) * G + g] = s;
      }
    }
    if (active && tq == 0) cxs[mg] = amax > 0.0f ? ldexpf(1.0f, -sh) : 0.0f;
    if (hook_pending) {  // this thread's first item read nothing
      after_first_loads();
      hook_pending = false;
    }
  }
  if (hook_pending) after_first_loads();
}

// MULTI == false: the workgroup has one wave per chunk of four groups (K <= 8192) and a wave's
// activation fragments stay in registers for the whole kernel. MULTI == true: longer rows; wave w
// takes chunks w, w + waves, ... of every row tile and re-reads the fragments of the chunk it is
// about to multiply from LDS (the read is issued with the weight loads, a chunk ahead).
template <typename T, int BITS, int M, bool MULTI, bool MERGE = false, bool HALF = false>
__device__ __forceinline__ void ksplit_body(const MfmaArgs& a, unsigned char* smem, const int first_tile,
                                            const int tile_stride, const int m_valid) {
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wv = tid / kWave;
  const int wk = blockDim.x / kWave;
  const int G = a.G;
  const int n_chunks = G / kGW;
  const LdsLayout L(M, G, wk, BITS == 4);
  int8_t* dig = reinterpret_cast<int8_t*>(smem + L.dig_off);
  float* cxs = reinterpret_cast<float*>(smem + L.cx_off);
  float* red = reinterpret_cast<float*>(smem + L.red_off);
  int* csum = reinterpret_cast<int*>(smem + L.csum_off);
  float* part = reinterpret_cast<float*>(smem + L.part_off);

  const int j = lane & 15;    // weight row within the tile (B column / D column)
  const int blk = lane >> 4;  // k-block of the operand; digit block of the result

  // HALF: heads of at most 64 values, each padded to a group of its own. The activation's upper
  // half of every group is zero whatever the weights there hold, so an int8 row's second 64 bytes
  // of a group are neither read nor multiplied. (A template parameter: a run-time test here, in
  // the middle of the load sequence, costs the ordinary case a quarter of its bandwidth.)
  static_assert(!HALF || (BITS == 8 && M == 1), "the half-group form is for int8 rows, one activation row");

  // ---- weight / scale loads of one chunk of one row tile ------------------------------------
  constexpr int kLoads = BITS == 8 ? (HALF ? kGW : 2 * kGW) : kGW;
  constexpr int kB = BITS == 8 && !HALF ? 2 : 1;  // operand registers per group
  v4i b[kLoads];
  float sc[kGW];
  auto issue_loads = [&](int tile, int chunk) {
    const int g0 = chunk * kGW;
    const int n = tile_row(a, tile, j);
    const uint8_t* row = a.qw + static_cast<int64_t>(n) * a.row_bytes;
#pragma unroll
    for (int gi = 0; gi < kGW; ++gi) {
      if constexpr (BITS == 8) {
        const uint8_t* p = row + (g0 + gi) * kGroup + blk * 16;
        b[kB * gi] = *reinterpret_cast<const v4i*>(p);
        if constexpr (!HALF) b[kB * gi + 1] = *reinterpret_cast<const v4i*>(p + 64);
      } else {
        b[gi] = *reinterpret_cast<const v4i*>(row + (g0 + gi) * (kGroup / 2) + blk * 16);
      }
    }
    const int srow = a.out_group > 0 ? n / a.out_group : n;
    // G and g0 are multiples of 4: the chunk's four scales are one aligned 128-bit load
    const u32x4 s4 = load16(a.ws + static_cast<int64_t>(srow) * G + g0);
    sc[0] = __builtin_bit_cast(float, s4.x); sc[1] = __builtin_bit_cast(float, s4.y);
    sc[2] = __builtin_bit_cast(float, s4.z); sc[3] = __builtin_bit_cast(float, s4.w);
  };

  // ---- a chunk's activation operands and constants, LDS -> registers ------------------------
  v4i afrag[kGW][2];
  float fscale[kGW][M];  // 2^-sh * 256^digit of the result block this lane sits in
  v4i cinit[kGW];
  auto load_fragments = [&](int chunk) {
    const int q = j >> 2, m = j & 3;  // A row j = 4*digit + m
    const float digit_weight = blk == 0 ? 1.0f : (blk == 1 ? 256.0f : 65536.0f);
#pragma unroll
    for (int gi = 0; gi < kGW; ++gi) {
      const int g = chunk * kGW + gi;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        afrag[gi][s] = v4i{0, 0, 0, 0};
        if (q < kDigits && m < M && !(s == 1 && HALF)) {
          afrag[gi][s] = *reinterpret_cast<const v4i*>(dig + (q * M + m) * L.plane + g * kGroup + s * 64 + blk * 16);
        }
      }
      cinit[gi] = v4i{0, 0, 0, 0};
#pragma unroll
      for (int r = 0; r < M; ++r) {
        fscale[gi][r] = blk < kDigits ? cxs[r * G + g] * digit_weight : 0.0f;
        if constexpr (BITS == 4) {
          if (blk < kDigits) cinit[gi][r] = -8 * csum[(blk * M + r) * G + g];
        }
      }
    }
  };

  const Prologue pro{a.prologue, a.norm_weight, a.eps, a.in_head_dim, a.attn_splits, a.attn_head_dim,
                     a.x_row_stride};
  const StageFirst first = stage_first<T, M, HALF>(static_cast<const T*>(a.x), G, pro, m_valid);
  // the first tile's weights: in flight while the activation is prepared, requested right after the
  // activation's own first loads
  int tile = first_tile;
  stage_activation<T, BITS, M, MERGE, HALF>(static_cast<const T*>(a.x), G, L, dig, cxs, csum, pro, red, first,
                                            m_valid, [&] {
                                              if (tile < a.n_tiles) issue_loads(tile, wv);
                                            });
  __syncthreads();
  load_fragments(wv);

  // ---- stream row tiles -----------------------------------------------------------------------
  T* __restrict__ out = static_cast<T*>(a.out);
  int buf = 0;
  for (; tile < a.n_tiles; tile += tile_stride) {
    float acc[M];
#pragma unroll
    for (int r = 0; r < M; ++r) acc[r] = 0.0f;
    for (int chunk = wv; chunk < n_chunks; chunk += wk) {
      v4i d[kGW];
#pragma unroll
      for (int gi = 0; gi < kGW; ++gi) {
        d[gi] = cinit[gi];
        if constexpr (BITS == 8) {
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[gi][0], b[kB * gi], d[gi], 0, 0, 0);
          if constexpr (!HALF) {
            d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[gi][1], b[kB * gi + 1], d[gi], 0, 0, 0);
          }
        } else {
          const v4i lo = b[gi] & 0x0f0f0f0f;
          const v4i hi = (b[gi] >> 4) & 0x0f0f0f0f;
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[gi][0], lo, d[gi], 0, 0, 0);
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[gi][1], hi, d[gi], 0, 0, 0);
        }
      }
      float s_now[kGW][M];
#pragma unroll
      for (int gi = 0; gi < kGW; ++gi)
#pragma unroll
        for (int r = 0; r < M; ++r) s_now[gi][r] = sc[gi] * fscale[gi][r];
      // operand registers are free: refill them with what this wave multiplies next
      const int next_chunk = MULTI ? chunk + wk : n_chunks;
      if (next_chunk < n_chunks) {
        issue_loads(tile, next_chunk);
        load_fragments(next_chunk);
      } else if (tile + tile_stride < a.n_tiles) {
        issue_loads(tile + tile_stride, wv);
        if constexpr (MULTI) load_fragments(wv);
      }
#pragma unroll
      for (int gi = 0; gi < kGW; ++gi) {
#pragma unroll
        for (int r = 0; r < M; ++r) acc[r] = fmaf(static_cast<float>(d[gi][r]), s_now[gi][r], acc[r]);
      }
      if constexpr (!MULTI) break;
    }
    float* pbuf = part + buf * wk * kDigits * M * kTileRows;
    if (blk < kDigits) {
#pragma unroll
      for (int r = 0; r < M; ++r) pbuf[((wv * kDigits + blk) * M + r) * kTileRows + j] = acc[r];
    }
    __syncthreads();
    if (wv == 0) {
      // lane = (wave subset ws, row jj): sums partials of waves ws, ws+4, ... in fixed order,
      // then the four subsets meet through two shuffles
      const int ws = lane >> 4, jj = lane & 15;
#pragma unroll
      for (int r = 0; r < M; ++r) {
        float total = 0.0f;
        for (int w = ws; w < wk; w += 4) {
#pragma unroll
          for (int q = kDigits - 1; q >= 0; --q) total += pbuf[((w * kDigits + q) * M + r) * kTileRows + jj];
        }
        total += __shfl_xor(total, 16, kWave);
        total += __shfl_xor(total, 32, kWave);
        if constexpr (M == 1) {
          store_row<T>(a, out, tile, jj, total, ws == 0);
        } else if (a.pair_half > 0) {
          // row r of several, gate|up pairs: see store_row
          const float up = dpp<kDppRor8>(total);
          if (ws == 0 && jj < 8 && r < m_valid) {
            const float gv = round_through<T>(total), uv = round_through<T>(up);
            const float silu = gv / (1.0f + expf(-gv));
            out[static_cast<int64_t>(r) * a.pair_half + tile * 8 + jj] = from_float<T>(round_through<T>(silu) * uv);
          }
        } else {
          const int n = tile * kTileRows + jj;
          if (ws == 0 && n < a.N && r < m_valid) {
            out[static_cast<int64_t>(r) * a.N + n] = finish<T>(total, a.residual, n);
          }
        }
      }
    }
    buf ^= 1;
  }
}

template <typename T, int BITS, int M, int MAXT, bool MULTI, bool MERGE = false, bool HALF = false>
__global__ __launch_bounds__(MAXT) void wq_gemv_mfma_kernel(const MfmaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  ksplit_body<T, BITS, M, MULTI, MERGE, HALF>(a, smem, blockIdx.x, gridDim.x, M);
}

// Many small GEMVs in one launch (the routed experts of a Mixture-of-Experts layer). Plan entry
// b = blockIdx.y names an expert's weight and a run of consecutive activation rows (a run never
// spans two experts); an entry with no rows costs a workgroup one load and an exit. Runs of up
// to kBatchedMaxRows rows are taken four at a time; a row's arithmetic is the single-launch
// kernel's, so its result does not depend on what it is batched with.
struct BatchPlan {
  const int32_t* expert;
  const int32_t* row0;
  const int32_t* rows;
  int n_experts, n_rows, n_blocks;
  int64_t weight_stride;  // bytes between experts' weights
  int64_t scale_stride;   // floats between experts' scales
};
constexpr int kBatchedMaxRows = 8;

template <typename T, int BITS, int MAXT, bool MULTI>
__global__ __launch_bounds__(MAXT) void wq_gemv_mfma_batched_kernel(MfmaArgs a, const BatchPlan plan) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // blockIdx.y counts the entries that hold rows, not the entries: with 8 of 64 experts routed, a
  // grid over all entries is seven eighths workgroups that start only to exit. Each wave finds the
  // entry for itself: 64 entries per step, one load, a ballot and a count.
  int b = -1;
  {
    const int lane = threadIdx.x & (kWave - 1);
    int seen = 0;
    for (int base = 0; base < plan.n_blocks; base += kWave) {
      const int idx = base + lane;
      const int r = idx < plan.n_blocks ? plan.rows[idx] : 0;
      unsigned long long mask = __ballot(r > 0);
      const int cnt = __popcll(mask);
      if (static_cast<int>(blockIdx.y) < seen + cnt) {
        for (int skip = static_cast<int>(blockIdx.y) - seen; skip > 0; --skip) mask &= mask - 1;
        b = base + __ffsll(static_cast<long long>(mask)) - 1;
        break;
      }
      seen += cnt;
    }
  }
  if (b < 0) return;  // fewer entries hold rows than the grid allows for
  const int rows = min(plan.rows[b], kBatchedMaxRows);
  if (rows <= 0) return;
  const int e = plan.expert[b], row0 = plan.row0[b];
  if (e < 0 || e >= plan.n_experts || row0 < 0 || row0 + rows > plan.n_rows) return;  // not a valid run
  a.qw += e * plan.weight_stride;
  a.ws += e * plan.scale_stride;
  const int64_t x_stride = a.x_row_stride >= 0 ? a.x_row_stride : static_cast<int64_t>(a.G) * kGroup;
  const int64_t out_stride = a.pair_half > 0 ? a.pair_half : a.N;
  const T* x = static_cast<const T*>(a.x);
  T* out = static_cast<T*>(a.out);
  if (rows == 1) {
    // the decode case (one token: every routed expert has one row): the single-row body, which
    // stages a quarter of the fragments and accumulators of the four-row one
    a.x = x + row0 * x_stride;
    a.out = out + row0 * out_stride;
    ksplit_body<T, BITS, 1, MULTI>(a, smem, blockIdx.x, gridDim.x, 1);
    return;
  }
  for (int done = 0; done < rows; done += 4) {
    if (done > 0) __syncthreads();  // the previous pass is done with the LDS
    a.x = x + (row0 + done) * x_stride;
    a.out = out + (row0 + done) * out_stride;
    ksplit_body<T, BITS, 4, MULTI>(a, smem, blockIdx.x, gridDim.x, min(4, rows - done));
  }
}

// Large N: a wave owns whole rows. With every group of the row in one wave there is nothing
// to exchange between waves, so after the activation is staged the main loop has no barrier:
// per chunk of four groups a wave issues its weight loads together with the LDS reads of the
// matching activation fragments (LDS bandwidth is an order of magnitude above what this
// needs), runs the MFMAs, refills the operand registers for the next chunk and only then does
// the scaled accumulate. Two shuffles bring the three digit blocks together at the end of
// a row tile, and 16 lanes store 16 results. One activation row only.
template <typename T, int BITS>
__global__ __launch_bounds__(256, 4) void wq_gemv_mfma_fullk_kernel(const MfmaArgs a) {
  constexpr int M = 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wv = tid / kWave;
  const int waves = blockDim.x / kWave;
  const int G = a.G;
  const LdsLayout L(M, G, 0, BITS == 4);
  int8_t* dig = reinterpret_cast<int8_t*>(smem + L.dig_off);
  float* cxs = reinterpret_cast<float*>(smem + L.cx_off);
  float* red = reinterpret_cast<float*>(smem + L.red_off);
  int* csum = reinterpret_cast<int*>(smem + L.csum_off);
  const int j = lane & 15;
  const int blk = lane >> 4;
  const int n_chunks = (G + kGW - 1) / kGW;

  constexpr int kLoads = BITS == 8 ? 2 * kGW : kGW;
  v4i b[kLoads];
  v4i af[kGW][2];
  float sc[kGW];
  float fs[kGW];   // 2^-sh of the chunk's groups, times this lane block's digit weight
  int bias[kGW];   // -8 * digit sum of the chunk's groups (int4)
  // A row j = 4*digit + m. Only the m == 0 rows of digits 0..2 carry data; what the other
  // rows hold is irrelevant, because their products land in result rows that are never read
  // (m != 0) or are weighted by zero (digit 3). So every lane loads from a valid plane and
  // no lane is masked.
  const int8_t* a_base = dig + min(j >> 2, kDigits - 1) * L.plane + blk * 16;
  const float digit_weight = blk == 0 ? 1.0f : (blk == 1 ? 256.0f : (blk == 2 ? 65536.0f : 0.0f));
  const int* csum_row = csum + (blk < kDigits ? blk : 0) * G;
  auto issue_weights = [&](const uint8_t* row, const float* sp, int c) {
#pragma unroll
    for (int gi = 0; gi < kGW; ++gi) {
      const int g = c * kGW + gi;
      if constexpr (BITS == 8) {
        const uint8_t* p = row + g * kGroup + blk * 16;
        b[2 * gi] = *reinterpret_cast<const v4i*>(p);
        b[2 * gi + 1] = *reinterpret_cast<const v4i*>(p + 64);
      } else {
        b[gi] = *reinterpret_cast<const v4i*>(row + g * (kGroup / 2) + blk * 16);
      }
    }
    const u32x4 s4 = load16(sp + c * kGW);
    sc[0] = __builtin_bit_cast(float, s4.x); sc[1] = __builtin_bit_cast(float, s4.y);
    sc[2] = __builtin_bit_cast(float, s4.z); sc[3] = __builtin_bit_cast(float, s4.w);
  };
  auto issue_fragments = [&](int c) {
#pragma unroll
    for (int gi = 0; gi < kGW; ++gi) {
      const int g = c * kGW + gi;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        af[gi][s] = *reinterpret_cast<const v4i*>(a_base + g * kGroup + s * 64);
      }
      fs[gi] = cxs[g] * digit_weight;
      if constexpr (BITS == 4) bias[gi] = -8 * csum_row[g];
    }
  };
  auto row_of = [&](int tile) {
    return a.qw + static_cast<int64_t>(tile_row(a, tile, j)) * a.row_bytes;
  };
  auto scales_of = [&](int tile) {
    const int n = tile_row(a, tile, j);
    return a.ws + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * G;
  };

  const Prologue pro{a.prologue, a.norm_weight, a.eps, a.in_head_dim, a.attn_splits, a.attn_head_dim};
  const StageFirst first = stage_first<T, M>(static_cast<const T*>(a.x), G, pro);
  const int stride = gridDim.x * waves;
  int tile = blockIdx.x * waves + wv;
  if (tile < a.n_tiles) issue_weights(row_of(tile), scales_of(tile), 0);

  stage_activation<T, BITS, M>(static_cast<const T*>(a.x), G, L, dig, cxs, csum, pro, red, first);
  __syncthreads();
  issue_fragments(0);

  T* __restrict__ out = static_cast<T*>(a.out);
  for (; tile < a.n_tiles; tile += stride) {
    const uint8_t* row = row_of(tile);
    const float* sp = scales_of(tile);
    const bool more = tile + stride < a.n_tiles;
    const uint8_t* next_row = more ? row_of(tile + stride) : row;
    const float* next_sp = more ? scales_of(tile + stride) : sp;
    float acc = 0.0f;
    for (int c = 0; c < n_chunks; ++c) {
      v4i d[kGW];
      float s_now[kGW];
#pragma unroll
      for (int gi = 0; gi < kGW; ++gi) {
        d[gi] = v4i{BITS == 4 ? bias[gi] : 0, 0, 0, 0};
        s_now[gi] = sc[gi] * fs[gi];
        if constexpr (BITS == 8) {
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][0], b[2 * gi], d[gi], 0, 0, 0);
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][1], b[2 * gi + 1], d[gi], 0, 0, 0);
        } else {
          const v4i lo = b[gi] & 0x0f0f0f0f;
          const v4i hi = (b[gi] >> 4) & 0x0f0f0f0f;
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][0], lo, d[gi], 0, 0, 0);
          d[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][1], hi, d[gi], 0, 0, 0);
        }
      }
      // operand registers are free again: refill them (next chunk, or the next tile's first
      // chunk; nothing after the last tile: a re-read there would cost 1/n_chunks of a tile of
      // HBM traffic per wave) before the epilogue
      const bool wrap = c + 1 == n_chunks;
      if (!wrap || more) issue_weights(wrap ? next_row : row, wrap ? next_sp : sp, wrap ? 0 : c + 1);
      issue_fragments(wrap ? 0 : c + 1);
#pragma unroll
      for (int gi = 0; gi < kGW; ++gi) acc = fmaf(static_cast<float>(d[gi][0]), s_now[gi], acc);
    }
    // digit blocks 0..2 of the same weight row sit 16 lanes apart
    const float hi = __shfl_down(acc, 32, kWave);
    const float mid = __shfl_down(acc, 16, kWave);
    const float total = (hi + mid) + acc;
    store_row<T>(a, out, tile, j, total, blk == 0);
  }
}

// The same kernel with DEPTH chunks of weights requested ahead instead of one. When a wave has
// only one or two row tiles (N of a few thousand rows) its time is a chain of memory round trips,
// one per chunk; with the whole row in flight at once the chain is one round trip long. DEPTH x 16
// (int4) or DEPTH x 32 (int8) registers hold the operands, so the kernel is built for two waves per
// SIMD rather than four. The row must be a whole number of DEPTH-chunk rounds.
template <typename T, int BITS, int DEPTH>
__global__ __launch_bounds__(256, 2) void wq_gemv_mfma_fullk_deep_kernel(const MfmaArgs a) {
  constexpr int M = 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wv = tid / kWave;
  const int waves = blockDim.x / kWave;
  const int G = a.G;
  const LdsLayout L(M, G, 0, BITS == 4);
  int8_t* dig = reinterpret_cast<int8_t*>(smem + L.dig_off);
  float* cxs = reinterpret_cast<float*>(smem + L.cx_off);
  float* red = reinterpret_cast<float*>(smem + L.red_off);
  int* csum = reinterpret_cast<int*>(smem + L.csum_off);
  const int j = lane & 15;
  const int blk = lane >> 4;
  const int n_chunks = G / kGW;

  constexpr int kLoads = BITS == 8 ? 2 * kGW : kGW;
  v4i b[DEPTH][kLoads];
  float sc[DEPTH][kGW];
  v4i af[kGW][2];
  float fs[kGW];
  int bias[kGW];
  const int8_t* a_base = dig + min(j >> 2, kDigits - 1) * L.plane + blk * 16;
  const float digit_weight = blk == 0 ? 1.0f : (blk == 1 ? 256.0f : (blk == 2 ? 65536.0f : 0.0f));
  const int* csum_row = csum + (blk < kDigits ? blk : 0) * G;
  auto issue_fragments = [&](int c) {
#pragma unroll
    for (int gi = 0; gi < kGW; ++gi) {
      const int g = c * kGW + gi;
#pragma unroll
      for (int s = 0; s < 2; ++s) af[gi][s] = *reinterpret_cast<const v4i*>(a_base + g * kGroup + s * 64);
      fs[gi] = cxs[g] * digit_weight;
      if constexpr (BITS == 4) bias[gi] = -8 * csum_row[g];
    }
  };
  auto row_of = [&](int tile) {
    return a.qw + static_cast<int64_t>(tile_row(a, tile, j)) * a.row_bytes;
  };
  auto scales_of = [&](int tile) {
    const int n = tile_row(a, tile, j);
    return a.ws + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * G;
  };
// slot D of the operand registers <- chunk C of the row at ROW / its scales at SP
#define LLMQ_FILL(D, ROW, SP, C)                                                                   \
  do {                                                                                             \
    _Pragma("unroll") for (int gi = 0; gi < kGW; ++gi) {                                           \
      const int g_ = (C) * kGW + gi;                                                               \
      if constexpr (BITS == 8) {                                                                   \
        const uint8_t* p_ = (ROW) + g_ * kGroup + blk * 16;                                        \
        b[D][2 * gi] = *reinterpret_cast<const v4i*>(p_);                                          \
        b[D][2 * gi + 1] = *reinterpret_cast<const v4i*>(p_ + 64);                                 \
      } else {                                                                                     \
        b[D][gi] = *reinterpret_cast<const v4i*>((ROW) + g_ * (kGroup / 2) + blk * 16);            \
      }                                                                                            \
    }                                                                                              \
    const u32x4 s4_ = load16((SP) + (C) * kGW);                                                    \
    sc[D][0] = __builtin_bit_cast(float, s4_.x); sc[D][1] = __builtin_bit_cast(float, s4_.y);      \
    sc[D][2] = __builtin_bit_cast(float, s4_.z); sc[D][3] = __builtin_bit_cast(float, s4_.w);      \
  } while (0)

  const Prologue pro{a.prologue, a.norm_weight, a.eps, a.in_head_dim, a.attn_splits, a.attn_head_dim};
  const StageFirst first = stage_first<T, M>(static_cast<const T*>(a.x), G, pro);
  const int stride = gridDim.x * waves;
  int tile = blockIdx.x * waves + wv;
  if (tile < a.n_tiles) {
    const uint8_t* row0 = row_of(tile);
    const float* sp0 = scales_of(tile);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) LLMQ_FILL(d, row0, sp0, d);
  }

  stage_activation<T, BITS, M>(static_cast<const T*>(a.x), G, L, dig, cxs, csum, pro, red, first);
  __syncthreads();
  issue_fragments(0);

  T* __restrict__ out = static_cast<T*>(a.out);
  for (; tile < a.n_tiles; tile += stride) {
    const uint8_t* row = row_of(tile);
    const float* sp = scales_of(tile);
    const bool more = tile + stride < a.n_tiles;
    const uint8_t* next_row = more ? row_of(tile + stride) : row;
    const float* next_sp = more ? scales_of(tile + stride) : sp;
    float acc = 0.0f;
    for (int c0 = 0; c0 < n_chunks; c0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int c = c0 + d;
        v4i r[kGW];
        float s_now[kGW];
#pragma unroll
        for (int gi = 0; gi < kGW; ++gi) {
          r[gi] = v4i{BITS == 4 ? bias[gi] : 0, 0, 0, 0};
          s_now[gi] = sc[d][gi] * fs[gi];
          if constexpr (BITS == 8) {
            r[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][0], b[d][2 * gi], r[gi], 0, 0, 0);
            r[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][1], b[d][2 * gi + 1], r[gi], 0, 0, 0);
          } else {
            const v4i lo = b[d][gi] & 0x0f0f0f0f;
            const v4i hi = (b[d][gi] >> 4) & 0x0f0f0f0f;
            r[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][0], lo, r[gi], 0, 0, 0);
            r[gi] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af[gi][1], hi, r[gi], 0, 0, 0);
          }
        }
        // slot d is free: DEPTH chunks ahead in this row, else the start of the next tile's row
        const int ahead = c + DEPTH;
        if (ahead < n_chunks) {
          LLMQ_FILL(d, row, sp, ahead);
        } else if (more) {
          LLMQ_FILL(d, next_row, next_sp, ahead - n_chunks);
        }
        issue_fragments(c + 1 == n_chunks ? 0 : c + 1);
#pragma unroll
        for (int gi = 0; gi < kGW; ++gi) acc = fmaf(static_cast<float>(r[gi][0]), s_now[gi], acc);
      }
    }
    const float hi = __shfl_down(acc, 32, kWave);
    const float mid = __shfl_down(acc, 16, kWave);
    const float total = (hi + mid) + acc;
    store_row<T>(a, out, tile, j, total, blk == 0);
  }
#undef LLMQ_FILL
}

// The whole-row kernel (a wave owns row tiles, no barrier) takes int4 weights of at least this many row tiles and
// bytes of codes; below, the K-split kernel's sixteen waves a CU win. Measured, replayed from a graph, whole-row /
// K-split: K = 2048: 1024 tiles 6.8 / 6.0 us, 3072: 13.5 / 12.4, 4096: 16.5 / 16.8, 8016 (lm_head): 27.4 / 29.9;
// K = 4096: 1024 tiles 11.5 / 9.7, 1536: 15.7 / 13.3, 2048: 16.6 / 18.1, 8016: 50.5 / 60.8; gate|up pairs with the
// RMSNorm in front, as a decode step runs them: 8192 pairs of K = 2048 7.3 / 7.1, 14336 pairs of K = 4096 17.9 / 14.6.
constexpr int kFullKMinTiles = 1024;
constexpr int64_t kFullKMinBytes = 64ll << 20;
constexpr int kLdsDefault = 64 * 1024;   // dynamic LDS a kernel may use without opting in
constexpr int kLdsMax = 160 * 1024;      // LDS of one gfx950 CU

template <typename T, int BITS, int M, int MAXT, bool MULTI, bool MERGE = false, bool HALF = false>
int launch_one(const MfmaArgs& a, int wk, int grid, int lds, hipStream_t stream) {
  auto kernel = wq_gemv_mfma_kernel<T, BITS, M, MAXT, MULTI, MERGE, HALF>;
  if (lds > kLdsDefault) {
    static bool raised = false;  // per instantiation; worst case two threads both set it
    if (!raised) {
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax);
      if (err != hipSuccess) {
        llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));
        return static_cast<int>(err);
      }
      raised = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(wk * kWave), lds, stream, a);
  return llmq_host::check_launch("wq_gemv_mfma_kernel");
}

template <typename T, int BITS, int M>
int launch_m(const MfmaArgs& a, int wk, int grid, int lds, hipStream_t stream) {
  if constexpr (M == 1 && BITS == 8) {
    // heads of at most half a group, each padded to a group of its own (o_proj of a model with
    // 64-wide heads): the variants that skip the padding
    if (a.in_head_dim > 0 && a.in_head_dim <= kGroup / 2 && wk * kGW == a.G) {
      if (a.prologue == LLMQ_PRO_ATTN_MERGE) {
        if (wk <= 4) return launch_one<T, 8, 1, 256, false, true, true>(a, wk, grid, lds, stream);
        if (wk <= 8) return launch_one<T, 8, 1, 512, false, true, true>(a, wk, grid, lds, stream);
        return launch_one<T, 8, 1, 1024, false, true, true>(a, wk, grid, lds, stream);
      }
      if (wk <= 4) return launch_one<T, 8, 1, 256, false, false, true>(a, wk, grid, lds, stream);
      if (wk <= 8) return launch_one<T, 8, 1, 512, false, false, true>(a, wk, grid, lds, stream);
      return launch_one<T, 8, 1, 1024, false, false, true>(a, wk, grid, lds, stream);
    }
  }
  if constexpr (M == 1) {
    if (a.prologue == LLMQ_PRO_ATTN_MERGE) {
      if (wk * kGW < a.G) return launch_one<T, BITS, 1, 512, true, true>(a, wk, grid, lds, stream);
      if (wk <= 4) return launch_one<T, BITS, 1, 256, false, true>(a, wk, grid, lds, stream);
      if (wk <= 8) return launch_one<T, BITS, 1, 512, false, true>(a, wk, grid, lds, stream);
      return launch_one<T, BITS, 1, 1024, false, true>(a, wk, grid, lds, stream);
    }
  }
  if (wk * kGW < a.G) return launch_one<T, BITS, M, 512, true>(a, wk, grid, lds, stream);
  if (wk <= 4) return launch_one<T, BITS, M, 256, false>(a, wk, grid, lds, stream);
  if (wk <= 8) return launch_one<T, BITS, M, 512, false>(a, wk, grid, lds, stream);
  return launch_one<T, BITS, M, 1024, false>(a, wk, grid, lds, stream);
}

// Waves per workgroup for rows of n_chunks chunks: one per chunk up to 16; beyond that (the
// multi-chunk kernel, which needs more registers than a 16-wave workgroup leaves) the largest
// count in 5..8 that divides the chunks evenly, else 8 (the last round is then partly idle).
int waves_for(int n_chunks) {
  if (n_chunks <= 16) return n_chunks;
  for (int w = 8; w >= 5; --w) {
    if (n_chunks % w == 0) return w;
  }
  return 8;
}

struct FusedOps {
  int prologue = LLMQ_PRO_NONE;
  const void* norm_weight = nullptr;
  float eps = 0.0f;
  int in_head_dim = 0;
  const void* residual = nullptr;
  int attn_splits = 0;
  int attn_head_dim = 0;
  int pair_half = 0;
};

template <typename T, int BITS>
int launch_typed(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                 int out_group, const FusedOps& ops, hipStream_t stream) {
  MfmaArgs a{};
  a.x = x; a.qw = static_cast<const uint8_t*>(qw); a.ws = ws; a.out = out;
  a.N = N; a.G = G; a.out_group = out_group;
  a.prologue = ops.prologue; a.norm_weight = ops.norm_weight; a.eps = ops.eps;
  a.in_head_dim = ops.in_head_dim; a.residual = ops.residual;
  a.attn_splits = ops.attn_splits; a.attn_head_dim = ops.attn_head_dim;
  a.pair_half = ops.pair_half;
  a.x_row_stride = -1;
  // (paired: N = 2 * pair_half weight rows, eight gate + eight up rows to a tile, the same count)
  // Rows of 64 groups make sixteen-wave workgroups, one a CU: an output of at most 128 row tiles then leaves half
  // the chip without work. Tiles of eight rows (the other eight lanes of a tile repeat them: same loads, coalesced,
  // same bits, nothing stored) put a workgroup on every CU: 2048 x 8192 int4, config 1's shape, 6.05 -> 5.65 us,
  // int8 7.40 -> 7.26. Shorter rows and larger outputs lose by it (4096 x 4096 int8: 6.4 -> 7.1 us).
  a.tile_rows = kTileRows;
  if (M == 1 && ops.pair_half == 0 && G / kGW == 16 && (N + kTileRows - 1) / kTileRows <= 128) a.tile_rows = 8;
  a.n_tiles = (N + a.tile_rows - 1) / a.tile_rows;
  a.row_bytes = G * kGroup * BITS / 8;
  // measured on lm_head (8016 row tiles): the barrier-free kernel wins for int4 (27.7 vs 30.7 us),
  // the K-split one for int8 (46.6 vs 49.9 us)
  // measured (graph replay): int4 lm_head 28.3 -> 27.2 us, 8B lm_head 55.0 -> 53.0 with four chunks ahead; for int8
  // (two chunks ahead fit) the K-split kernel below stays faster
  constexpr int kDeep = 4;
  // (rows so long that the staged activation exceeds the default LDS limit go to the K-split kernel,
  // whose launch raises the limit)
  const bool fullk_ok = M == 1 && BITS == 4 && a.n_tiles >= kFullKMinTiles &&
                        static_cast<int64_t>(a.n_tiles) * kTileRows * a.row_bytes >= kFullKMinBytes &&
                        a.prologue != LLMQ_PRO_ATTN_MERGE && LdsLayout(1, G, 0, true).part_off <= kLdsDefault;
  if (fullk_ok && (G / kGW) % kDeep == 0) {
    const LdsLayout L(1, G, 0, BITS == 4);
    auto kernel = wq_gemv_mfma_fullk_deep_kernel<T, BITS, kDeep>;
    constexpr int per_cu = 2;
    int grid = 256 * per_cu;
    if (grid * 4 > a.n_tiles) grid = (a.n_tiles + 3) / 4;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), L.part_off, stream, a);
    return llmq_host::check_launch("wq_gemv_mfma_fullk_deep_kernel");
  }
  if (fullk_ok) {
    const LdsLayout L(1, G, 0, BITS == 4);
    auto kernel = wq_gemv_mfma_fullk_kernel<T, BITS>;
    // exactly as many workgroups as are resident at once (the launch bounds hold the kernel to
    // 128 registers: four waves per SIMD, four 256-thread workgroups per CU), so every wave
    // walks the same number of row tiles, give or take one
    constexpr int per_cu = 4;
    int grid = 256 * per_cu;
    if (grid * 4 > a.n_tiles) grid = (a.n_tiles + 3) / 4;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), L.part_off, stream, a);
    return llmq_host::check_launch("wq_gemv_mfma_fullk_kernel");
  }
  const int wk = waves_for(G / kGW);
  const LdsLayout L(M, G, wk, BITS == 4);
  // Resident workgroups: the kernel's ~100 registers allow 16 waves per CU, and the LDS must fit.
  // A workgroup stages the activation once and then walks row tiles, so for mid-sized N the grid
  // is sized to be resident all at once and to give every workgroup the same number of tiles.
  int per_cu = 16 / wk;
  // With the RMSNorm in front (every workgroup reduces the whole activation row before its first multiply) three
  // four-wave workgroups a CU do better than four: the gate|up pairs of a decode step, 1024 row tiles of K = 2048
  // int4, replayed alone: 7.1-7.2 us on 1024 workgroups, 6.95 on 512, 6.75 on 640, 6.35-6.39 on 768, 7.4 on 896; in
  // the step 1865 -> 1905 tok/s. (int8: 8.9 either way; eight-wave workgroups, K = 4096: two a CU stay best.)
  if (ops.prologue == LLMQ_PRO_RMSNORM && wk == 4) per_cu = 3;
  const int by_lds = kLdsMax / L.total;
  if (per_cu > by_lds) per_cu = by_lds;
  if (per_cu < 1) per_cu = 1;
  const int resident = 256 * per_cu;
  int grid;
  if (a.n_tiles >= 4 * resident) {
    // long streams: more workgroups than are resident, so that a CU always has a workgroup staging its activation
    // while the others stream, about two row tiles each (the second one's loads are requested under the first
    // one's multiplies) and at least twice the resident count. Measured on lm_head, 8016 tiles of K = 2048, 1024
    // resident: 51.0 us at 1x, 48.2 at 2x, 45.9 at 4x, 45.5 at 6x, 46.2 at 8x; K = 4096, 512 resident: 93.7 at 2x,
    // 92.4 at 8x; 2048 tiles of K = 4096: 28.2 at 2x, 28.7 at 4x (one tile each), 33.6 at 8x (idle workgroups).
    grid = 2 * resident;
    if (a.n_tiles / 2 > grid) grid = a.n_tiles / 2;
  } else {
    // Every workgroup the same number of tiles -- unless the last round would be at most half full: then all
    // resident slots are used and some workgroups walk one tile more (measured, K = 4096 int8, 2 x 256 slots:
    // 640 tiles 14.4 -> 12.0 us, 768: 15.0 -> 13.5, 1152: 20.1 -> 18.6; 896 and 1408 tiles, last round three
    // quarters full: 15.7 -> 16.2 and 21.4 -> 22.5 the other way).
    const int rounds = (a.n_tiles + resident - 1) / resident;
    const int last_round = a.n_tiles - (rounds - 1) * resident;
    grid = rounds > 1 && 2 * last_round <= resident ? resident : (a.n_tiles + rounds - 1) / rounds;
  }
  switch (M) {
    case 1: return launch_m<T, BITS, 1>(a, wk, grid, L.total, stream);
    case 2: return launch_m<T, BITS, 2>(a, wk, grid, L.total, stream);
    case 3: return launch_m<T, BITS, 3>(a, wk, grid, L.total, stream);
    default: return launch_m<T, BITS, 4>(a, wk, grid, L.total, stream);
  }
}

}  // namespace

namespace llmq_host {

// Whether the matrix-core GEMV can take this problem (else the caller uses the ALU kernel).
bool gemv_mfma_supported(const void* x, const void* qw, const float* ws, int M, int G, int gs,
                         int wformat) {
  if (gs != kGroup || G < kGW || G % kGW || M < 1 || M > 4) return false;
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED) return false;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qw) |
                         reinterpret_cast<uintptr_t>(ws);
  if (bits & 15u) return false;
  return LdsLayout(M, G, waves_for(G / kGW), wformat == LLMQ_W_INT4_PACKED).total <= kLdsMax - 1024;
}

int gemv_mfma_launch(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                     int out_group, int wformat, int dtype, hipStream_t stream) {
  return gemv_mfma_launch_fused(x, qw, ws, out, M, N, G, out_group, wformat, dtype, LLMQ_PRO_NONE, nullptr,
                                0.0f, 0, nullptr, stream);
}

int gemv_mfma_launch_fused(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                           int out_group, int wformat, int dtype, int prologue, const void* norm_weight,
                           float eps, int in_head_dim, const void* residual, hipStream_t stream, int attn_splits,
                           int attn_head_dim, int pair_half) {
  FusedOps ops;
  ops.pair_half = pair_half;
  ops.prologue = prologue; ops.norm_weight = norm_weight; ops.eps = eps;
  ops.in_head_dim = in_head_dim; ops.residual = residual;
  ops.attn_splits = attn_splits; ops.attn_head_dim = attn_head_dim;
#define LLMQ_DISPATCH(T)                                                                          \
  (wformat == LLMQ_W_INT8 ? launch_typed<T, 8>(x, qw, ws, out, M, N, G, out_group, ops, stream)   \
                          : launch_typed<T, 4>(x, qw, ws, out, M, N, G, out_group, ops, stream))
  switch (dtype) {
    case LLMQ_F32: return LLMQ_DISPATCH(float);
    case LLMQ_F16: return LLMQ_DISPATCH(f16_t);
    case LLMQ_BF16: return LLMQ_DISPATCH(bf16_t);
  }
#undef LLMQ_DISPATCH
  return fail_invalid("x must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

namespace {
template <typename T, int BITS>
int launch_batched(const MfmaArgs& a, const BatchPlan& plan, int n_blocks, hipStream_t stream) {
  const int wk = waves_for(a.G / kGW);
  const bool multi = wk * kGW < a.G;
  const LdsLayout L(4, a.G, wk, BITS == 4);
  // about five hundred workgroups (all resident at once at this kernel's register count) over the
  // entries that can hold rows: at most one per row
  const int live = plan.n_rows < n_blocks ? plan.n_rows : n_blocks;
  int gx = 512 / (live > 0 ? live : 1);
  if (gx < 16) gx = 16;
  if (gx > a.n_tiles) gx = a.n_tiles;
  const dim3 grid(gx, live), block(wk * kWave);
#define LLMQ_BATCHED(MAXT, MULTI)                                                                   \
  do {                                                                                              \
    auto kernel = wq_gemv_mfma_batched_kernel<T, BITS, MAXT, MULTI>;                                \
    static bool raised = false; /* per instantiation; worst case two threads both set it */        \
    if (L.total > kLdsDefault && !raised) {                                                         \
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),             \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax); \
      if (err != hipSuccess) {                                                                      \
        set_error("raising the LDS limit failed: %s", hipGetErrorString(err));                      \
        return static_cast<int>(err);                                                               \
      }                                                                                             \
      raised = true;                                                                                \
    }                                                                                               \
    hipLaunchKernelGGL(kernel, grid, block, L.total, stream, a, plan);                              \
  } while (0)
  if (multi) LLMQ_BATCHED(512, true);
  else if (wk <= 4) LLMQ_BATCHED(256, false);
  else if (wk <= 8) LLMQ_BATCHED(512, false);
  else LLMQ_BATCHED(1024, false);
#undef LLMQ_BATCHED
  return check_launch("wq_gemv_mfma_batched_kernel");
}
}  // namespace

// Whether the matrix-core batched GEMV can take the problem: the single-launch kernel's
// conditions for four rows.
bool gemv_batched_mfma_supported(const void* x, const void* qw, const float* ws, int G, int gs, int wformat) {
  return gemv_mfma_supported(x, qw, ws, 4, G, gs, wformat);
}

int gemv_batched_mfma_launch(const void* x, const void* qw, const float* ws, void* out, const int32_t* block_expert,
                             const int32_t* block_row0, const int32_t* block_rows, int n_blocks, int n_rows,
                             int n_experts, int N, int G, int out_group, int wformat, int dtype,
                             hipStream_t stream, int64_t x_row_stride, int pair_half) {
  MfmaArgs a{};
  a.x = x; a.qw = static_cast<const uint8_t*>(qw); a.ws = ws; a.out = out;
  a.N = N; a.G = G; a.out_group = out_group;
  a.x_row_stride = x_row_stride; a.pair_half = pair_half;
  a.tile_rows = kTileRows;
  a.n_tiles = (N + kTileRows - 1) / kTileRows;
  a.row_bytes = G * kGroup * (wformat == LLMQ_W_INT8 ? 8 : 4) / 8;
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  BatchPlan plan{block_expert, block_row0, block_rows, n_experts, n_rows, n_blocks,
                 static_cast<int64_t>(N) * a.row_bytes, scale_rows * G};
#define LLMQ_DISPATCH(T) \
  (wformat == LLMQ_W_INT8 ? launch_batched<T, 8>(a, plan, n_blocks, stream) : launch_batched<T, 4>(a, plan, n_blocks, stream))
  switch (dtype) {
    case LLMQ_F32: return LLMQ_DISPATCH(float);
    case LLMQ_F16: return LLMQ_DISPATCH(f16_t);
    case LLMQ_BF16: return LLMQ_DISPATCH(bf16_t);
  }
#undef LLMQ_DISPATCH
  return fail_invalid("x must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

}  // namespace llmq_host
