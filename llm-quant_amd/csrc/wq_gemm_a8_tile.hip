// Integer prefill GEMM, the fast form: int8 activations (one scale per token and group) times int4 / int8
// group-quantized weights on the int8 matrix core,
//
//   out[m, n] = sum over g of  sx[m, g] * sw[sr(n), g] * (float)(sum_k a[m, g, k] * q[n, g, k])
//
// the A8 branch of RealQuantLinear.forward (llmquant/quantizers/real.py:94-99) with the same exact integer
// group sums but not the same fp32 roundings: there each group contributes ((float)isum * sw) * sx, added to
// the total, four separately rounded operations in group order (llmq_wq_gemm_a8 reproduces exactly that,
// and is bound by those four vector-ALU instructions per output and group); here a group contributes
// fma((float)isum * sw, sx, total), three instructions and one rounding fewer, and the reduction axis may be
// split across workgroups, so results agree with real mode to fp32 rounding (~1e-7), not bit for bit.
//
// Shape: that of the tiled bf16 GEMM (wq_gemm_a16_tile.hip). A workgroup of eight waves, two per SIMD, owns a
// 128 (m) x 256 (n) output tile; a wave owns 64 x 64: 2 x 2 tiles of v_mfma_i32_32x32x32_i8, four k-steps of
// 32 per group, int32 group sums and fp32 totals in vector registers. All operands reach LDS straight from
// global memory (global_load_lds, 1 KB per wave instruction; 16-byte slots XOR-swizzled by row so that the
// operand reads of 16 consecutive rows are conflict-free), three or four stages deep: the activation tile
// [128 rows][128 bytes], the raw codes of the 256 weight rows, the 128 activation scales and the 256 weight
// scales of the group. A lane reads the activation operand of a k-step from LDS (one read feeds two MFMAs)
// and its own column's codes once per group. int4 is unpacked in registers as the stored nibbles n = code + 8
// (one AND for the even codes of a word, a shift and an AND for the odd ones), and the 8 is taken back out by
// starting each group's sum at -8 * (sum of the group's activations) instead of zero: the preparation pass
// writes that number per token and group, and it reaches the matrix core as the C operand of the first
// k-step. Unpacking leaves the even codes of a 32-bit word in one operand register and the odd ones in the
// next, so the activation is prepared once per call (act_prep_i8_kernel) with the bytes of every 8 in the same
// order: a sum does not care about the order of its terms as long as both operands agree.
//
// The kernel is bound by vector-ALU issue, not by the matrix core: folding a group's 64 x 64 sums into the
// totals is 3 instructions per output (convert, two scales) = 12 per MFMA, against the MFMA's 8 issue slots.
//
// Small N: the reduction axis is split across workgroups, fp32 partial tiles in a workspace, added in a fixed
// order (and the bias after them) by a second launch.
#include "llmq_device.h"

namespace {

using namespace llmq;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;
constexpr int kBM = 128, kBN = 256;
constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr int kWaveM = 64, kWaveN = 64;
constexpr int kMT = kWaveM / 32, kNT = kWaveN / 32;
constexpr int kARowBytes = kGroup;                // int8 activation row of one group
constexpr int kATileBytes = kBM * kARowBytes;     // 16 KB
template <int BITS> constexpr int kCodeRowBytes = BITS == 4 ? kGroup / 2 : kGroup;
template <int BITS> constexpr int kCodeTileBytes = kBN * kCodeRowBytes<BITS>;
constexpr int kSxTileBytes = kBM * 4, kSwTileBytes = kBN * 4, kStartTileBytes = kBM * 4;
template <int BITS>
constexpr int kStageBytes = kATileBytes + kCodeTileBytes<BITS> + kSxTileBytes + kSwTileBytes + kStartTileBytes;
template <int BITS> constexpr int kStages = BITS == 4 ? 4 : 3;   // 136 KB / 150 KB of the 160 KB
template <int BITS> constexpr int kLdsBytes = kStages<BITS> * kStageBytes<BITS>;

// ---- activation preparation: rows padded to whole tiles, bytes in operand order -------------------------
// One lane per 16-byte chunk, eight lanes per group. For int4 weights the bytes of each 8 become
// (0 2 4 6 1 3 5 7), and start[m, g] = -8 * sum of the group's 128 activations is written beside them.
__global__ __launch_bounds__(256) void act_prep_i8_kernel(const u32x4* __restrict__ a, u32x4* __restrict__ ap,
                                                          int* __restrict__ start, const int64_t n_chunks,
                                                          const int int4) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const bool live = i < n_chunks;   // (n_chunks is a multiple of 8: the eight lanes of a group live together)
  u32x4 v = live ? a[i] : u32x4{0, 0, 0, 0};
  if (int4) {
    u32x4 o;
    o.x = __builtin_amdgcn_perm(v.y, v.x, 0x06040200u);
    o.y = __builtin_amdgcn_perm(v.y, v.x, 0x07050301u);
    o.z = __builtin_amdgcn_perm(v.w, v.z, 0x06040200u);
    o.w = __builtin_amdgcn_perm(v.w, v.z, 0x07050301u);
    v = o;
    const int ones = 0x01010101;
    int sum = __builtin_amdgcn_sdot4(static_cast<int>(v.x), ones, 0, false);
    sum = __builtin_amdgcn_sdot4(static_cast<int>(v.y), ones, sum, false);
    sum = __builtin_amdgcn_sdot4(static_cast<int>(v.z), ones, sum, false);
    sum = __builtin_amdgcn_sdot4(static_cast<int>(v.w), ones, sum, false);
    sum += __shfl_xor(sum, 1);
    sum += __shfl_xor(sum, 2);
    sum += __shfl_xor(sum, 4);
    if (live && (threadIdx.x & 7) == 0) start[i >> 3] = -8 * sum;
  }
  if (live) ap[i] = v;
}

struct A8Args {
  const uint8_t* ap;   // [M padded to 128, G*128] int8, bytes in operand order
  const int* start;    // [M, G] int4 weights: what each group's integer sum starts at
  const float* sx;     // [M, G], or [M] (one scale per token)
  const uint8_t* qw;   // [N, G, 128] int8 or [N, G, 64] packed int4
  const float* sw;     // [scale_rows, G]
  const float* bias;   // [N] or null (applied here with one split, else by the second launch)
  void* out;           // [M, N]
  float* partial;      // [splits][M][N]
  int M, N, G, out_group;
  int m_tiles, n_tiles, splits, groups_per_split;
};

template <int BITS> __device__ __forceinline__ int code_slot(int row, int c) {
  return BITS == 4 ? c ^ ((row >> 2) & 3) : c ^ ((row >> 1) & 7);
}

// The 16 codes of one k-step of this lane as an int8 operand (int4: the stored nibbles, code + 8).
template <int BITS>
__device__ __forceinline__ v4i code_operand(const u32x4* raw, int step) {
  if constexpr (BITS == 4) {
    const u32x4 q = raw[step >> 1];
    const uint32_t w0 = (step & 1) ? q.z : q.x, w1 = (step & 1) ? q.w : q.y;
    constexpr uint32_t kLow = 0x0f0f0f0fu;
    return v4i{static_cast<int>(w0 & kLow), static_cast<int>((w0 >> 4) & kLow), static_cast<int>(w1 & kLow),
               static_cast<int>((w1 >> 4) & kLow)};
  } else {
    return __builtin_bit_cast(v4i, raw[step]);
  }
}

// TOKEN: one activation scale per token (sx[M]) instead of one per token and group (sx[M, G]): the scale leaves
// the sum over groups, a group's sums are folded in with two instructions per output instead of three, and
// the token's scale is applied once, at the store.
template <typename T, int BITS, bool TOKEN>
__global__ __launch_bounds__(kThreads, 1) void wq_gemm_a8_tile_kernel(const A8Args a) {
  extern __shared__ __attribute__((aligned(256))) uint8_t smem[];

  // consecutive logical tiles (the m-tiles of one n-tile first) on one XCD: the codes come out of its L2
  const int n_work = a.m_tiles * a.n_tiles * a.splits;
  const int per_xcd = (n_work + 7) / 8;
  const int logical = static_cast<int>(blockIdx.x % 8) * per_xcd + static_cast<int>(blockIdx.x / 8);
  if (logical >= n_work) return;
  const int mt = logical % a.m_tiles;
  const int nt = (logical / a.m_tiles) % a.n_tiles;
  const int sp = logical / (a.m_tiles * a.n_tiles);

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int wm = wv & 1, wn = wv >> 1;
  const int lm = lane & 31, lh = lane >> 5;
  const int m0 = mt * kBM, n0 = nt * kBN;
  const int g_begin = sp * a.groups_per_split;
  const int g_end = min(g_begin + a.groups_per_split, a.G);

  // ---- global -> LDS ----------------------------------------------------------------------------------------
  // activation: 2 instructions per wave, 8 rows each; lane = (row, slot), slot p of row r holds chunk
  // p ^ ((r >> 1) & 7)
  constexpr int kAInstr = kATileBytes / 1024 / kWaves;  // 2
  const uint32_t a_row_bytes = static_cast<uint32_t>(a.G) * kARowBytes;
  uint32_t a_off[kAInstr];
#pragma unroll
  for (int i = 0; i < kAInstr; ++i) {
    const int row = (wv * kAInstr + i) * 8 + (lane >> 3);
    a_off[i] = static_cast<uint32_t>(m0 + row) * a_row_bytes + (((lane & 7) ^ ((row >> 1) & 7)) << 4);
  }
  constexpr int kCodeInstr = kCodeTileBytes<BITS> / 1024 / kWaves;  // 2 or 4
  constexpr int kRowsPerInstr = 1024 / kCodeRowBytes<BITS>;
  constexpr int kSlots = kCodeRowBytes<BITS> / 16;
  const uint32_t w_row_bytes = static_cast<uint32_t>(a.G) * kCodeRowBytes<BITS>;
  uint32_t w_off[kCodeInstr];
#pragma unroll
  for (int i = 0; i < kCodeInstr; ++i) {
    const int row = (wv * kCodeInstr + i) * kRowsPerInstr + lane / kSlots;
    w_off[i] = static_cast<uint32_t>(min(n0 + row, a.N - 1)) * w_row_bytes + (code_slot<BITS>(row, lane % kSlots) << 4);
  }
  // scales, one 4-byte value per lane: waves 0, 1 the activation's (64 rows each), waves 2..5 the weight's
  // (64 columns each), waves 6, 7 the rows' group starts (int4; for int8 they repeat the activation scales)
  const float* s_lane;
  int s_at, s_step = 1;
  constexpr int kScalesAt = kATileBytes + kCodeTileBytes<BITS>;
  if (wv < 2 || wv >= 6) {
    const int row = min(m0 + (wv & 1) * 64 + lane, a.M - 1);
    const bool starts = BITS == 4 && wv >= 6;
    if (starts) {
      s_lane = reinterpret_cast<const float*>(a.start) + static_cast<int64_t>(row) * a.G;
    } else if (TOKEN) {
      s_lane = a.sx + row, s_step = 0;   // (the tile is not read: the transfer keeps every wave's count the same)
    } else {
      s_lane = a.sx + static_cast<int64_t>(row) * a.G;
    }
    s_at = kScalesAt + (starts ? kSxTileBytes + kSwTileBytes : 0) + (wv & 1) * 256;
  } else {
    const int n = min(n0 + (wv - 2) * 64 + lane, a.N - 1);
    s_lane = a.sw + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * a.G;
    s_at = kScalesAt + kSxTileBytes + (wv - 2) * 256;
  }
  constexpr int kDmaPerWave = kAInstr + kCodeInstr + 1;

  auto request = [&](int g, int st) {
    uint8_t* stage = smem + st * kStageBytes<BITS>;
    const uint8_t* ag = a.ap + static_cast<uint32_t>(g) * kARowBytes;
#pragma unroll
    for (int i = 0; i < kAInstr; ++i) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(ag + a_off[i]),
                                       reinterpret_cast<u32x4*>(stage + (wv * kAInstr + i) * 1024), 16, 0, 0);
    }
    const uint8_t* wg = a.qw + static_cast<uint32_t>(g) * kCodeRowBytes<BITS>;
#pragma unroll
    for (int i = 0; i < kCodeInstr; ++i) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(wg + w_off[i]),
                                       reinterpret_cast<u32x4*>(stage + kATileBytes + (wv * kCodeInstr + i) * 1024), 16, 0,
                                       0);
    }
    __builtin_amdgcn_global_load_lds(s_lane + g * s_step, reinterpret_cast<float*>(stage + s_at), 4, 0, 0);
  };
  // Wait until at most `younger` of this wave's request batches are still in flight.
  auto wait_requests = [&](int younger) {
    if (younger <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (younger == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDmaPerWave) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDmaPerWave) : "memory");
  };
  static_assert(kStages<BITS> <= 4 && 2 * kDmaPerWave < 64, "wait_requests");

  // ---- LDS -> operands ------------------------------------------------------------------------------------
  // activation operand of k-step j, row tile mi: row wm*64 + mi*32 + lm, chunk 4 lh + j
  uint32_t a_rd[kMT][4];
#pragma unroll
  for (int mi = 0; mi < kMT; ++mi) {
    const int row = wm * 64 + mi * 32 + lm;
#pragma unroll
    for (int j = 0; j < 4; ++j) a_rd[mi][j] = row * kARowBytes + (((4 * lh + j) ^ ((row >> 1) & 7)) << 4);
  }
  // codes: weight row wn*64 + ni*32 + lm, k in [64 lh, 64 lh + 64): chunks lh * kRawLoads + q
  constexpr int kRawLoads = BITS == 4 ? 2 : 4;
  uint32_t c_rd[kNT][kRawLoads];
#pragma unroll
  for (int ni = 0; ni < kNT; ++ni) {
    const int row = wn * kWaveN + ni * 32 + lm;
#pragma unroll
    for (int q = 0; q < kRawLoads; ++q)
      c_rd[ni][q] = kATileBytes + row * kCodeRowBytes<BITS> + (code_slot<BITS>(row, lh * kRawLoads + q) << 4);
  }
  // per-row values of this lane's outputs (rows 8 q + 4 lh + 0..3 of row tile mi): scales, group starts
  const uint32_t row_rd = kScalesAt + (wm * 64 + 4 * lh) * 4;
  const uint32_t sw_rd = kScalesAt + kSxTileBytes + (wn * kWaveN + lm) * 4;
  auto read16 = [&](const uint8_t* stage, uint32_t offset) { return *reinterpret_cast<const u32x4*>(stage + offset); };

  float total[kMT][kNT][16];
#pragma unroll
  for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) total[mi][ni][r] = 0.0f;

  const int n_groups = g_end - g_begin;
#pragma unroll
  for (int st = 0; st < kStages<BITS>; ++st) {
    if (st < n_groups) request(g_begin + st, st);
  }
  wait_requests(min(kStages<BITS>, n_groups) - 1);
  __builtin_amdgcn_s_barrier();

  // The two waves of a SIMD work half a group apart. Between two barriers waves 0..3 multiply the group and
  // then fold its sums into their totals; waves 4..7 first fold the sums of the group before and then
  // multiply: while one wave keeps the matrix core busy the other keeps the vector ALU busy, instead of both
  // queueing for the same unit.
  const int late = __builtin_amdgcn_readfirstlane(wv >> 2);

  v16i acc[kMT][kNT];
  u32x4 sx_now[kMT][4];
  float sw_now[kNT];
  // register r of a 32 x 32 tile is row 8 (r / 4) + 4 lh + r % 4
  auto fold = [&]() {
    if constexpr (TOKEN) {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            total[mi][ni][r] = fmaf(static_cast<float>(acc[mi][ni][r]), sw_now[ni], total[mi][ni][r]);
    } else {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float sx[4] = {__builtin_bit_cast(float, sx_now[mi][q].x), __builtin_bit_cast(float, sx_now[mi][q].y),
                               __builtin_bit_cast(float, sx_now[mi][q].z), __builtin_bit_cast(float, sx_now[mi][q].w)};
#pragma unroll
          for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float d = static_cast<float>(acc[mi][ni][4 * q + i]) * sw_now[ni];
              total[mi][ni][4 * q + i] = fmaf(d, sx[i], total[mi][ni][4 * q + i]);
            }
        }
    }
  };

  int st = 0;
  for (int g = g_begin; g < g_end; ++g) {
    const uint8_t* stage = smem + st * kStageBytes<BITS>;
    if (late && g > g_begin) fold();

    // what a lane holds of the group: its own columns' codes and weight scales, the first activation operand
    u32x4 raw[kNT][kRawLoads], fa[2][kMT];
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
      for (int q = 0; q < kRawLoads; ++q) raw[ni][q] = read16(stage, c_rd[ni][q]);
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi) fa[0][mi] = read16(stage, a_rd[mi][0]);
    v16i begin[kMT];
    if constexpr (BITS == 4) {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const u32x4 b = read16(stage, row_rd + kSxTileBytes + kSwTileBytes + (mi * 32 + 8 * q) * 4);
          begin[mi][4 * q] = static_cast<int>(b.x), begin[mi][4 * q + 1] = static_cast<int>(b.y);
          begin[mi][4 * q + 2] = static_cast<int>(b.z), begin[mi][4 * q + 3] = static_cast<int>(b.w);
        }
    } else {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) begin[mi][r] = 0;
    }
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni) sw_now[ni] = *reinterpret_cast<const float*>(stage + sw_rd + ni * 128);

#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v4i fb[kNT];
#pragma unroll
      for (int ni = 0; ni < kNT; ++ni) fb[ni] = code_operand<BITS>(raw[ni], j);
      if (j < 3) {
#pragma unroll
        for (int mi = 0; mi < kMT; ++mi) fa[(j + 1) & 1][mi] = read16(stage, a_rd[mi][j + 1]);
      } else if constexpr (!TOKEN) {
        // activation scales of this lane's output rows (rows 8 q + 4 lh + 0..3 of each row tile)
#pragma unroll
        for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            sx_now[mi][q] = read16(stage, row_rd + (mi * 32 + 8 * q) * 4);
      }
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni) {
          const v4i av = __builtin_bit_cast(v4i, fa[j & 1][mi]);
          acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, fb[ni], j == 0 ? begin[mi] : acc[mi][ni], 0, 0, 0);
        }
    }
    if (!late) fold();

    // The workgroup meets at the end of the group: every read of this stage has returned, so it can take the
    // group kStages ahead; and each wave's own transfers of the next group have landed (younger batches may
    // stay in flight), so behind the barrier the next group's stage is complete.
    if (g + 1 < g_end) {
      wait_requests(min(kStages<BITS> - 2, g_end - 2 - g));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      if (g + kStages<BITS> < g_end) request(g + kStages<BITS>, st);
    }
    st = st + 1 == kStages<BITS> ? 0 : st + 1;
  }
  if (late) fold();

  // ---- store ------------------------------------------------------------------------------------------------
  if constexpr (TOKEN) {
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sx = a.sx[min(m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3), a.M - 1)];
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni) total[mi][ni][r] *= sx;
      }
  }
  if (a.splits == 1) {
    T* __restrict__ out = static_cast<T*>(a.out);
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni) {
      const int n = n0 + wn * kWaveN + ni * 32 + lm;
      const float b = (a.bias != nullptr && n < a.N) ? a.bias[n] : 0.0f;
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (m < a.M && n < a.N) out[static_cast<int64_t>(m) * a.N + n] = from_float<T>(total[mi][ni][r] + b);
        }
    }
  } else {
    float* __restrict__ part = a.partial + static_cast<int64_t>(sp) * a.M * a.N;
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni) {
      const int n = n0 + wn * kWaveN + ni * 32 + lm;
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * 64 + mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (m < a.M && n < a.N) part[static_cast<int64_t>(m) * a.N + n] = total[mi][ni][r];
        }
    }
  }
}

// out[m, n] = T(partial[0][m, n] + partial[1][m, n] + ... (+ bias[n])), slices in order.
template <typename T>
__global__ __launch_bounds__(256) void add_splits_bias_kernel(const float* __restrict__ partial, const float* __restrict__ bias,
                                                              T* __restrict__ out, const int64_t count, const int N,
                                                              const int splits) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= count) return;
  float s = partial[i];
  for (int k = 1; k < splits; ++k) s = s + partial[k * count + i];
  if (bias != nullptr) s = s + bias[i % N];
  out[i] = from_float<T>(s);
}

constexpr size_t kAlign = 256;
size_t aligned(size_t bytes) { return (bytes + kAlign - 1) / kAlign * kAlign; }

struct Plan {
  int m_tiles, n_tiles, splits, groups_per_split;
  size_t ap_bytes, start_bytes, partial_bytes;
};

Plan plan_for(int M, int N, int G) {
  Plan p{};
  p.m_tiles = (M + kBM - 1) / kBM;
  p.n_tiles = (N + kBN - 1) / kBN;
  const int tiles = p.m_tiles * p.n_tiles;
  int splits = 1;
  if (tiles < 160) {  // too few tiles to occupy the chip: cut the reduction axis, at least four groups a slice
    splits = (256 + tiles - 1) / tiles;
    if (splits > G / 4) splits = G / 4;
    if (splits < 1) splits = 1;
  }
  p.groups_per_split = (G + splits - 1) / splits;
  p.splits = (G + p.groups_per_split - 1) / p.groups_per_split;
  p.ap_bytes = aligned(static_cast<size_t>(p.m_tiles) * kBM * G * kARowBytes);
  p.start_bytes = aligned(static_cast<size_t>(M) * G * sizeof(int));
  p.partial_bytes = p.splits > 1 ? aligned(static_cast<size_t>(p.splits) * M * N * sizeof(float)) : 0;
  return p;
}

template <typename T, int BITS, bool TOKEN>
int launch_tiles(const A8Args& a, dim3 grid, hipStream_t stream) {
  auto kernel = wq_gemm_a8_tile_kernel<T, BITS, TOKEN>;
  static bool raised = false;  // per instantiation; worst case two threads both set it
  if (!raised) {
    const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes<BITS>);
    if (err != hipSuccess) {
      llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));
      return static_cast<int>(err);
    }
    raised = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), kLdsBytes<BITS>, stream, a);
  return llmq_host::check_launch("wq_gemm_a8_tile_kernel");
}

template <typename T>
int run_typed(A8Args& a, const Plan& p, int wformat, bool token, hipStream_t s) {
  const int total = p.m_tiles * p.n_tiles * p.splits;
  const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
  int rc;
  if (wformat == LLMQ_W_INT4_PACKED) rc = token ? launch_tiles<T, 4, true>(a, grid, s) : launch_tiles<T, 4, false>(a, grid, s);
  else rc = token ? launch_tiles<T, 8, true>(a, grid, s) : launch_tiles<T, 8, false>(a, grid, s);
  if (rc) return rc;
  if (p.splits > 1) {
    const int64_t count = static_cast<int64_t>(a.M) * a.N;
    hipLaunchKernelGGL((add_splits_bias_kernel<T>), dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s,
                       a.partial, a.bias, static_cast<T*>(a.out), count, a.N, p.splits);
    return llmq_host::check_launch("add_splits_bias_kernel");
  }
  return 0;
}

}  // namespace

extern "C" size_t llmq_wq_gemm_a8_fast_workspace_bytes(int M, int N, int G) {
  if (M <= 0 || N <= 0 || G <= 0) return 0;
  const Plan p = plan_for(M, N, G);
  return p.ap_bytes + p.start_bytes + p.partial_bytes;
}

extern "C" int llmq_wq_gemm_a8_fast(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                                    const float* bias_or_null, void* out, void* workspace, size_t workspace_bytes,
                                    int M, int N, int G, int sx_groups, int gs, int out_group, int wformat,
                                    int dtype, llmq_stream_t stream) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs != kGroup) return llmq_host::fail_invalid("the integer GEMM needs group_size 128, got %d", gs);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (sx_groups != 1 && sx_groups != G)
    return llmq_host::fail_invalid("activation scales per token must be 1 or G=%d, got %d", G, sx_groups);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("out must be float32, float16 or bfloat16, got dtype code %d", dtype);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!a || !sx || !qweight || !wscale || !out || !workspace) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return llmq_host::fail_invalid("activation, weight and workspace pointers must be 16-byte aligned");
  if ((static_cast<uint64_t>(M) + kBM) * G * kARowBytes >= (1ull << 32) ||
      static_cast<uint64_t>(N) * G * kGroup >= (1ull << 32))
    return llmq_host::fail_invalid("operands of %d x %d and %d x %d are beyond the kernel's 32-bit offsets", M,
                                   G * kGroup, N, G * kGroup);
  const Plan p = plan_for(M, N, G);
  const size_t need = p.ap_bytes + p.start_bytes + p.partial_bytes;
  if (workspace_bytes < need)
    return llmq_host::fail_invalid("workspace of %zu bytes is too small, need %zu", workspace_bytes, need);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  const int64_t n_chunks = static_cast<int64_t>(M) * G * (kARowBytes / 16);
  hipLaunchKernelGGL(act_prep_i8_kernel, dim3(static_cast<unsigned>((n_chunks + 255) / 256)), dim3(256), 0, s,
                     reinterpret_cast<const u32x4*>(a), reinterpret_cast<u32x4*>(ws),
                     reinterpret_cast<int*>(ws + p.ap_bytes), n_chunks, wformat == LLMQ_W_INT4_PACKED ? 1 : 0);
  if (int rc = llmq_host::check_launch("act_prep_i8_kernel")) return rc;
  A8Args args{ws, reinterpret_cast<const int*>(ws + p.ap_bytes), sx, static_cast<const uint8_t*>(qweight), wscale,
              bias_or_null, out, reinterpret_cast<float*>(ws + p.ap_bytes + p.start_bytes), M, N, G, out_group,
              p.m_tiles, p.n_tiles, p.splits, p.groups_per_split};
  const bool token = sx_groups == 1 && G > 1;
  switch (dtype) {
    case LLMQ_F32: return run_typed<float>(args, p, wformat, token, s);
    case LLMQ_F16: return run_typed<f16_t>(args, p, wformat, token, s);
    default: return run_typed<bf16_t>(args, p, wformat, token, s);
  }
}
