// Integer prefill GEMM, the fast form: int8 activations (one scale per token and group, or one per token) times
// int4 / int8 group-quantized weights on the int8 matrix core,
//
//   out[m, n] = sum over g of  sx[m, g] * sw[sr(n), g] * (float)(sum_k a[m, g, k] * q[n, g, k])
//
// the A8 branch of RealQuantLinear.forward (llmquant/quantizers/real.py:94-99) with the same exact integer
// group sums but not the same fp32 roundings: there each group contributes ((float)isum * sw) * sx, added to
// the total, four separately rounded operations in group order (llmq_wq_gemm_a8 reproduces exactly that,
// and is bound by those four vector-ALU instructions per output and group); here a group contributes
// fma((float)isum * sw, sx, total), three instructions and one rounding fewer (two with one scale per token,
// which leaves the sum), and the reduction axis may be split across workgroups, so results agree with real
// mode to fp32 rounding (~1e-7), not bit for bit.
//
// llmq_wq_gemm_a8_fast has two kernels behind it. Where the output alone has tiles enough to fill the chip it
// is the kernel of llmq_wq_gemm_a8 with the relaxed epilogue (wq_gemm_a8.hip, MODE 1 / 2). Where it has not
// (a weight of a few thousand rows under a prompt of a few hundred tokens: N = 4096, K = 14336, M = 128 leaves
// that kernel at 4 % of the matrix core's peak), the reduction axis is split across workgroups by the kernel
// of this file: fp32 partial tiles in a workspace, added in a fixed order (and the bias after them) by a second
// launch.
//
// Shape: that of the tiled bf16 GEMM (wq_gemm_a16_tile.hip). A workgroup of eight waves, two per SIMD, owns a
// 128 (m) x 256 (n) output tile over its slice of the groups; a wave owns 64 x 64: 2 x 2 tiles of
// v_mfma_i32_32x32x32_i8, four k-steps of 32 per group, int32 group sums and fp32 totals in vector registers.
// All operands
// reach LDS straight from global memory (global_load_lds, 1 KB per wave instruction; 16-byte slots
// XOR-swizzled by row so that the operand reads of 16 consecutive rows are conflict-free), three or four
// stages deep: the activation tile [128 rows][128 bytes], the raw codes of the weight rows, the 128 activation
// scales and the weight scales of the group. A lane reads the activation operand of a k-step from LDS (one
// read feeds two MFMAs) and its own column's codes once per group. int4 is unpacked in registers as the
// stored nibbles n = code + 8 (one AND for the even codes of a word, a shift and an AND for the odd ones), and
// the 8 is taken back out by starting each group's sum at -8 * (sum of the group's activations) instead of
// zero: the preparation pass writes that number per token and group, and it reaches the matrix core as the C
// operand of the first k-step. Unpacking leaves the even codes of a 32-bit word in one operand register and
// the odd ones in the next, so the activation is prepared once per call (act_prep_i8_kernel) with the bytes
// of every 8 in the same order: a sum does not care about the order of its terms as long as both operands
// agree.
//
// What bounds the kernel is the vector ALU's issue port, which the matrix core shares: measured on this GPU,
// a SIMD that issues one 32x32x32 int8 MFMA and v other vector instructions per wave takes about
// 16 + 4 v cycles per MFMA (the MFMA holds the port for half of its 32 cycles; only the other half is free for
// other waves' instructions). Folding a group's 64 x 64 sums into the totals is 3 instructions per output
// (convert, two scales) = 12 per MFMA, 8 with one activation scale per token, and unpacking int4 is 3 more:
// 60-70 issue cycles per MFMA against the MFMA's own 32, so the matrix core cannot be more than about half
// busy whatever the schedule (interleaving the fold under the MFMAs by hand, a fifth k-step for the -8
// instead of the C operand, DPP-broadcast scales and deeper LDS prefetch all measured the same or slower).
#include "llmq_device.h"

namespace {

using namespace llmq;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;
constexpr int kBM = 128;
constexpr int kWaves = 8, kThreads = kWaves * kWave;
constexpr int kARowBytes = kGroup;                // int8 activation row of one group
constexpr int kATileBytes = kBM * kARowBytes;     // 16 KB
template <int BITS> constexpr int kCodeRowBytes = BITS == 4 ? kGroup / 2 : kGroup;
constexpr int kSxTileBytes = kBM * 4, kStartTileBytes = kBM * 4;

// The shape of a workgroup's tile: 128 rows by BN columns, eight waves as WM x WN, a wave owning MT x NT MFMA
// tiles of 32 x 32. MT = NT = 2 (2 x 4 waves of 64 x 64, BN = 256): every operand read from LDS feeds two MFMAs.
template <int BITS, int MT, int NT>
struct Shape {
  static constexpr int kWM = kBM / (32 * MT), kWN = kWaves / kWM;
  static constexpr int kWaveM = 32 * MT, kWaveN = 32 * NT;
  static constexpr int kBN = kWN * kWaveN;
  static constexpr int kCodeTileBytes = kBN * kCodeRowBytes<BITS>;
  static constexpr int kSwTileBytes = kBN * 4;
  static constexpr int kScalesAt = kATileBytes + kCodeTileBytes;
  static constexpr int kStageBytes = kScalesAt + kSxTileBytes + kSwTileBytes + kStartTileBytes;
  static constexpr int kStages = kStageBytes * 4 <= 160 * 1024 ? 4 : 3;
  static constexpr int kLdsBytes = kStages * kStageBytes;
  // transfers of 64 lanes each that fill one stage: 1 KB of activations or codes, or 64 four-byte values
  static constexpr int kAUnits = kATileBytes / 1024, kCodeUnits = kCodeTileBytes / 1024;
  static constexpr int kSxUnits = kBM / 64, kSwUnits = kBN / 64, kStartUnits = BITS == 4 ? kBM / 64 : 0;
  static constexpr int kUnits = kAUnits + kCodeUnits + kSxUnits + kSwUnits + kStartUnits;
  static constexpr int kDmaPerWave = (kUnits + kWaves - 1) / kWaves;
  static_assert(kBM % kWaveM == 0 && kWM * kWN == kWaves && kBN % 64 == 0 && kCodeTileBytes % 1024 == 0, "tile shape");
  // every wave the same kinds of transfer in the same slots: the widths are compile-time facts
  static_assert(kAUnits % kWaves == 0 && kCodeUnits % kWaves == 0 && kSxUnits + kSwUnits + kStartUnits <= kWaves, "slots");
};

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
  const float* bias;   // [N] or null (added by the second launch)
  void* out;           // [M, N] (written by the second launch)
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
template <int BITS, bool TOKEN, int MT, int NT>
__global__ __launch_bounds__(kThreads, 1) void wq_gemm_a8_tile_kernel(const A8Args a) {
  using S = Shape<BITS, MT, NT>;
  constexpr int kMT = MT, kNT = NT, kBN = S::kBN, kWaveM = S::kWaveM, kWaveN = S::kWaveN;
  constexpr int kScalesAt = S::kScalesAt, kSwTileBytes = S::kSwTileBytes, kStageBytes = S::kStageBytes;
  constexpr int kStages = S::kStages, kDmaPerWave = S::kDmaPerWave;
  extern __shared__ __attribute__((aligned(256))) uint8_t smem[];

  // consecutive logical tiles (the m-tiles of one n-tile first) on one XCD: the codes come out of its L2
  const int n_work = a.m_tiles * a.n_tiles * a.splits;
  const int per_xcd = (n_work + 7) / 8;
  const int logical = static_cast<int>(blockIdx.x % 8) * per_xcd + static_cast<int>(blockIdx.x / 8);
  if (logical >= n_work) return;
  const int mt = logical % a.m_tiles;
  const int nt = (logical / a.m_tiles) % a.n_tiles;
  const int sp = logical / (a.m_tiles * a.n_tiles);

  const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wv % S::kWM, wn = wv / S::kWM;
  const int lm = lane & 31, lh = lane >> 5;
  const int m0 = mt * kBM, n0 = nt * kBN;
  const int g_begin = sp * a.groups_per_split;
  const int g_end = min(g_begin + a.groups_per_split, a.G);

  // ---- global -> LDS ----------------------------------------------------------------------------------------
  // A stage is filled by transfers of 64 lanes: 16 of activations (8 rows each; lane = (row, slot), slot p of
  // row r holds chunk p ^ ((r >> 1) & 7)), the codes (1 KB each, slots swizzled by code_slot), and four bytes
  // a lane for the activation scales of 64 rows, the weight scales of 64 columns and (int4) the group starts
  // of 64 rows. Every wave issues kDmaPerWave of them per group: its share of the activation and code units
  // and one of the 64-value vectors (a wave beyond their count repeats one, with the same bytes, so that every
  // wave has the same number in flight and one vmcnt serves all).
  constexpr int kRowsPerUnit = 1024 / kCodeRowBytes<BITS>;
  constexpr int kSlots = kCodeRowBytes<BITS> / 16;
  const uint8_t* dma_base[kDmaPerWave];
  uint32_t dma_off[kDmaPerWave], dma_step[kDmaPerWave], dma_dst[kDmaPerWave];
  bool dma_wide[kDmaPerWave];
  // unit u of the activation tile / the code tile / the 64-value vectors, as this lane's part of a transfer
  auto a_unit = [&](int i, int u) {
    const int row = u * 8 + (lane >> 3);
    dma_base[i] = a.ap, dma_step[i] = kARowBytes, dma_dst[i] = u * 1024, dma_wide[i] = true;
    dma_off[i] = static_cast<uint32_t>(m0 + row) * (static_cast<uint32_t>(a.G) * kARowBytes) +
                 (((lane & 7) ^ ((row >> 1) & 7)) << 4);
  };
  auto code_unit = [&](int i, int u) {
    const int row = u * kRowsPerUnit + lane / kSlots;
    dma_base[i] = a.qw, dma_step[i] = kCodeRowBytes<BITS>, dma_dst[i] = kATileBytes + u * 1024, dma_wide[i] = true;
    dma_off[i] = static_cast<uint32_t>(min(n0 + row, a.N - 1)) * (static_cast<uint32_t>(a.G) * kCodeRowBytes<BITS>) +
                 (code_slot<BITS>(row, lane % kSlots) << 4);
  };
  auto vector_unit = [&](int i, int u) {   // u counts through the activation scales, the weight scales, the starts
    dma_wide[i] = false, dma_step[i] = 4;
    if (u < S::kSxUnits) {
      const uint32_t row = static_cast<uint32_t>(min(m0 + u * 64 + lane, a.M - 1));
      dma_base[i] = reinterpret_cast<const uint8_t*>(a.sx), dma_dst[i] = kScalesAt + u * 256;
      // (TOKEN: the tile is not read; the transfer keeps every wave's count of requests in flight the same)
      dma_off[i] = TOKEN ? row * 4 : row * static_cast<uint32_t>(a.G) * 4;
      if (TOKEN) dma_step[i] = 0;
    } else if (u < S::kSxUnits + S::kSwUnits) {
      u -= S::kSxUnits;
      const int n = min(n0 + u * 64 + lane, a.N - 1);
      dma_base[i] = reinterpret_cast<const uint8_t*>(a.sw), dma_dst[i] = kScalesAt + kSxTileBytes + u * 256;
      dma_off[i] = static_cast<uint32_t>(a.out_group > 0 ? n / a.out_group : n) * static_cast<uint32_t>(a.G) * 4;
    } else {
      u -= S::kSxUnits + S::kSwUnits;
      const uint32_t row = static_cast<uint32_t>(min(m0 + u * 64 + lane, a.M - 1));
      dma_base[i] = reinterpret_cast<const uint8_t*>(a.start);
      dma_dst[i] = kScalesAt + kSxTileBytes + kSwTileBytes + u * 256;
      dma_off[i] = row * static_cast<uint32_t>(a.G) * 4;
    }
  };
  constexpr int kVectorUnits = S::kSxUnits + S::kSwUnits + S::kStartUnits;
  constexpr int kA = S::kAUnits / kWaves, kC = S::kCodeUnits / kWaves;
  static_assert(kDmaPerWave == kA + kC + 1, "slots");
#pragma unroll
  for (int i = 0; i < kA; ++i) a_unit(i, wv * kA + i);
#pragma unroll
  for (int i = 0; i < kC; ++i) code_unit(kA + i, wv * kC + i);
  vector_unit(kA + kC, wv % kVectorUnits);

  auto request = [&](int g, int st) {
    uint8_t* stage = smem + st * kStageBytes;
#pragma unroll
    for (int i = 0; i < kDmaPerWave; ++i) {
      const uint8_t* from = dma_base[i] + dma_off[i] + static_cast<uint32_t>(g) * dma_step[i];
      if (dma_wide[i]) {
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(from), reinterpret_cast<u32x4*>(stage + dma_dst[i]),
                                         16, 0, 0);
      } else {
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const float*>(from), reinterpret_cast<float*>(stage + dma_dst[i]),
                                         4, 0, 0);
      }
    }
  };
  // Wait until at most `younger` of this wave's request batches are still in flight.
  auto wait_requests = [&](int younger) {
    if (younger <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (younger == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kDmaPerWave) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kDmaPerWave) : "memory");
  };
  static_assert(kStages <= 4 && 2 * kDmaPerWave < 64, "wait_requests");

  // ---- LDS -> operands ------------------------------------------------------------------------------------
  // activation operand of k-step j, row tile mi: row wm*64 + mi*32 + lm, chunk 4 lh + j
  uint32_t a_rd[kMT][4];
#pragma unroll
  for (int mi = 0; mi < kMT; ++mi) {
    const int row = wm * kWaveM + mi * 32 + lm;
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
  const uint32_t row_rd = kScalesAt + (wm * kWaveM + 4 * lh) * 4;
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
  for (int st = 0; st < kStages; ++st) {
    if (st < n_groups) request(g_begin + st, st);
  }
  wait_requests(min(kStages, n_groups) - 1);
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
    const uint8_t* stage = smem + st * kStageBytes;
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

    // activation scales of this lane's output rows (rows 8 q + 4 lh + 0..3 of each row tile)
    auto read_row_scales = [&]() {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int q = 0; q < 4; ++q) sx_now[mi][q] = read16(stage, row_rd + (mi * 32 + 8 * q) * 4);
    };

#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v4i fb[kNT];
#pragma unroll
      for (int ni = 0; ni < kNT; ++ni) fb[ni] = code_operand<BITS>(raw[ni], j);
      if (j < 3) {
#pragma unroll
        for (int mi = 0; mi < kMT; ++mi) fa[(j + 1) & 1][mi] = read16(stage, a_rd[mi][j + 1]);
      } else if constexpr (!TOKEN) {
        read_row_scales();   // (while the stage still holds them)
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
      wait_requests(min(kStages - 2, g_end - 2 - g));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
      if (g + kStages < g_end) request(g + kStages, st);
    }
    st = st + 1 == kStages ? 0 : st + 1;
  }
  if (late) fold();

  // ---- store ------------------------------------------------------------------------------------------------
  if constexpr (TOKEN) {
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float sx = a.sx[min(m0 + wm * kWaveM + mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3), a.M - 1)];
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni) total[mi][ni][r] *= sx;
      }
  }
  // this slice's partial tile; the second launch adds the slices in order, then the bias
  float* __restrict__ part = a.partial + static_cast<int64_t>(sp) * a.M * a.N;
#pragma unroll
  for (int ni = 0; ni < kNT; ++ni) {
    const int n = n0 + wn * kWaveN + ni * 32 + lm;
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * kWaveM + mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < a.M && n < a.N) part[static_cast<int64_t>(m) * a.N + n] = total[mi][ni][r];
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

constexpr int kTileBN = Shape<4, 2, 2>::kBN;
constexpr int kFillTiles = 160;   // fewer workgroups than this leave too much of the 256-CU chip idle

// splits == 1: the kernel of llmq_wq_gemm_a8 with the relaxed epilogue takes the call (no preparation pass,
// several independent workgroups per CU, 64 x 64 tiles where 128 x 128 are too few). This file's kernel takes
// it where the output has too few tiles and the rows are long, the reduction axis cut into slices of at
// least four groups. Measured, int4, us (that kernel / this one): 128 x 4096 x 14336 64.5 / 32.8;
// 512 x 4096 x 14336 85.5 / 67.4; but 128 x 14336 x 4096 (32 groups a row) 29.2 / 51.6; and where neither
// splits, 2048 x 14336 x 4096 252 / 261, 2048 x 4096 x 14336 209 / 214.
constexpr int kSplitMinGroups = 64;
Plan plan_for(int M, int N, int G) {
  Plan p{};
  p.m_tiles = (M + kBM - 1) / kBM;
  p.n_tiles = (N + kTileBN - 1) / kTileBN;
  const int tiles = p.m_tiles * p.n_tiles;
  int splits = 1;
  if (tiles < kFillTiles && G >= kSplitMinGroups) {
    splits = (256 + tiles - 1) / tiles;
    if (splits > G / 4) splits = G / 4;
    if (splits < 1) splits = 1;
  }
  p.groups_per_split = (G + splits - 1) / splits;
  p.splits = (G + p.groups_per_split - 1) / p.groups_per_split;
  if (p.splits == 1) return p;   // (no workspace)
  p.ap_bytes = aligned(static_cast<size_t>(p.m_tiles) * kBM * G * kARowBytes);
  p.start_bytes = aligned(static_cast<size_t>(M) * G * sizeof(int));
  p.partial_bytes = aligned(static_cast<size_t>(p.splits) * M * N * sizeof(float));
  return p;
}

template <int BITS, bool TOKEN, int MT, int NT>
int launch_tiles(const A8Args& a, dim3 grid, hipStream_t stream) {
  auto kernel = wq_gemm_a8_tile_kernel<BITS, TOKEN, MT, NT>;
  constexpr int kLds = Shape<BITS, MT, NT>::kLdsBytes;
  static bool raised = false;  // per instantiation; worst case two threads both set it
  if (!raised) {
    const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (err != hipSuccess) {
      llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));
      return static_cast<int>(err);
    }
    raised = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(kThreads), kLds, stream, a);
  return llmq_host::check_launch("wq_gemm_a8_tile_kernel");
}

template <typename T>
int run_typed(A8Args& a, const Plan& p, int wformat, bool token, hipStream_t s) {
  const int total = p.m_tiles * p.n_tiles * p.splits;
  const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
  int rc;
  if (wformat == LLMQ_W_INT4_PACKED) rc = token ? launch_tiles<4, true, 2, 2>(a, grid, s) : launch_tiles<4, false, 2, 2>(a, grid, s);
  else rc = token ? launch_tiles<8, true, 2, 2>(a, grid, s) : launch_tiles<8, false, 2, 2>(a, grid, s);
  if (rc) return rc;
  const int64_t count = static_cast<int64_t>(a.M) * a.N;
  hipLaunchKernelGGL((add_splits_bias_kernel<T>), dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s,
                     a.partial, a.bias, static_cast<T*>(a.out), count, a.N, p.splits);
  return llmq_host::check_launch("add_splits_bias_kernel");
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
  const Plan p = plan_for(M, N, G);
  const size_t need = p.ap_bytes + p.start_bytes + p.partial_bytes;
  if (!a || !sx || !qweight || !wscale || !out || (need > 0 && !workspace)) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return llmq_host::fail_invalid("activation, weight and workspace pointers must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool token = sx_groups == 1 && G > 1;
  if (p.splits == 1) {
    return llmq_host::gemm_a8_relaxed(a, sx, qweight, wscale, bias_or_null, out, M, N, G, token, out_group, wformat, dtype, s);
  }
  if ((static_cast<uint64_t>(M) + kBM) * G * kARowBytes >= (1ull << 32) ||
      static_cast<uint64_t>(N) * G * kGroup >= (1ull << 32))
    return llmq_host::fail_invalid("operands of %d x %d and %d x %d are beyond the kernel's 32-bit offsets", M,
                                   G * kGroup, N, G * kGroup);
  if (workspace_bytes < need)
    return llmq_host::fail_invalid("workspace of %zu bytes is too small, need %zu", workspace_bytes, need);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  const int64_t n_chunks = static_cast<int64_t>(M) * G * (kARowBytes / 16);
  hipLaunchKernelGGL(act_prep_i8_kernel, dim3(static_cast<unsigned>((n_chunks + 255) / 256)), dim3(256), 0, s,
                     reinterpret_cast<const u32x4*>(a), reinterpret_cast<u32x4*>(ws),
                     reinterpret_cast<int*>(ws + p.ap_bytes), n_chunks, wformat == LLMQ_W_INT4_PACKED ? 1 : 0);
  if (int rc = llmq_host::check_launch("act_prep_i8_kernel")) return rc;
  A8Args args{ws, reinterpret_cast<const int*>(ws + p.ap_bytes), sx, static_cast<const uint8_t*>(qweight), wscale,
              bias_or_null, out, reinterpret_cast<float*>(ws + p.ap_bytes + p.start_bytes), M, N, G, out_group,
              p.m_tiles, p.n_tiles, p.splits, p.groups_per_split};
  switch (dtype) {
    case LLMQ_F32: return run_typed<float>(args, p, wformat, token, s);
    case LLMQ_F16: return run_typed<f16_t>(args, p, wformat, token, s);
    default: return run_typed<bf16_t>(args, p, wformat, token, s);
  }
}
