// Weight-only quantized GEMM for prompt-sized activations (M in the hundreds and thousands), gfx950:
// bf16 (or fp16) activations times int4 / int8 group-quantized weights on the 16-bit matrix core, with no dense
// copy of the weight anywhere. The text below describes the bf16 form; what differs for fp16 is said at kBiased.
//
//   out[m, n] = sum over g of  wscale[sr(n), g] * sum_k x[m, g*128 + k] * code[n, g, k]
//
// the weight-only branch of RealQuantLinear.forward (llmquant/quantizers/real.py:84-91): products of a
// bf16 value and a small integer are exact in fp32, the matrix core adds them in fp32, and the scale is
// applied once per group. (The reference's kernel mode dequantizes the whole weight to the activation
// dtype and calls the BLAS library for M > 4, llmquant/quantizers/kernel.py:68-79,88-91: nine times the
// int4 codes' bytes through HBM per call, and a second rounding per weight.)
//
// Shape. A workgroup of eight waves (two per SIMD) owns a 128 (m) x 256 (n) tile of the output; every wave owns
// 32 of the 256 columns and all 128 rows: 4 x 1 MFMA tiles of 32 x 32 (v_mfma_f32_32x32x16_bf16), eight
// k-steps of 16 per group. A lane converts the codes of one column only, and each converted operand feeds four
// MFMAs (with 64 x 64 per wave two waves converted the same codes: measured 3-4 % slower on the large shapes).
// Everything reaches LDS straight from global memory (global_load_lds_dwordx4, 1 KB per wave instruction,
// XOR-swizzled by row so that the operand reads are conflict-free), three stages deep for int4, two for int8:
// the activation tile, the raw codes of the 256 weight rows, the activation-sum records and the group's scales.
// The workgroup meets once per group, before the last k-step, and the next group's operands are read from LDS
// behind that barrier.
//
// Codes become bf16 without a conversion instruction: a nibble n = code + 8 placed in the mantissa of
// 16.0 (bits 0x4180 | n << 3) IS the bf16 value 16 + n, two nibbles per AND-OR (int8: code + 128 through
// v_cvt_f32_ubyte, whose upper half is the bf16 value). The matrix core therefore sums x * (code + B),
// B = 24 or 128, and B * sum_k x is taken out again per group by one more k-step in front of the eight: the
// group's activation sum, cut into three bf16 pieces, against the constant -B. The fp32 group sum is then
// folded into the fp32 total with one multiply-add by the group's weight scale.
//
// The activation is prepared once per call by act_prep_kernel: rows padded to whole tiles, within every
// 16-byte chunk the eight values reordered to (0, 4, 1, 5, 2, 6, 3, 7), the order in which the AND-OR above
// leaves the codes (a sum does not care about the order of its terms, as long as both operands agree), and
// the per-group sums written as records of bf16 pieces.
//
// Small N: a split of the reduction axis across workgroups, fp32 partial tiles in a workspace, added in a
// fixed order by a second launch (the result does not depend on which workgroup finished first).
#include <stdlib.h>

#include <type_traits>

#include "llmq_device.h"

namespace {

using namespace llmq;

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// bfloat16: the matrix core sums x * (code + B) and B * sum x is taken out again (below). float16 has the mantissa
// to hold B + code as well, but the pieces of a group's activation sum do not fit its exponent range (128 values of
// up to 65504, and pieces of a small sum fall below its smallest step), so there the bias is subtracted from the
// operand itself, exactly, with one packed add per two codes, and there is no correction step.
template <typename T> constexpr bool kBiased = std::is_same<T, bf16_t>::value;
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;
constexpr int kRowBytes = kGroup * 2;          // one activation row of one group
template <int BITS> constexpr int kCodeRowBytes = BITS == 4 ? kGroup / 2 : kGroup;

// The workgroup's tile: BM activation rows x 32 COLS weight rows; a wave owns 32 of the columns, all the rows and
// one KH-th of every group's k-steps. Wide (128 x 256, eight waves, two per SIMD) is the throughput shape. Narrow
// (64 x 128) is for outputs that have too few wide tiles to occupy the chip (a 512-token prompt against a 3072-row
// weight: 48 wide tiles, 192 narrow ones): its eight waves are four column blocks times two halves of the group
// (still two waves per SIMD, so that one converts codes while the other multiplies), the halves' totals are added
// through LDS once, at the end, and the smaller stages leave LDS for four of them in flight.
template <int BM, int COLS, int KH> struct Shape {
  static constexpr int kBM = BM;                 // activation rows per workgroup
  static constexpr int kWaveM = BM;              // ... and per wave
  static constexpr int kWaveN = 32;              // weight rows (output columns) per wave
  static constexpr int kColWaves = COLS;         // column blocks
  static constexpr int kKH = KH;                 // waves that share a column block, each with 8 / KH k-steps of a group
  static constexpr int kWaves = COLS * KH;
  static constexpr int kBN = kWaveN * COLS;
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int kTileBytes = BM * kRowBytes;
  static constexpr int kMT = BM / 32, kNT = kWaveN / 32;
  static constexpr int kRecTileBytes = BM * 16;
  static constexpr int kScaleTileBytes = kBN * 4;
  static constexpr int kRecWaves = BM / 64;      // waves that fetch the activation-sum records (64 rows each)
  static constexpr int kScaleWaves = kBN / 64;   // ... and, after them, the scales (64 columns each)
  template <int BITS> static constexpr int kCodeTileBytes = kBN * kCodeRowBytes<BITS>;
  template <int BITS>
  static constexpr int kStageBytes = kTileBytes + kCodeTileBytes<BITS> + kRecTileBytes + kScaleTileBytes;
  // as many stages as fit the 160 KB of LDS, at most four: a group's transfers are requested kStages - 1 groups
  // before it is multiplied (wide: three for int4, 153 KB, two for int8; narrow: four)
  template <int BITS>
  static constexpr int kStages = (160 * 1024 / kStageBytes<BITS>) >= 4 ? 4 : (160 * 1024 / kStageBytes<BITS>);
  template <int BITS> static constexpr int kLdsBytes = kStages<BITS> * kStageBytes<BITS>;
};
using Wide = Shape<128, 8, 1>;
using Narrow = Shape<64, 4, 2>;
// (what the host side sizes for when it does not say which: the wide tile)
constexpr int kBM = Wide::kBM, kBN = Wide::kBN;


// ---- activation preparation -----------------------------------------------------------------------
// One lane per 16-byte chunk, 16 lanes per (row, group): `v` holds the chunk's eight bf16 values (zeros in a lane
// with nothing to do; a row of 16 lanes is active or idle as one). Writes the reordered chunk, and from the row's
// first lane the record of the group's sum.
template <typename T>
__device__ __forceinline__ void emit_prepared(const u32x4 v, const bool active, const bool first_of_row,
                                              u32x4* __restrict__ chunk_out, u32x4* __restrict__ record_out) {
  if constexpr (!kBiased<T>) {
    // (no correction step: the records stay part of the layout and are zeros)
    if (!active) return;
    *chunk_out = interleave_halves(v);
    if (first_of_row) *record_out = u32x4{0u, 0u, 0u, 0u};
    return;
  }
  float f[8];
  Pack<bf16_t>::unpack(v, f);
  float s = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
  s = row16_sum(s);
  if (!active) return;
  // (x0 x1)(x2 x3)(x4 x5)(x6 x7) -> (x0 x4)(x1 x5)(x2 x6)(x3 x7)
  u32x4 o;
  o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
  o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
  o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
  o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
  *chunk_out = o;
  if (first_of_row) {
    // s = hi + mid + lo, each a bf16: 24 bits of the sum
    const uint32_t hi = bf16_bits_rne(s);
    const float r1 = s - __builtin_bit_cast(float, hi << 16);
    const uint32_t mid = bf16_bits_rne(r1);
    const float r2 = r1 - __builtin_bit_cast(float, mid << 16);
    const uint32_t lo = bf16_bits_rne(r2);
    *record_out = u32x4{hi | (mid << 16), lo, 0u, 0u};  // k' slots 0..2 of the correction step
  }
}

template <typename T>
__global__ __launch_bounds__(256) void act_prep_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ xp,
                                                       u32x4* __restrict__ rec, const int64_t n_chunks) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const bool active = i < n_chunks;  // n_chunks is a multiple of 16: a row of 16 lanes is active or idle as one
  u32x4 v = {0u, 0u, 0u, 0u};
  if (active) v = x[i];
  emit_prepared<T>(v, active, (threadIdx.x & 15) == 0, xp + (active ? i : 0), rec + (active ? i >> 4 : 0));
}

// LlamaRMSNorm (optionally on x + delta, the residual add in front of it, which is stored as well) whose result
// goes straight into prepared form: what act_prep_kernel would make of llmq_add_rmsnorm's output, without that
// tensor and without the second launch. One workgroup per row, the arithmetic and rounding points of
// rmsnorm_kernel (csrc/prefill_ops.hip): out = w * bf16(x_f32 * rsqrt(mean(x_f32^2) + eps)), rounded to bf16.
// hidden is a multiple of 128, so the 16 lanes of a (row, group) are in the loop together.
constexpr int kNormThreads = 256;
template <typename T, bool ADD>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_prep_kernel(const T* __restrict__ x,
                                                                   const T* __restrict__ delta,
                                                                   const T* __restrict__ w,
                                                                   T* __restrict__ sum_out, u32x4* __restrict__ xp,
                                                                   u32x4* __restrict__ rec, const int hidden,
                                                                   const float eps) {
  __shared__ float red[kNormThreads / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * hidden;
  const T* row = x + base;
  const int tid = threadIdx.x;
  float ss = 0.0f;
  for (int i = tid * 8; i < hidden; i += kNormThreads * 8) {
    float f[8];
    Pack<T>::unpack(load16(row + i), f);
    if constexpr (ADD) {
      float d[8];
      Pack<T>::unpack(load16(delta + base + i), d);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = round_through<T>(f[e] + d[e]);
      store16(sum_out + base + i, Pack<T>::pack(f));
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
  }
  ss = wave_sum(ss);
  if ((tid & (kWave - 1)) == 0) red[tid / kWave] = ss;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int k = 0; k < kNormThreads / kWave; ++k) total += red[k];
  const float inv_rms = rsqrtf(total / static_cast<float>(hidden) + eps);
  // (with ADD a thread reads back exactly the packets it stored above)
  const T* src = ADD ? sum_out + base : row;
  const int64_t chunk0 = base >> 3;   // the row's first chunk; 16 chunks a group
  for (int i = tid * 8; i < hidden; i += kNormThreads * 8) {
    float f[8], g[8];
    Pack<T>::unpack(load16(src + i), f);
    Pack<T>::unpack(load16(w + i), g);
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = g[e] * round_through<T>(f[e] * inv_rms);
    const int64_t chunk = chunk0 + (i >> 3);
    emit_prepared<T>(Pack<T>::pack(f), true, (tid & 15) == 0, xp + chunk, rec + (chunk >> 4));
  }
}

struct TileArgs {
  const uint8_t* xp;   // [M, G*128] bf16, chunks reordered
  const uint8_t* rec;  // [M, G] records of 16 bytes
  const uint8_t* qw;   // [N, G, 128] int8 or [N, G, 64] packed int4
  const float* sw;     // [scale_rows, G]
  void* out;           // [M, N] bf16 (one split)
  float* partial;      // [splits][M][N] fp32 (more)
  int M, N, G, out_group;
  int m_tiles, n_tiles, splits, groups_per_split;
  // kEpiGateUpSilu: the prepared activation of the next GEMM (its xp and rec, next_G groups a row)
  uint8_t* next_xp;
  uint8_t* next_rec;
  int next_G;
};

// What a workgroup does with its totals. kEpiStore: rounds them to bf16 into out (or leaves fp32 partial tiles).
// kEpiGateUpSilu: the weight is gate_proj's rows followed by up_proj's (N = 2 I); a tile is 128 gate rows and the
// 128 up rows that belong to them, and the workgroup writes act = silu(bf16 gate) * bf16 up (the rounding points of
// `act_fn(gate) * up` on bf16 tensors) for its 128 x 128 block straight into the next GEMM's prepared activation:
// the block is one group of 128 of that activation's reduction axis, so its chunks and records are complete.
enum Epilogue { kEpiStore = 0, kEpiGateUpSilu = 1 };
constexpr int kEpiRowBytes = 128 * 2 + 16;   // a row of the gate (or up) block in LDS: 16 bytes of padding per row

// LDS, per stage: the activation tile [BM rows][16 slots of 16 bytes], the raw codes of the workgroup's weight rows
// for one group ([BN][64] bytes of int4 or [BN][128] of int8, slots XOR-swizzled by row like the activation), the
// activation-sum records and the group's scales.
// slot of chunk c in weight row `row`: 16 consecutive rows read the same chunk at once and must land in
// 16 different bank quads
template <int BITS> __device__ __forceinline__ int code_slot(int row, int c) {
  return BITS == 4 ? c ^ ((row >> 2) & 3) : c ^ ((row >> 1) & 7);
}


// The four operand words of a k-step of the wave (`raw`: its k-steps' codes one after the other, one 32-bit word
// of int4 or two of int8 a step); operand word i pairs codes i and i + 4.
template <typename T, int BITS>
__device__ __forceinline__ u32x4 operand_words(const uint32_t* raw, int step, uint32_t magic) {
  u32x4 w = BiasedCodes<T, BITS>::operand(raw, step, magic);
  if constexpr (!kBiased<T>) {
    const _Float16 b = static_cast<_Float16>(BiasedCodes<T, BITS>::kBias);
    const h2 bias = {b, b};
    w.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w.x) - bias);
    w.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w.y) - bias);
    w.z = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w.z) - bias);
    w.w = __builtin_bit_cast(uint32_t, __builtin_bit_cast(h2, w.w) - bias);
  }
  return w;
}

template <typename T> __device__ __forceinline__ v16f mfma(const u32x4& a, const u32x4& b, const v16f& c) {
  if constexpr (std::is_same<T, bf16_t>::value)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}
template <typename T> __device__ __forceinline__ uint16_t bits16(float v) {
  return __builtin_bit_cast(uint16_t, from_float<T>(v));
}

template <typename T, int BITS, int EPI, typename S>
__global__ __launch_bounds__(S::kThreads, 1) void wq_gemm_a16_tile_kernel(const TileArgs a) {
  extern __shared__ __attribute__((aligned(256))) uint8_t smem[];
  static_assert(EPI == kEpiStore || std::is_same<S, Wide>::value, "the gate|up epilogue is laid out for the wide tile");
  constexpr int kBM = S::kBM, kBN = S::kBN, kWaveM = S::kWaveM, kWaveN = S::kWaveN, kWaves = S::kWaves;
  constexpr int kThreads = S::kThreads, kTileBytes = S::kTileBytes, kMT = S::kMT, kNT = S::kNT;
  constexpr int kRecTileBytes = S::kRecTileBytes, kRecWaves = S::kRecWaves, kScaleWaves = S::kScaleWaves;
  constexpr int kCodeTileB = S::template kCodeTileBytes<BITS>, kStageB = S::template kStageBytes<BITS>;
  constexpr int kStagesN = S::template kStages<BITS>;
  constexpr int kKH = S::kKH, kSteps = 8 / kKH;   // k-steps of a group that one wave multiplies

  // Workgroups are dealt to the 8 XCDs round-robin by their index; a run of consecutive logical tiles
  // (the m-tiles of one n-tile first: they read the same weights) is put on one XCD, so the codes come
  // out of that XCD's L2 after the first reader.
  const int n_work = a.m_tiles * a.n_tiles * a.splits;
  const int per_xcd = (n_work + 7) / 8;
  const int logical = static_cast<int>(blockIdx.x % 8) * per_xcd + static_cast<int>(blockIdx.x / 8);
  if (logical >= n_work) return;
  const int mt = logical % a.m_tiles;
  const int nt = (logical / a.m_tiles) % a.n_tiles;
  const int sp = logical / (a.m_tiles * a.n_tiles);

  // (the wave's index as a scalar: LDS addresses of the transfers are then scalar arithmetic into M0)
  const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  // every wave all the rows, 32 of the columns, and half kh of every group's k-steps (kKH == 1: all of them)
  const int wm = 0, wn = wv % S::kColWaves;
  const int kh = kKH == 1 ? 0 : __builtin_amdgcn_readfirstlane(wv / S::kColWaves);
  static_assert(kKH == 1 || (kKH == kMT && kNT == 1), "the waves of a column block keep one 32 x 32 row tile each");
  const int lm = lane & 31, lh = lane >> 5;
  // (kEpiGateUpSilu: n0 is the tile's first gate row; column c of the tile is weight row weight_row(c))
  const int m0 = mt * kBM, n0 = EPI == kEpiGateUpSilu ? nt * (kBN / 2) : nt * kBN;
  auto weight_row = [&](int c) {
    if constexpr (EPI == kEpiGateUpSilu) return c < kBN / 2 ? n0 + c : a.N / 2 + n0 + (c - kBN / 2);
    else return min(n0 + c, a.N - 1);
  };
  const int g_begin = sp * a.groups_per_split;
  const int g_end = min(g_begin + a.groups_per_split, a.G);

  // ---- global -> LDS: what this lane fetches for each of its wave's transfer instructions -------------
  // One instruction moves 64 x 16 bytes into 1 KB of consecutive LDS; which global chunk a lane fetches
  // for its place there carries the swizzle. The activation and its records are the kernel's own
  // buffers, padded to whole tiles of rows, so their rows need no clamping.
  // activation: instruction i of a wave = rows wv*16 + 4 i .. + 3, lane = (row, slot); slot p of row r
  // holds chunk p ^ (r & 15), and r & 15 = 4 i + lane / 16
  constexpr int kXInstr = kBM / 4 / kWaves;  // 4
  const uint32_t x_row_bytes = static_cast<uint32_t>(a.G) * kRowBytes;
  uint32_t x_off[kXInstr];
#pragma unroll
  for (int i = 0; i < kXInstr; ++i) {
    const int row = wv * (kBM / kWaves) + i * 4 + (lane >> 4);
    x_off[i] = static_cast<uint32_t>(m0 + row) * x_row_bytes + (((lane & 15) ^ (row & 15)) << 4);
  }
  // codes: instructions of 16 (int4) or 8 (int8) weight rows each; kCodeInstr per wave (wide: 2 / 4), and where
  // that does not come out even, one more from each of the first kLeftCodes waves
  constexpr int kCodeInstr = kCodeTileB / 1024 / kWaves, kLeftCodes = kCodeTileB / 1024 % kWaves;
  constexpr int kRowsPerInstr = 1024 / kCodeRowBytes<BITS>;
  constexpr int kSlots = kCodeRowBytes<BITS> / 16;
  const uint32_t w_row_bytes = static_cast<uint32_t>(a.G) * kCodeRowBytes<BITS>;
  uint32_t w_off[kCodeInstr + 1];
#pragma unroll
  for (int i = 0; i < kCodeInstr + 1; ++i) {
    const int instr = i < kCodeInstr ? wv * kCodeInstr + i : kWaves * kCodeInstr + wv % (kLeftCodes ? kLeftCodes : 1);
    const int row = instr * kRowsPerInstr + lane / kSlots;
    const int chunk = code_slot<BITS>(row, lane % kSlots);  // the swizzle is its own inverse
    w_off[i] = static_cast<uint32_t>(weight_row(row)) * w_row_bytes + chunk * 16;
  }
  // One further instruction from the waves after those: the records (kRecWaves waves, 64 rows each), then the
  // scales (kScaleWaves waves, 64 columns each).
  constexpr int kExtraWaves = kLeftCodes + kRecWaves + kScaleWaves;
  static_assert(kExtraWaves <= kWaves, "at most one transfer instruction per wave beyond the even share");
  const int rec_wave = (wv + kWaves - kLeftCodes) % kWaves % kRecWaves;
  const int scale_wave = (wv + kWaves - kLeftCodes - kRecWaves) % kWaves % kScaleWaves;
  const uint32_t r_off = static_cast<uint32_t>(m0 + rec_wave * 64 + lane) * a.G * 16;
  const float* sw_lane;
  {
    const int n = weight_row(scale_wave * 64 + lane);
    sw_lane = a.sw + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * a.G;
  }

  // (a lane's 32-bit offset goes through an empty asm where it is used: the compiler then adds it to the scalar
  // base inside the instruction, scalar base + 32-bit lane offset, instead of keeping a 64-bit address per lane
  // and transfer across the loop and adding the group's step to each with the vector ALU)
  auto here = [](uint32_t offset) {
    asm volatile("" : "+v"(offset));
    return offset;
  };
  auto request = [&](int g, int buf) {
    uint8_t* stage = smem + buf * kStageB;
    const uint8_t* xg = a.xp + static_cast<uint32_t>(g) * kRowBytes;
#pragma unroll
    for (int i = 0; i < kXInstr; ++i) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(xg + here(x_off[i])),
                                       reinterpret_cast<u32x4*>(stage + (wv * (kBM / kWaves) + i * 4) * kRowBytes), 16,
                                       0, 0);
    }
    const uint8_t* wg = a.qw + static_cast<uint32_t>(g) * kCodeRowBytes<BITS>;
#pragma unroll
    for (int i = 0; i < kCodeInstr; ++i) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(wg + here(w_off[i])),
                                       reinterpret_cast<u32x4*>(stage + kTileBytes + (wv * kCodeInstr + i) * 1024), 16,
                                       0, 0);
    }
    if (wv < kLeftCodes) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(wg + here(w_off[kCodeInstr])),
                                       reinterpret_cast<u32x4*>(stage + kTileBytes + (kWaves * kCodeInstr + wv) * 1024),
                                       16, 0, 0);
    } else if (wv < kLeftCodes + kRecWaves) {
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(a.rec + static_cast<uint32_t>(g) * 16 + here(r_off)),
                                       reinterpret_cast<u32x4*>(stage + kTileBytes + kCodeTileB + rec_wave * 1024),
                                       16, 0, 0);
    } else if (wv < kExtraWaves) {
      // the scales of 64 columns, one float per lane
      __builtin_amdgcn_global_load_lds(
          sw_lane + g, reinterpret_cast<float*>(stage + kTileBytes + kCodeTileB + kRecTileBytes + scale_wave * 256),
          4, 0, 0);
    }
  };
  // transfer instructions per wave and group (a compile-time count per branch: the waits below name how many
  // of the youngest may still be in flight)
  constexpr int kDmaPerWave = kXInstr + kCodeInstr + 1;   // the first kExtraWaves waves; the others: one fewer

  // ---- LDS -> operands ----------------------------------------------------------------------------------
  // activation operand of k-step j, row tile mi: row mi*32 + lm, chunk (8 lh + j) ^ (lm & 15)
  // (the wave's own k-steps are kh * kSteps + j, j < kSteps: its step j is at a_base ^ (j << 4))
  const uint32_t a_base = (wm * kWaveM + lm) * kRowBytes + (((8 * lh + kh * kSteps) ^ (lm & 15)) << 4);
  // this lane's codes of a group: weight row wn*32 + lm, k in [64 lh, 64 lh + 64), of which the wave's k-steps are
  // kRawBytes bytes: the 16-byte chunks (lh kKH + kh) kRawLoads + q, at c_base ^ (q << 4), or (8 bytes) one half
  // of a chunk
  constexpr int kRawBytes = kSteps * (BITS == 4 ? 4 : 8);
  constexpr int kRawLoads = kRawBytes / 16, kRawWords = kRawBytes / 4;
  static_assert(kRawBytes == 8 || kRawBytes % 16 == 0, "a wave's codes of a group: 16-byte chunks, or half of one");
  uint32_t c_base[kNT];
#pragma unroll
  for (int ni = 0; ni < kNT; ++ni) {
    const int row = wn * kWaveN + ni * 32 + lm;
    const int first = (lh * kKH + kh) * kRawBytes;   // byte of the lane's row
    c_base[ni] = kTileBytes + row * kCodeRowBytes<BITS> + code_slot<BITS>(row, first >> 4) * 16 + (first & 15);
  }
  auto read16 = [&](const uint8_t* stage, uint32_t offset) { return *reinterpret_cast<const u32x4*>(stage + offset); };

  float total[kMT][kNT][16];
#pragma unroll
  for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) total[mi][ni][r] = 0.0f;
  uint32_t sixteen = BiasedCodes<T, BITS>::kMagic;  // 16.0 (int8 in float16: 256.0) twice; kept in a vector register (see and_or)
  asm volatile("" : "+v"(sixteen));
  const uint32_t nb = bf16_bits_rne(-BiasedCodes<T, BITS>::kBias);  // exact (read where kBiased<T> only)
  const uint32_t nb2 = (lh || kh) ? 0u : (nb | (nb << 16));   // (the correction step belongs to the group's first k-steps)
  const u32x4 bias_operand = {nb2, nb2, 0u, 0u};

  // ---- prologue: the first groups on their way, the first one's operands in registers ---------------------
#pragma unroll
  for (int st = 0; st < kStagesN; ++st) {
    if (g_begin + st < g_end) request(g_begin + st, st);
  }
  // (the first group's transfers only, where all kStages batches exist: the loop waits for each later one in turn)
  if (g_end - g_begin >= kStagesN) {
    if (wv < kExtraWaves) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStagesN - 1) * kDmaPerWave) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStagesN - 1) * (kDmaPerWave - 1)) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();

  // What a lane holds of the group it is about to multiply: the records (operand of the correction
  // step), its raw codes, its columns' scales and the activation operands of k-step 0.
  u32x4 rec[kMT], fa[2][kMT];
  uint32_t raw[kNT][kRawWords];
  float scale[kNT];
  auto fetch_group_operands = [&](int st) {
    const uint8_t* stage = smem + st * kStageB;
    if constexpr (kBiased<T>) {
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
        rec[mi] = read16(stage, kTileBytes + kCodeTileB + (wm * kWaveM + mi * 32 + lm) * 16);
    }
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni) {
      if constexpr (kRawBytes == 8) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(stage + c_base[ni]);
        raw[ni][0] = v.x, raw[ni][1] = v.y;
      } else {
#pragma unroll
        for (int q = 0; q < kRawLoads; ++q) {
          const u32x4 v = read16(stage, c_base[ni] ^ (q << 4));
          raw[ni][4 * q] = v.x, raw[ni][4 * q + 1] = v.y, raw[ni][4 * q + 2] = v.z, raw[ni][4 * q + 3] = v.w;
        }
      }
    }
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni)
      scale[ni] = *reinterpret_cast<const float*>(stage + kTileBytes + kCodeTileB + kRecTileBytes +
                                                  (wn * kWaveN + ni * 32 + lm) * 4);
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi) fa[0][mi] = read16(stage, mi * 32 * kRowBytes + a_base);
  };
  fetch_group_operands(0);

  // Two waves share a SIMD: while one converts codes or adds its group sums into the totals, the other
  // keeps the matrix core busy. Within a wave the next k-step's activation operands are requested before
  // the current step's multiplications. The workgroup meets once per group, before the last k-step: by
  // then every read of the group's LDS stage has been issued and has returned (the last step's operands are
  // in registers), so behind the barrier that stage takes the transfers of the group kStages ahead; and each
  // wave has waited, in front of the barrier, for its own transfers of the next group (requested kStages - 1
  // groups ago), so behind the barrier the next group's stage is complete: the last k-step runs while the
  // next group's operands come out of it, and no wave starts a group waiting for memory or LDS.
  int st = 0;  // the stage of group g
  for (int g = g_begin; g < g_end; ++g) {
    const uint8_t* stage = smem + st * kStageB;
    const int st_next = st + 1 == kStagesN ? 0 : st + 1;
    float scale_now[kNT];
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni) scale_now[ni] = scale[ni];

    // The group's sums start at -B * xsum[m] (one k-step: the three bf16 pieces of the activation sum
    // against the constant -B; the upper half of the wave, k' 8..15, multiplies zeros), then take the
    // eight k-steps of x * (code + B).
    v16f acc[kMT][kNT];
    {
      const v16f zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni) acc[mi][ni] = kBiased<T> && kh == 0 ? mfma<T>(rec[mi], bias_operand, zero) : zero;
    }
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
      u32x4 fb[kNT];
#pragma unroll
      for (int ni = 0; ni < kNT; ++ni) fb[ni] = operand_words<T, BITS>(raw[ni], j, sixteen);
      if (j < kSteps - 1) {
#pragma unroll
        for (int mi = 0; mi < kMT; ++mi) fa[(j + 1) & 1][mi] = read16(stage, mi * 32 * kRowBytes + (a_base ^ ((j + 1) << 4)));
      } else {
        // own transfers of the next group have landed (the youngest kStages - 2 batches may stay in flight)
        if (kStagesN >= 3 && g + kStagesN - 1 < g_end) {  // (the batches of groups g + 2 .. exist and are younger)
          if (wv < kExtraWaves) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStagesN - 2) * kDmaPerWave) : "memory");
          else asm volatile("s_waitcnt vmcnt(%0)" ::"n"((kStagesN - 2) * (kDmaPerWave - 1)) : "memory");
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        if (g + kStagesN < g_end) request(g + kStagesN, st);
        if (g + 1 < g_end) fetch_group_operands(st_next);  // (fa[0]: the last step multiplies out of fa[1])
      }
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
        for (int ni = 0; ni < kNT; ++ni) acc[mi][ni] = mfma<T>(fa[j & 1][mi], fb[ni], acc[mi][ni]);
    }
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
      for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) total[mi][ni][r] = fmaf(scale_now[ni], acc[mi][ni][r], total[mi][ni][r]);
    st = st_next;
  }

  // ---- store: register r of a 32 x 32 tile is row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
  if constexpr (EPI == kEpiGateUpSilu) {
    // Waves 0..3 hold the block's gate columns, 4..7 its up columns: both go to LDS as bf16 (no wave reads a
    // stage any more: the loop's last barrier came after every wave's last operand read), then a lane takes a
    // 16-byte chunk of a row at a time, 16 lanes a row, as act_prep_kernel does with a tensor in memory.
    __builtin_amdgcn_s_barrier();
    uint8_t* block = smem + (wn >> 2) * (kBM * kEpiRowBytes);
    const int col = (wn & 3) * 32 + lm;
#pragma unroll
    for (int mi = 0; mi < kMT; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = mi * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
        *reinterpret_cast<uint16_t*>(block + row * kEpiRowBytes + col * 2) = bits16<T>(total[mi][0][r]);
      }
    __syncthreads();
    u32x4* __restrict__ next_xp = reinterpret_cast<u32x4*>(a.next_xp);
    u32x4* __restrict__ next_rec = reinterpret_cast<u32x4*>(a.next_rec);
#pragma unroll
    for (int pass = 0; pass < kBM * 16 / kThreads; ++pass) {
      const int q = pass * kThreads + tid, row = q >> 4, chunk = q & 15;
      float g[8], u[8];
      Pack<T>::unpack(read16(smem, row * kEpiRowBytes + chunk * 16), g);
      Pack<T>::unpack(read16(smem, kBM * kEpiRowBytes + row * kEpiRowBytes + chunk * 16), u);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = round_through<T>(g[e] / (1.0f + expf(-g[e]))) * u[e];
      const int64_t at = static_cast<int64_t>(m0 + row) * a.next_G + nt;   // (row, group) of the next activation
      emit_prepared<T>(Pack<T>::pack(g), true, chunk == 0, next_xp + at * 16 + chunk, next_rec + at);
    }
    return;
  }
  // one 32 x 32 tile of totals, whose first row is m_first and whose column (this lane's) is n
  auto store_tile = [&](const float (&v)[16], int m_first, int n) {
    if (a.splits == 1) {
      T* __restrict__ out = static_cast<T*>(a.out);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m_first + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < a.M && n < a.N) out[static_cast<int64_t>(m) * a.N + n] = from_float<T>(v[r]);
      }
    } else {
      float* __restrict__ part = a.partial + static_cast<int64_t>(sp) * a.M * a.N;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m_first + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (m < a.M && n < a.N) part[static_cast<int64_t>(m) * a.N + n] = v[r];
      }
    }
  };
  if constexpr (kKH > 1) {
    // The kKH waves of a column block hold the totals of their parts of every group. Wave kh keeps row tile kh and
    // hands the others over through LDS (4 KB a tile, [register][lane]; the stages are free: the loop's last
    // barrier came after every wave's last operand read and its last transfer), then adds the parts of its tile in
    // the order of the waves, its own in its place.
    float* exchange = reinterpret_cast<float*>(smem);
    auto slot = [&](int from, int tile) { return ((from * S::kColWaves + wn) * (kKH - 1) + (tile - (tile > from))) * 1024; };
    float own[16];
#pragma unroll
    for (int t = 0; t < kKH; ++t) {
      if (t == kh) {
#pragma unroll
        for (int r = 0; r < 16; ++r) own[r] = total[t][0][r];
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) exchange[slot(kh, t) + r * 64 + lane] = total[t][0][r];
      }
    }
    __syncthreads();
    float sum[16];
#pragma unroll
    for (int from = 0; from < kKH; ++from) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float part = from == kh ? own[r] : exchange[slot(from, kh) + r * 64 + lane];
        sum[r] = from == 0 ? part : sum[r] + part;
      }
    }
    store_tile(sum, m0 + kh * 32, n0 + wn * kWaveN + lm);
  } else {
#pragma unroll
    for (int ni = 0; ni < kNT; ++ni)
#pragma unroll
      for (int mi = 0; mi < kMT; ++mi)
        store_tile(total[mi][ni], m0 + wm * kWaveM + mi * 32, n0 + wn * kWaveN + ni * 32 + lm);
  }
}

// out[i] = bf16(partial[0][i] + partial[1][i] + ...), slices added in order; four values per lane.
template <typename T>
__global__ __launch_bounds__(256) void add_splits_kernel(const float* __restrict__ partial, T* __restrict__ out,
                                                         const int64_t count, const int splits) {
  const int64_t i4 = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i4 >= count) return;
  if (i4 + 4 <= count && (count & 3) == 0) {
    u32x4 v = load16(partial + i4);
    float s[4];
    Pack<float>::unpack(v, s);
    for (int k = 1; k < splits; ++k) {
      float t[4];
      Pack<float>::unpack(load16(partial + k * count + i4), t);
#pragma unroll
      for (int e = 0; e < 4; ++e) s[e] = s[e] + t[e];
    }
    *reinterpret_cast<u32x2*>(out + i4) =
        u32x2{static_cast<uint32_t>(bits16<T>(s[0])) | static_cast<uint32_t>(bits16<T>(s[1])) << 16,
              static_cast<uint32_t>(bits16<T>(s[2])) | static_cast<uint32_t>(bits16<T>(s[3])) << 16};
  } else {
    // a count that is not a multiple of four leaves the later slices off 16-byte alignment: this lane's own
    // (up to) four values one at a time
    const int64_t end = i4 + 4 < count ? i4 + 4 : count;
    for (int64_t i = i4; i < end; ++i) {
      float s = partial[i];
      for (int k = 1; k < splits; ++k) s = s + partial[k * count + i];
      out[i] = from_float<T>(s);
    }
  }
}

template <typename T, int BITS, int EPI, typename S = Wide>
int launch_tiles(const TileArgs& a, dim3 grid, hipStream_t stream) {
  auto kernel = wq_gemm_a16_tile_kernel<T, BITS, EPI, S>;
  constexpr int kLds = S::template kLdsBytes<BITS>;
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
  hipLaunchKernelGGL(kernel, grid, dim3(S::kThreads), kLds, stream, a);
  return llmq_host::check_launch("wq_gemm_a16_tile_kernel");
}

constexpr size_t kAlign = 256;
size_t aligned(size_t bytes) { return (bytes + kAlign - 1) / kAlign * kAlign; }

struct Plan {
  int m_tiles, n_tiles, splits, groups_per_split;
  size_t xp_bytes, rec_bytes, partial_bytes;
};

// LLMQ_A16_TILE=wide / narrow in the environment pins the tile shape whatever the problem (read per call; the
// tests run shapes through both).
int forced_shape() {
  const char* v = getenv("LLMQ_A16_TILE");
  if (v == nullptr) return 0;
  return v[0] == 'w' ? 1 : (v[0] == 'n' ? 2 : 0);
}

Plan plan_for(int M, int N, int G, bool narrow = false) {
  Plan p{};
  p.m_tiles = narrow ? (M + Narrow::kBM - 1) / Narrow::kBM : (M + kBM - 1) / kBM;
  p.n_tiles = narrow ? (N + Narrow::kBN - 1) / Narrow::kBN : (N + kBN - 1) / kBN;
  const int tiles = p.m_tiles * p.n_tiles;
  // fewer tiles than would occupy most CUs: cut the reduction axis, at least four groups per slice and no more
  // workgroups than CUs (a workgroup has a CU's LDS to itself: one over is a second round)
  int splits = 1;
  if (tiles < 160) {
    splits = 256 / tiles;
    if (splits > G / 4) splits = G / 4;
    if (splits < 1) splits = 1;
  }
  p.groups_per_split = (G + splits - 1) / splits;
  p.splits = (G + p.groups_per_split - 1) / p.groups_per_split;  // every slice holds at least one group
  // (rows padded to whole wide tiles, which covers whole narrow ones: the kernel reads them without clamping; what
  // the pad rows hold is never stored)
  const size_t padded_rows = static_cast<size_t>((M + kBM - 1) / kBM) * kBM;
  p.xp_bytes = aligned(padded_rows * G * kRowBytes);
  p.rec_bytes = aligned(padded_rows * G * 16);
  p.partial_bytes = p.splits > 1 ? aligned(static_cast<size_t>(p.splits) * M * N * sizeof(float)) : 0;
  return p;
}

// What a plan costs, in microseconds, from the measured shape of a launch: rounds of 256 workgroups, each a fixed
// part (first transfers from memory, the store) plus a time per group of the reduction axis (wide 8 + 1.93 / 2.1 a
// group for int4 / int8, narrow 6 + 0.75 / 1.0), and where the axis is cut the partial tiles' way through memory
// and the second launch (3 us + 8 bytes per partial value at 9 TB/s: most of it overlaps the tiles). Within a
// tenth of the measured launches.
double plan_cost(const Plan& p, int M, int N, bool narrow, bool int4) {
  const double fixed = narrow ? 6.0 : 8.0;
  const double per_group = narrow ? (int4 ? 0.75 : 1.0) : (int4 ? 1.93 : 2.1);
  const int workgroups = p.m_tiles * p.n_tiles * p.splits;
  const double rounds = static_cast<double>((workgroups + 255) / 256);
  double cost = rounds * (fixed + p.groups_per_split * per_group);
  if (p.splits > 1) cost += 3.0 + static_cast<double>(p.splits) * M * N * 8.0 / 9.0e6;
  return cost;
}

// Whether the 64 x 128 tile is the faster one: outputs of few 128 x 256 tiles, where the narrow tile fills the
// chip without cutting the reduction axis (512 x 3072 x 2048 int8: 24.4 us against 29.3; 128 x 14336 x 4096 int4:
// 31.7 / 36.4), and not where its tiles need a second round (1024 x 3072 x 2048: 42.6 / 33.0) or the rows are long
// enough for the wide tile's slices to pay for their partial sums (512 x 4096 x 4096: 41.2 / 37.2).
bool narrow_tile(int M, int N, int G, bool int4) {
  const int forced = forced_shape();
  if (forced) return forced == 2;
  return plan_cost(plan_for(M, N, G, true), M, N, true, int4) < plan_cost(plan_for(M, N, G, false), M, N, false, int4);
}

}  // namespace

extern "C" size_t llmq_wq_gemm_a16_tile_workspace_bytes(int M, int N, int G) {
  if (M <= 0 || N <= 0 || G <= 0) return 0;
  // (the larger of the two shapes' needs: the shape is chosen per call, and may be pinned from the environment)
  const Plan w = plan_for(M, N, G, false), n = plan_for(M, N, G, true);
  return w.xp_bytes + w.rec_bytes + (w.partial_bytes > n.partial_bytes ? w.partial_bytes : n.partial_bytes);
}

namespace {

// The checks the three entry points share; `x` is null when the activation is already prepared.
int check_common(const void* x, bool prepared, const void* qweight, const float* wscale, const void* workspace, int M,
                 int N, int G, int gs, int out_group, int wformat, int dtype) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs != kGroup) return llmq_host::fail_invalid("the tiled fused GEMM needs group_size 128, got %d", gs);
  if (dtype != LLMQ_BF16 && dtype != LLMQ_F16)
    return llmq_host::fail_invalid("the tiled fused GEMM takes bfloat16 or float16 activations, got dtype code %d", dtype);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if ((!prepared && !x) || !qweight || !wscale || !workspace) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return llmq_host::fail_invalid("activation, weight, output and workspace pointers must be 16-byte aligned");
  if ((static_cast<uint64_t>(M) + kBM) * G * kRowBytes >= (1ull << 32))
    return llmq_host::fail_invalid("activation of %d x %d values is beyond the kernel's 32-bit offsets", M, G * kGroup);
  if (static_cast<uint64_t>(N) * G * kGroup >= (1ull << 32))
    return llmq_host::fail_invalid("weight of %d x %d codes is beyond the kernel's 32-bit offsets", N, G * kGroup);
  return 0;
}

int prepare(const void* x, uint8_t* xp, uint8_t* rec, int M, int G, int dtype, hipStream_t s) {
  const int64_t n_chunks = static_cast<int64_t>(M) * G * 16;
  const dim3 grid(static_cast<unsigned>((n_chunks + 255) / 256));
  if (dtype == LLMQ_BF16) {
    hipLaunchKernelGGL(act_prep_kernel<bf16_t>, grid, dim3(256), 0, s, static_cast<const u32x4*>(x),
                       reinterpret_cast<u32x4*>(xp), reinterpret_cast<u32x4*>(rec), n_chunks);
  } else {
    hipLaunchKernelGGL(act_prep_kernel<f16_t>, grid, dim3(256), 0, s, static_cast<const u32x4*>(x),
                       reinterpret_cast<u32x4*>(xp), reinterpret_cast<u32x4*>(rec), n_chunks);
  }
  return llmq_host::check_launch("act_prep_kernel");
}

// The kernel for a weight format, an epilogue and a tile shape, by activation dtype.
template <int EPI, typename S>
int launch_by_type(const TileArgs& a, dim3 grid, int wformat, int dtype, hipStream_t s) {
  const bool int4 = wformat == LLMQ_W_INT4_PACKED;
  if (dtype == LLMQ_BF16) return int4 ? launch_tiles<bf16_t, 4, EPI, S>(a, grid, s) : launch_tiles<bf16_t, 8, EPI, S>(a, grid, s);
  return int4 ? launch_tiles<f16_t, 4, EPI, S>(a, grid, s) : launch_tiles<f16_t, 8, EPI, S>(a, grid, s);
}

// x (or, x null, the prepared activation already in the workspace) times the weight, into out.
int run_store(const void* x, const void* qweight, const float* wscale, void* out, void* workspace,
              size_t workspace_bytes, int M, int N, int G, int gs, int out_group, int wformat, int dtype,
              hipStream_t s) {
  if (int rc = check_common(x, x == nullptr, qweight, wscale, workspace, M, N, G, gs, out_group, wformat, dtype)) return rc;
  if (M == 0 || N == 0) return 0;
  if (!out || (reinterpret_cast<uintptr_t>(out) & 15u)) return llmq_host::fail_invalid("out must be a 16-byte aligned pointer");
  const bool narrow = narrow_tile(M, N, G, wformat == LLMQ_W_INT4_PACKED);
  const Plan p = plan_for(M, N, G, narrow);
  if (workspace_bytes < p.xp_bytes + p.rec_bytes + p.partial_bytes)
    return llmq_host::fail_invalid("workspace of %zu bytes is too small, need %zu", workspace_bytes,
                                   p.xp_bytes + p.rec_bytes + p.partial_bytes);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  uint8_t* xp = ws;
  uint8_t* rec = ws + p.xp_bytes;
  float* partial = reinterpret_cast<float*>(ws + p.xp_bytes + p.rec_bytes);
  if (x != nullptr) {
    if (int rc = prepare(x, xp, rec, M, G, dtype, s)) return rc;
  }
  TileArgs a{xp, rec, static_cast<const uint8_t*>(qweight), wscale, out, partial, M, N, G, out_group,
             p.m_tiles, p.n_tiles, p.splits, p.groups_per_split, nullptr, nullptr, 0};
  const int total = p.m_tiles * p.n_tiles * p.splits;
  const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
  const int rc = narrow ? launch_by_type<kEpiStore, Narrow>(a, grid, wformat, dtype, s)
                        : launch_by_type<kEpiStore, Wide>(a, grid, wformat, dtype, s);
  if (rc) return rc;
  if (p.splits > 1) {
    const int64_t count = static_cast<int64_t>(M) * N;
    const dim3 add_grid(static_cast<unsigned>((count / 4 + 256) / 256));
    if (dtype == LLMQ_BF16) {
      hipLaunchKernelGGL(add_splits_kernel<bf16_t>, add_grid, dim3(256), 0, s, partial, static_cast<bf16_t*>(out), count, p.splits);
    } else {
      hipLaunchKernelGGL(add_splits_kernel<f16_t>, add_grid, dim3(256), 0, s, partial, static_cast<f16_t*>(out), count, p.splits);
    }
    return llmq_host::check_launch("add_splits_kernel");
  }
  return 0;
}

}  // namespace

extern "C" int llmq_wq_gemm_a16_tile(const void* x, const void* qweight, const float* wscale, void* out,
                                     void* workspace, size_t workspace_bytes, int M, int N, int G, int gs,
                                     int out_group, int wformat, int dtype, llmq_stream_t stream) {
  if (M > 0 && N > 0 && !x) return llmq_host::fail_invalid("null tensor pointer");
  return run_store(x, qweight, wscale, out, workspace, workspace_bytes, M, N, G, gs, out_group, wformat, dtype,
                   static_cast<hipStream_t>(stream));
}

extern "C" int llmq_wq_gemm_a16_tile_prepared(const void* qweight, const float* wscale, void* out, void* workspace,
                                              size_t workspace_bytes, int M, int N, int G, int gs, int out_group,
                                              int wformat, int dtype, llmq_stream_t stream) {
  return run_store(nullptr, qweight, wscale, out, workspace, workspace_bytes, M, N, G, gs, out_group, wformat, dtype,
                   static_cast<hipStream_t>(stream));
}

extern "C" size_t llmq_wq_gemm_a16_tile_prepared_bytes(int M, int G) {
  if (M <= 0 || G <= 0) return 0;
  const Plan p = plan_for(M, kBN, G);   // (the prepared part of the workspace does not depend on N)
  return p.xp_bytes + p.rec_bytes;
}

namespace {

// x null: the activation is already in `workspace` in prepared form.
int run_gate_up_silu(const void* x, const void* qweight, const float* wscale, void* workspace, size_t workspace_bytes,
                     void* next_workspace, size_t next_workspace_bytes, int M, int I, int G, int gs, int out_group,
                     int wformat, int dtype, llmq_stream_t stream) {
  if (I < 0 || I > (1 << 29)) return llmq_host::fail_invalid("bad intermediate size %d", I);
  if (int rc = check_common(x, x == nullptr, qweight, wscale, workspace, M, 2 * I, G, gs, out_group, wformat, dtype)) return rc;
  if (M == 0 || I == 0) return 0;
  if (I % (kBN / 2)) return llmq_host::fail_invalid("the intermediate size must be a multiple of %d, got %d", kBN / 2, I);
  if (!next_workspace || (reinterpret_cast<uintptr_t>(next_workspace) & 15u))
    return llmq_host::fail_invalid("next_workspace must be a 16-byte aligned pointer");
  const int next_G = I / kGroup;
  Plan p = plan_for(M, 2 * I, G);
  const Plan next = plan_for(M, kBN, next_G);
  if (workspace_bytes < p.xp_bytes + p.rec_bytes)
    return llmq_host::fail_invalid("workspace of %zu bytes is too small, need %zu", workspace_bytes, p.xp_bytes + p.rec_bytes);
  if (next_workspace_bytes < next.xp_bytes + next.rec_bytes)
    return llmq_host::fail_invalid("next_workspace of %zu bytes is too small, need %zu", next_workspace_bytes,
                                   next.xp_bytes + next.rec_bytes);
  if ((static_cast<uint64_t>(M) + kBM) * next_G * kRowBytes >= (1ull << 32))
    return llmq_host::fail_invalid("activation of %d x %d values is beyond the next GEMM's 32-bit offsets", M, I);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  uint8_t* xp = ws;
  uint8_t* rec = ws + p.xp_bytes;
  if (x != nullptr) {
    if (int rc = prepare(x, xp, rec, M, G, dtype, s)) return rc;
  }
  uint8_t* nws = static_cast<uint8_t*>(next_workspace);
  // whole reduction axis per workgroup: a tile's epilogue needs its finished totals
  TileArgs a{xp, rec, static_cast<const uint8_t*>(qweight), wscale, nullptr, nullptr, M, 2 * I, G, out_group,
             p.m_tiles, I / (kBN / 2), 1, G, nws, nws + next.xp_bytes, next_G};
  const int total = a.m_tiles * a.n_tiles;
  const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
  return launch_by_type<kEpiGateUpSilu, Wide>(a, grid, wformat, dtype, s);
}

}  // namespace

extern "C" int llmq_wq_gemm_a16_tile_gate_up_silu(const void* x, const void* qweight, const float* wscale,
                                                  void* workspace, size_t workspace_bytes, void* next_workspace,
                                                  size_t next_workspace_bytes, int M, int I, int G, int gs,
                                                  int out_group, int wformat, int dtype, llmq_stream_t stream) {
  if (M > 0 && I > 0 && !x) return llmq_host::fail_invalid("null tensor pointer");
  return run_gate_up_silu(x, qweight, wscale, workspace, workspace_bytes, next_workspace, next_workspace_bytes, M, I,
                          G, gs, out_group, wformat, dtype, stream);
}

extern "C" int llmq_wq_gemm_a16_tile_gate_up_silu_prepared(const void* qweight, const float* wscale, void* workspace,
                                                           size_t workspace_bytes, void* next_workspace,
                                                           size_t next_workspace_bytes, int M, int I, int G, int gs,
                                                           int out_group, int wformat, int dtype,
                                                           llmq_stream_t stream) {
  return run_gate_up_silu(nullptr, qweight, wscale, workspace, workspace_bytes, next_workspace, next_workspace_bytes,
                          M, I, G, gs, out_group, wformat, dtype, stream);
}

extern "C" int llmq_add_rmsnorm_prepared(const void* x, const void* delta_or_null, const void* weight,
                                         void* sum_out_or_null, void* workspace, size_t workspace_bytes, int rows,
                                         int hidden, float eps, int dtype, llmq_stream_t stream) {
  if (rows < 0 || hidden <= 0) return llmq_host::fail_invalid("bad dimension rows=%d hidden=%d", rows, hidden);
  if (dtype != LLMQ_BF16 && dtype != LLMQ_F16)
    return llmq_host::fail_invalid("the prepared form is of bfloat16 or float16 activations, got dtype code %d", dtype);
  if (hidden % kGroup) return llmq_host::fail_invalid("hidden must be a multiple of %d, got %d", kGroup, hidden);
  if (rows == 0) return 0;
  if (!x || !weight || !workspace) return llmq_host::fail_invalid("null tensor pointer");
  if ((delta_or_null == nullptr) != (sum_out_or_null == nullptr))
    return llmq_host::fail_invalid("delta and sum_out go together");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(workspace) |
       reinterpret_cast<uintptr_t>(delta_or_null) | reinterpret_cast<uintptr_t>(sum_out_or_null)) & 15u)
    return llmq_host::fail_invalid("tensors and the workspace must be 16-byte aligned");
  const int G = hidden / kGroup;
  if ((static_cast<uint64_t>(rows) + kBM) * G * kRowBytes >= (1ull << 32))
    return llmq_host::fail_invalid("activation of %d x %d values is beyond the tiled GEMM's 32-bit offsets", rows, hidden);
  const Plan p = plan_for(rows, kBN, G);
  if (workspace_bytes < p.xp_bytes + p.rec_bytes)
    return llmq_host::fail_invalid("workspace of %zu bytes is too small, need %zu", workspace_bytes, p.xp_bytes + p.rec_bytes);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  u32x4* xp = reinterpret_cast<u32x4*>(ws);
  u32x4* rec = reinterpret_cast<u32x4*>(ws + p.xp_bytes);
#define LLMQ_NORM_PREP(T, ADD)                                                                                      \
  hipLaunchKernelGGL((rmsnorm_prep_kernel<T, ADD>), dim3(rows), dim3(kNormThreads), 0, s, static_cast<const T*>(x), \
                     static_cast<const T*>(delta_or_null), static_cast<const T*>(weight),                           \
                     static_cast<T*>(sum_out_or_null), xp, rec, hidden, eps)
  if (dtype == LLMQ_BF16) {
    if (delta_or_null) LLMQ_NORM_PREP(bf16_t, true); else LLMQ_NORM_PREP(bf16_t, false);
  } else {
    if (delta_or_null) LLMQ_NORM_PREP(f16_t, true); else LLMQ_NORM_PREP(f16_t, false);
  }
#undef LLMQ_NORM_PREP
  return llmq_host::check_launch("rmsnorm_prep_kernel");
}
