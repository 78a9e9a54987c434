// Integer prefill GEMM on the int8 matrix core (v_mfma_i32_32x32x32_i8), gfx950: int8
// activations (quantized per token x group) times int4 / int8 group-quantized weights.
//
//   out[m, n] = sum over groups g, in order, of  ((float)(sum_k a[m,g,k] * q[n,g,k]) * sw[sr(n),g]) * sx[m,g]
//
// This is the A8 branch of RealQuantLinear.forward (llmquant/quantizers/real.py:76-103) with
// its rounding points kept: the group's integer sum is exact (128 * 127 * 127 < 2^24), it is
// converted to fp32, multiplied by the weight scale, then by the activation scale, then added
// to the running fp32 total -- four separately rounded operations, in group order. The file is
// built with -ffp-contract=off so no multiply-add is fused; results equal the reference's
// real mode bit for bit.
//
// Shape. A workgroup (4 waves) owns a 128 x 128 output tile (64 x 64 when the problem has too
// few tiles to fill the chip; the text below describes the large one) and walks K one group
// (128) at a time. Activations [M, K] int8 and weights [N, K(/2)] are staged in LDS, weights unpacked
// there to signed int8 in natural k order (packed int4: 16 x (nibble - 8) by a mask and a sign-bit
// flip per four codes, the 16 folded into the weight scale; even/odd nibbles re-interleaved with
// v_perm). Each wave
// computes a 64 x 64 quadrant as 2 x 2 MFMA tiles of 32 x 32 (A = activations, rows m;
// B = weights, columns n), 4 k-slabs of 32 per group. The next group's global loads are in
// flight while the current one is multiplied. After each group the int32 sums go through the
// scale epilogue above: four vector-ALU operations per output element per group, against 256
// multiply-adds on the matrix core, which makes the vector ALU the unit that bounds this
// kernel (two waves per SIMD, so that one wave's epilogue runs under the other's MFMAs).
//
// MODE. 0 is the arithmetic above, bit for bit. 1 and 2 are the tolerance forms behind llmq_wq_gemm_a8_fast:
// the same exact integer group sums, folded in with fewer vector instructions: 1: fma((float)isum * sw, sx,
// total), three per output and group instead of four; 2: one activation scale per token (sx[M]), which
// leaves the sum over groups: fma((float)isum, sw, total), two, and the token's scale once at the store.
#include <stdlib.h>

#include <type_traits>

#include "llmq_device.h"

namespace {

using namespace llmq;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;
constexpr int kThreads = 256;
constexpr int kRowStride = kGroup + 16;  // bytes; padding keeps 16-byte reads off the same banks
// the group-parallel kernel (exact form) takes outputs of up to this many 32 x 32 tiles per round of 256 of the
// tiled kernel's 64 x 64 tiles
constexpr int kLargeTileMin = 300;   // 128 x 128 tiles from this many up (256 CUs)
constexpr int kGroupsTilesPerRound = 640;
constexpr int kGroupsTilesOperandOrder = 1100;   // (512 x 4096 x 14336, 2048 tiles: 101 us against 82 tiled)

struct GemmArgs {
  const int8_t* a;     // [M, G*128]
  const float* sx;     // [M, G]; MODE 2: [M]
  const uint8_t* qw;   // [N, G, 128] int8 or [N, G, 64] packed
  const float* sw;     // [scale_rows, G]
  const float* bias;   // [N] or null
  void* out;           // [M, N]
  int M, N, G, out_group;
};

// a 32-bit offset the compiler must take as it is, inside the loop: the load then has the form scalar base +
// vector offset, and the base moves from group to group with two scalar additions instead of one 64-bit vector
// addition per load
__device__ __forceinline__ uint32_t here(uint32_t& v) {
  asm volatile("" : "+v"(v));  // (in place: a copy would cost a move per load)
  return v;
}

// W: the wave's quadrant is (32 W) x (32 W), the workgroup's tile (64 W) x (64 W). W = 2 is the
// throughput shape; W = 1 gives four times as many workgroups when the problem is too small to
// fill the chip with 128 x 128 tiles.
template <typename T, int BITS, int W, int MODE>
__global__ __launch_bounds__(kThreads, 2) void wq_gemm_a8_kernel(const GemmArgs g) {
  constexpr int kBM = 64 * W, kBN = 64 * W;
  __shared__ __attribute__((aligned(16))) int8_t s_a[2][kBM * kRowStride];
  __shared__ __attribute__((aligned(16))) int8_t s_b[2][kBN * kRowStride];
  __shared__ __attribute__((aligned(16))) float s_scale[2][kBM + kBN];  // activation scales, then weight scales

  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wv >> 1, wn = wv & 1;  // quadrant of the tile
  const int m0 = blockIdx.y * kBM, n0 = blockIdx.x * kBN;
  const int64_t k_total = static_cast<int64_t>(g.G) * kGroup;
  const int64_t w_row_bytes = BITS == 8 ? k_total : k_total / 2;
  constexpr int kWGroupBytes = BITS == 8 ? kGroup : kGroup / 2;

  // ---- staging: who loads what ------------------------------------------------------------------
  // A tile: kBM rows x 128 B = 8 kBM 16-byte packets. Thread t: packets t + 256*i:
  // row = p / 8, piece = p % 8.
  // B tile int8: same. B tile int4: kBN rows x 64 B = 4 kBN packets: row = p / 4.
  // Addresses are the tile's first row (the same in every lane) plus an offset per thread that does not change
  // from group to group (at most 128 rows: 32 bits hold it, the host checks the row length).
  constexpr int kAPackets = kBM * 8 / kThreads;
  constexpr int kBPackets = (BITS == 8 ? kBN * 8 : kBN * 4) / kThreads;
  const int8_t* a_tile = g.a + static_cast<int64_t>(m0) * k_total;
  const uint8_t* b_tile = g.qw + static_cast<int64_t>(n0) * w_row_bytes;
  uint32_t a_off[kAPackets], b_off[kBPackets];
#pragma unroll
  for (int i = 0; i < kAPackets; ++i) {
    const int p = tid + kThreads * i;
    a_off[i] = static_cast<uint32_t>(min(p >> 3, g.M - 1 - m0)) * static_cast<uint32_t>(k_total) + (p & 7) * 16;
  }
#pragma unroll
  for (int i = 0; i < kBPackets; ++i) {
    const int p = tid + kThreads * i;
    const int row = min(BITS == 8 ? p >> 3 : p >> 2, g.N - 1 - n0);
    b_off[i] = static_cast<uint32_t>(row) * static_cast<uint32_t>(w_row_bytes) + (BITS == 8 ? (p & 7) : (p & 3)) * 16;
  }
  // One scale per thread and group: the first kBM / 64 waves load activation scales, the others weight scales
  // (waves past the tile's rows and columns, and the first ones in MODE 2, which has no activation scale per
  // group, repeat a weight scale's address): a fixed number of loads per group lets the waits before the LDS
  // stores count the loads that may stay in flight instead of draining them all.
  const bool sx_wave = MODE != 2 && wv < kBM / 64;
  const int sc_idx = wv < kBM / 64 ? tid : (tid - kBM) & (kBN - 1);
  auto scale_row = [&](int n) { return g.out_group > 0 ? n / g.out_group : n; };
  const char* sc_tile = sx_wave ? reinterpret_cast<const char*>(g.sx + static_cast<int64_t>(m0) * g.G)
                                : reinterpret_cast<const char*>(g.sw + static_cast<int64_t>(scale_row(n0)) * g.G);
  uint32_t sc_off =
      static_cast<uint32_t>(sx_wave ? min(sc_idx, g.M - 1 - m0) : scale_row(min(n0 + sc_idx, g.N - 1)) - scale_row(n0)) *
      static_cast<uint32_t>(g.G) * 4u;
  const float scale_factor = BITS == 4 && wv >= kBM / 64 ? 0.0625f : 1.0f;  // see the unpack of packed weights
  // LDS addresses of a thread's first packets; the others are whole rows further on
  const int a_lds = (tid >> 3) * kRowStride + (tid & 7) * 16;
  const int b_lds = BITS == 8 ? a_lds : (tid >> 2) * kRowStride + (tid & 3) * 32;
  constexpr int kARowsPerPass = kThreads / 8, kBRowsPerPass = BITS == 8 ? kThreads / 8 : kThreads / 4;

  // what a thread holds of one group between its global loads and its LDS stores
  struct Staged {
    u32x4 ra[kAPackets], rb[kBPackets];
    float r_s;
  };
  // The small tile has little work per group, so with one group in flight its loop runs at one
  // memory round trip per iteration: it keeps two register sets and requests a group three
  // iterations before it is multiplied. The large tile has no registers for that: it requests the
  // next group at the top of an iteration and moves it to LDS at the bottom.
  constexpr int kAhead = W == 1 ? 2 : 0;
  constexpr int kSets = kAhead > 0 ? kAhead : 1;
  Staged st[kSets];

  auto load_group = [&](int grp, Staged& t) {
    const int8_t* ag = a_tile + static_cast<uint32_t>(grp) * kGroup;
#pragma unroll
    for (int i = 0; i < kAPackets; ++i) t.ra[i] = load16(ag + here(a_off[i]));
    const uint8_t* bg = b_tile + static_cast<uint32_t>(grp) * kWGroupBytes;
#pragma unroll
    for (int i = 0; i < kBPackets; ++i) t.rb[i] = load16(bg + here(b_off[i]));
    t.r_s = *reinterpret_cast<const float*>(sc_tile + static_cast<uint32_t>(grp) * 4 + here(sc_off));
  };
  auto store_group = [&](auto buffer, const Staged& t) {
    constexpr int buf = decltype(buffer)::value;
#pragma unroll
    for (int i = 0; i < kAPackets; ++i) store16(&s_a[buf][a_lds + i * kARowsPerPass * kRowStride], t.ra[i]);
#pragma unroll
    for (int i = 0; i < kBPackets; ++i) {
      int8_t* dst = &s_b[buf][b_lds + i * kBRowsPerPass * kRowStride];
      if constexpr (BITS == 8) {
        store16(dst, t.rb[i]);
      } else {
        // 16 packed bytes = 32 codes -> 32 signed bytes in natural k order, each 16 x its code:
        // a nibble n = code + 8 moved to the top of its byte and its top bit flipped reads, as a
        // signed byte, 16 (n - 8). The factor 16 leaves the integer sums exact (< 2^26) and is
        // taken back out of the weight scale, a power of two, so no rounding changes.
        const uint32_t w[4] = {t.rb[i].x, t.rb[i].y, t.rb[i].z, t.rb[i].w};
        uint32_t o[8];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t lo = ((w[d] << 4) & 0xf0f0f0f0u) ^ 0x80808080u;  // codes k = 8d + {0,2,4,6}
          const uint32_t hi = (w[d] & 0xf0f0f0f0u) ^ 0x80808080u;         // codes k = 8d + {1,3,5,7}
          // bytes (lo0, hi0, lo1, hi1) and (lo2, hi2, lo3, hi3); v_perm selects from {hi:lo}
          o[2 * d] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
          o[2 * d + 1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
        }
        store16(dst, u32x4{o[0], o[1], o[2], o[3]});
        store16(dst + 16, u32x4{o[4], o[5], o[6], o[7]});
      }
    }
    if (kBM + kBN == kThreads || wv < (kBM + kBN) / 64) s_scale[buf][tid] = t.r_s * scale_factor;
  };

  float acc[W][W][16];
#pragma unroll
  for (int mi = 0; mi < W; ++mi)
#pragma unroll
    for (int ni = 0; ni < W; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

  load_group(0, st[0]);
  store_group(std::integral_constant<int, 0>{}, st[0]);
  __syncthreads();
#pragma unroll
  for (int a = 0; a < kAhead; ++a) {
    if (1 + a < g.G) load_group(1 + a, st[a]);  // st[a] will hold groups 1 + a, 1 + a + kAhead, ...
  }

  const int frag = (lane & 31) * kRowStride + (lane >> 5) * 16;  // a lane's row and k half within a 32-row block
  // One group: multiply it from LDS buffer `buffer` (= grp & 1, a compile-time value so that every LDS address
  // is a register plus a constant), move group grp + 1 (in `next`) into the other buffer, and with kAhead > 0
  // request group grp + 1 + kAhead into the registers that frees. `steady`: the caller guarantees that groups
  // grp + 1 and grp + 1 + kAhead exist, so the body has no branch around its loads and stores.
  auto iterate = [&](int grp, Staged& next, auto buffer, auto steady) {
    constexpr int buf = decltype(buffer)::value;
    constexpr bool kSteady = decltype(steady)::value;
    if (kAhead == 0 && (kSteady || grp + 1 < g.G)) load_group(grp + 1, next);  // in flight during the MFMAs below

    v4i fa[W][kGroup / 32], fb[kGroup / 32];
#pragma unroll
    for (int mi = 0; mi < W; ++mi)
#pragma unroll
      for (int ks = 0; ks < kGroup / 32; ++ks)
        fa[mi][ks] = *reinterpret_cast<const v4i*>(&s_a[buf][(wm * W + mi) * 32 * kRowStride + frag + ks * 32]);
    auto load_b = [&](int ni) {
#pragma unroll
      for (int ks = 0; ks < kGroup / 32; ++ks)
        fb[ks] = *reinterpret_cast<const v4i*>(&s_b[buf][(wn * W + ni) * 32 * kRowStride + frag + ks * 32]);
    };
    auto multiply = [&](int mi) {
      v16i d = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      __builtin_amdgcn_s_setprio(3);  // the wave that feeds the matrix core goes first; epilogues fill in
#pragma unroll
      for (int ks = 0; ks < kGroup / 32; ++ks) d = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[mi][ks], fb[ks], d, 0, 0, 0);
      __builtin_amdgcn_s_setprio(0);
      return d;
    };
    // result register r of a 32 x 32 tile is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
    auto scale_in = [&](const v16i& d, int mi, int ni) {
      const float sw = s_scale[buf][kBM + (wn * W + ni) * 32 + (lane & 31)];
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        // four consecutive rows: one 128-bit LDS read of their activation scales
        const int row = (wm * W + mi) * 32 + 8 * r4 + 4 * (lane >> 5);
        const u32x4 s4 = MODE == 2 ? u32x4{0, 0, 0, 0} : *reinterpret_cast<const u32x4*>(&s_scale[buf][row]);
        const float sx4[4] = {__builtin_bit_cast(float, s4.x), __builtin_bit_cast(float, s4.y),
                              __builtin_bit_cast(float, s4.z), __builtin_bit_cast(float, s4.w)};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float f = static_cast<float>(d[4 * r4 + i]);
          if constexpr (MODE == 0) {
            f = f * sw;
            f = f * sx4[i];
            acc[mi][ni][4 * r4 + i] = acc[mi][ni][4 * r4 + i] + f;
          } else if constexpr (MODE == 1) {
            acc[mi][ni][4 * r4 + i] = fmaf(f * sw, sx4[i], acc[mi][ni][4 * r4 + i]);
          } else {
            acc[mi][ni][4 * r4 + i] = fmaf(f, sw, acc[mi][ni][4 * r4 + i]);
          }
        }
      }
    };
    load_b(0);
    if constexpr (W == 2) {
      // All sixteen multiplies of the group first, then the next group's unpacking and LDS stores (its loads
      // were requested at the top and have had the multiplies to arrive in), then the four epilogues: the LDS
      // stores are long done when the epilogue reaches the barrier. Measured against the epilogues between the
      // multiplies and against the stores after the epilogues or before the multiplies: the orders differ by a
      // few percent, this one is the best on most shapes. The empty instructions pin it: left alone the compiler
      // arrives at the same order but runs out of registers on the way (32 spilled with int8 weights).
      v16i d0 = multiply(0);
      v16i d1 = multiply(1);
      load_b(1);
      v16i d2 = multiply(0);
      v16i d3 = multiply(1);
      asm volatile("" : "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3));
      if (kSteady || grp + 1 < g.G) store_group(std::integral_constant<int, buf ^ 1>{}, next);
      asm volatile("" : "+v"(d0), "+v"(d1), "+v"(d2), "+v"(d3));
      scale_in(d0, 0, 0);
      scale_in(d1, 1, 0);
      scale_in(d2, 0, 1);
      scale_in(d3, 1, 1);
    } else {
      scale_in(multiply(0), 0, 0);
    }

    if constexpr (W != 2) {
      if (kSteady || grp + 1 < g.G) store_group(std::integral_constant<int, buf ^ 1>{}, next);  // nobody reads that buffer any more: see barrier below
      if (kAhead > 0 && (kSteady || grp + 1 + kAhead < g.G)) load_group(grp + 1 + kAhead, next);
    }
    __syncthreads();
  };
  // Two groups a trip, one per LDS buffer. Steady state: every group a trip touches exists (the last one is
  // grp + 1 + 1 + kAhead), so its bodies have no branch around their loads and stores and the compiler waits
  // for exactly the loads an LDS store needs instead of draining everything in flight.
  int grp = 0;
  for (; grp + 2 + kAhead < g.G; grp += 2) {
    iterate(grp, st[0], std::integral_constant<int, 0>{}, std::true_type{});
    iterate(grp + 1, st[kSets - 1], std::integral_constant<int, 1>{}, std::true_type{});
  }
  for (; grp < g.G; grp += 2) {
    iterate(grp, st[0], std::integral_constant<int, 0>{}, std::false_type{});
    if (grp + 1 < g.G) iterate(grp + 1, st[kSets - 1], std::integral_constant<int, 1>{}, std::false_type{});
  }

  T* __restrict__ out = static_cast<T*>(g.out);
#pragma unroll
  for (int ni = 0; ni < W; ++ni) {
    const int n = n0 + (wn * W + ni) * 32 + (lane & 31);
    const float b = (g.bias != nullptr && n < g.N) ? g.bias[n] : 0.0f;
#pragma unroll
    for (int mi = 0; mi < W; ++mi) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + (wm * W + mi) * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (m < g.M && n < g.N) {
          if constexpr (MODE == 2) acc[mi][ni][r] *= g.sx[m];
          const float v = g.bias != nullptr ? acc[mi][ni][r] + b : acc[mi][ni][r];
          out[static_cast<int64_t>(m) * g.N + n] = from_float<T>(v);
        }
      }
    }
  }
}

template <typename T, int W, int MODE>
int launch_tile(const GemmArgs& g, int wformat, hipStream_t stream) {
  constexpr int kTile = 64 * W;
  const dim3 grid((g.N + kTile - 1) / kTile, (g.M + kTile - 1) / kTile), block(kThreads);
  // (the kernel addresses a tile's rows with 32-bit offsets from its first row)
  if (g.G > (1 << 17)) return llmq_host::fail_invalid("rows of more than 2^24 codes are not supported, got %d groups", g.G);
  if (wformat == LLMQ_W_INT8) {
    hipLaunchKernelGGL((wq_gemm_a8_kernel<T, 8, W, MODE>), grid, block, 0, stream, g);
  } else {
    hipLaunchKernelGGL((wq_gemm_a8_kernel<T, 4, W, MODE>), grid, block, 0, stream, g);
  }
  return llmq_host::check_launch("wq_gemm_a8_kernel");
}

// LLMQ_A8_FORM=tile / groups in the environment pins the exact GEMM to the tiled kernels or to the group-parallel
// kernel (wq_gemm_a8_groups.hip) whatever the shape: the two are bit-identical, and the tests run every shape
// through both. Read per call.
int forced_form() {
  const char* v = getenv("LLMQ_A8_FORM");
  if (v == nullptr) return 0;
  return v[0] == 't' ? 1 : (v[0] == 'g' ? 2 : 0);
}

// The exact form: a tile's groups are a chain of dependent steps, and with few tiles the chip waits on few
// chains. The group-parallel kernel computes eight groups of a 32 x 32 tile at once and only orders the
// additions (same bits).
// Which is faster, measured on 32-group and 112-group rows at M = 128 ... 2048 (int4): the tiled kernel takes
// ~0.57 us per group and round of 256 of its 64 x 64 tiles, this one ~0.7 ns per group and 32 x 32 tile (it pays
// for staging and unpacking per wave): it wins where the output is a few hundred 32 x 32 tiles and the rows are
// long -- 128 x 4096 x 14336: 38 us against 61; 128 x 14336 x 4096: 38 against 27, which stays tiled.
// operand_order: the activation codes come in the group-parallel kernel's operand order (llmq_wq_gemm_a8_tiled):
// ~0.5 ns per group and tile then, 128 x 4096 x 14336 in 30 us, and on long rows it stays ahead up to about a
// thousand tiles (256 x 4096 x 14336: 55 us against 64).
bool takes_groups(int M, int N, int G, bool operand_order = false) {
  const int form = forced_form();
  const int64_t big_tiles = static_cast<int64_t>((N + 127) / 128) * ((M + 127) / 128);
  const int64_t tiles32 = static_cast<int64_t>((N + 31) / 32) * ((M + 31) / 32);
  const int64_t tiles64 = static_cast<int64_t>((N + 63) / 64) * ((M + 63) / 64);
  bool pays = big_tiles < 256 && G >= 16 && tiles32 <= kGroupsTilesPerRound * ((tiles64 + 255) / 256);
  if (operand_order && G >= 64 && tiles32 <= kGroupsTilesOperandOrder) pays = true;
  return (form == 2 || (form == 0 && pays)) && llmq_host::gemm_a8_groups_supported(M, N, G);
}

template <typename T, int MODE>
int launch_typed(const GemmArgs& g, int wformat, hipStream_t stream) {
  // 128 x 128 tiles when there are clearly more of them than CUs, else 64 x 64
  const int64_t big_tiles = static_cast<int64_t>((g.N + 127) / 128) * ((g.M + 127) / 128);
  if constexpr (MODE == 0) {
    if (takes_groups(g.M, g.N, g.G)) {
      const int dtype = sizeof(T) == 4 ? LLMQ_F32 : (std::is_same<T, f16_t>::value ? LLMQ_F16 : LLMQ_BF16);
      return llmq_host::gemm_a8_groups(g.a, g.sx, g.qw, g.sw, g.bias, g.out, g.M, g.N, g.G, g.out_group, wformat, dtype,
                                       stream);
    }
  }
  // (measured, bit-exact form, int4: 256 large tiles, one a CU: 53.7 us against 48.9 on 64 x 64 tiles at 1024 x 4096 x
  // 4096 and 52.6 against 47.8 at 512 x 8192 x 4096; 336 large tiles: 61.1 against 68.2; 448: 77.3 against 87.5)
  return big_tiles >= kLargeTileMin ? launch_tile<T, 2, MODE>(g, wformat, stream) : launch_tile<T, 1, MODE>(g, wformat, stream);
}

template <int MODE>
int launch_mode(const GemmArgs& g, int wformat, int dtype, hipStream_t s) {
  switch (dtype) {
    case LLMQ_F32: return launch_typed<float, MODE>(g, wformat, s);
    case LLMQ_F16: return launch_typed<f16_t, MODE>(g, wformat, s);
    case LLMQ_BF16: return launch_typed<bf16_t, MODE>(g, wformat, s);
  }
  return llmq_host::fail_invalid("out must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

}  // namespace

extern "C" int llmq_wq_gemm_a8(const int8_t* a, const float* sx, const void* qweight,
                               const float* wscale, const float* bias_or_null, void* out, int M,
                               int N, int G, int gs, int out_group, int wformat, int dtype,
                               llmq_stream_t stream) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs != kGroup) return llmq_host::fail_invalid("the integer GEMM needs group_size 128, got %d", gs);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!a || !sx || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(qweight)) & 15u)
    return llmq_host::fail_invalid("activation and weight pointers must be 16-byte aligned");
  GemmArgs g{a, sx, static_cast<const uint8_t*>(qweight), wscale, bias_or_null, out, M, N, G, out_group};
  return launch_mode<0>(g, wformat, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int llmq_wq_gemm_a8_takes_groups(int M, int N, int G) {
  return M > 0 && N > 0 && G > 0 && takes_groups(M, N, G, true) ? 1 : 0;
}

// The tolerance forms of the same kernel (arguments already checked by llmq_wq_gemm_a8_fast).
int llmq_host::gemm_a8_relaxed(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                               const float* bias_or_null, void* out, int M, int N, int G, bool token_scale,
                               int out_group, int wformat, int dtype, hipStream_t stream) {
  GemmArgs g{a, sx, static_cast<const uint8_t*>(qweight), wscale, bias_or_null, out, M, N, G, out_group};
  return token_scale ? launch_mode<2>(g, wformat, dtype, stream) : launch_mode<1>(g, wformat, dtype, stream);
}
