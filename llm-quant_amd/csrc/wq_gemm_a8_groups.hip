// The exact integer prefill GEMM for outputs with too few tiles to fill the chip, gfx950.
//
//   out[m, n] = sum over groups g, IN ORDER, of  ((float)(sum_k a[m,g,k] * q[n,g,k]) * sw[sr(n),g]) * sx[m,g]
//
// -- the A8 branch of RealQuantLinear.forward (llmquant/quantizers/real.py:76-103), bit for bit, as
// wq_gemm_a8.hip computes it. What is fixed by that arithmetic is the order of the fp32 ADDITIONS; the terms
//   p[m, n, g] = fl(fl(float(isum) * sw) * sx)
// do not depend on one another. A workgroup that walks the groups of its tile one after the other (as the tiled
// kernel does) is a chain of G dependent steps, each a load -> multiply -> scale round trip, and with few tiles
// (M = 128 against a weight of a few thousand rows) the chip waits on 128 such chains: 64 us for 112 groups.
//
// Here the eight waves of a workgroup take DIFFERENT groups of the same 32 x 32 output tile: in round r, wave w
// computes p for group 8 r + w (operands of its own, nothing shared, no barrier: loaded as whole rows a round
// ahead and turned into matrix-core operand layout through the wave's LDS slot) and leaves the 32 x 32 fp32 terms
// in that slot; the round ends with one barrier, and during the NEXT round (whose terms go to a second set of
// slots) every wave adds, for its eighth of the tile, slot 0, slot 1, ... slot 7 of the round before onto its
// running totals: the additions happen in group order, one at a time, exactly as in the serial walk, under the
// next round's loads and multiplies. A tile's chain is G / 8 rounds long. Cost: every term crosses LDS once
// (8 bytes per output and group).
//
// Operand layout. v_mfma_i32_32x32x32_i8 takes from lane l: row l % 32, sixteen k-values of half l / 32. A lane
// owns one half of a group's 128 k-values (64 contiguous bytes of a row of activations, 32 bytes of packed
// weights); a sum over k does not care about the order inside the half as long as both operands agree on it.
// Packed int4: a 32-bit word w of eight codes gives (w << 4 & 0xf0f0f0f0) ^ 0x80808080 = the even codes and
// (w & 0xf0f0f0f0) ^ 0x80808080 = the odd codes as signed bytes 16 * code (the 16 leaves through the weight
// scale, a power of two: no rounding changes); the activation bytes are brought into the same even / odd order
// with one byte permute per word.
//
// Activation codes in operand order (TILED_A). Turning the activation rows into operand layout through LDS is two
// fifths of a round's LDS traffic and, for packed weights, sixteen byte permutes per wave. The quantizer that makes
// the codes can write them where the matrix core wants them instead (act_quant_tiled_kernel): blocks of 32 rows x
// one group (4 KB) in the order [m-tile][group], inside a block [k-step 0..3][lane 0..63][16 bytes], lane = row %
// 32 + 32 * k-half, and for packed weights every eight bytes as even k, then odd k. A wave then loads its operand
// with four contiguous 1 KB instructions and multiplies it as it comes.
#include "llmq_device.h"

namespace {

using namespace llmq;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGroup = 128;
constexpr int kWaysLog2 = 3;
constexpr int kWays = 1 << kWaysLog2;       // waves of a workgroup = groups of a round
constexpr int kThreads = kWays * kWave;
constexpr int kTM = 32, kTN = 32;           // output tile of a workgroup (and of every wave)
constexpr int kSlotFloats = kTM * kTN;      // one wave's terms of one group

constexpr int kBlockBytes = kTM * kGroup;   // activation codes of 32 rows x one group

struct GroupArgs {
  const int8_t* a;     // [M, G*128], or (TILED_A) [ceil(M / 32)][G][4096] in operand order
  const float* sx;     // [M, G]
  const uint8_t* qw;   // [N, G, 128] int8 or [N, G, 64] packed
  const float* sw;     // [scale_rows, G]
  const float* bias;   // [N] or null
  void* out;           // [M, N]
  int M, N, G, out_group;
};

// What a wave holds of one group between its loads and its multiply: the 16-byte packets of its operand tiles as
// they lie in memory. Packet p = 64 i + lane of the activation tile is row p / 8, piece p % 8 (eight whole rows of
// 128 bytes per load instruction); of the weight tile, row p / 4, piece p % 4 (int4: 64 bytes a row) or row p / 8,
// piece p % 8 (int8). Loading straight in operand layout instead (lane = row, 16 bytes of it) touches 32 cache
// lines per instruction, and the address unit then sets the pace (measured: 4x slower).
template <int BITS> struct Operands {
  u32x4 ra[4];
  u32x4 rb[BITS == 8 ? 4 : 2];
};

constexpr int kChunkGroups = 16;   // groups whose scales sit in LDS at a time (two such chunks: one in use, one coming)



template <typename T, int BITS, bool TILED_A>
__device__ __forceinline__ void groups_body(const GroupArgs& g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* slots = reinterpret_cast<float*>(smem);                       // [2][kWays][kSlotFloats]: rounds alternate
  float* s_sx = slots + 2 * kWays * kSlotFloats;                       // [2][kChunkGroups][kTM]: chunks alternate
  float* s_sw = s_sx + 2 * kChunkGroups * kTM;                         // [2][kChunkGroups][kTN]

  const int tid = threadIdx.x, lane = tid & (kWave - 1), wv = tid >> 6;
  const int col = lane & 31, half = lane >> 5;
  const int m0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
  const uint32_t k_total = static_cast<uint32_t>(g.G) * kGroup;
  const uint32_t w_row_bytes = BITS == 8 ? k_total : k_total / 2;
  constexpr int kBPackets = BITS == 8 ? 4 : 2;
  constexpr int kGroupBytesB = BITS == 8 ? kGroup : kGroup / 2;

  // byte offsets of the lane's packets in group 0 (rows past the end clamped: loaded, never stored); the host
  // has checked that both operands are smaller than 4 GB
  uint32_t a_off[4], b_off[kBPackets];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int p = i * kWave + lane;
    a_off[i] = static_cast<uint32_t>(min(m0 + (p >> 3), g.M - 1)) * k_total + (p & 7) * 16;
  }
#pragma unroll
  for (int i = 0; i < kBPackets; ++i) {
    const int p = i * kWave + lane;
    const int row = BITS == 8 ? p >> 3 : p >> 2, piece = BITS == 8 ? p & 7 : p & 3;
    b_off[i] = static_cast<uint32_t>(min(n0 + row, g.N - 1)) * w_row_bytes + piece * 16;
  }
  const uint32_t a_block0 = static_cast<uint32_t>(blockIdx.y) * g.G * kBlockBytes + lane * 16;   // (TILED_A)
  auto load = [&](Operands<BITS>& o, int grp) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (TILED_A) o.ra[i] = load16(g.a + (a_block0 + static_cast<uint32_t>(grp) * kBlockBytes + i * 1024));
      else o.ra[i] = load16(g.a + (a_off[i] + static_cast<uint32_t>(grp) * kGroup));
    }
#pragma unroll
    for (int i = 0; i < kBPackets; ++i) o.rb[i] = load16(g.qw + (b_off[i] + static_cast<uint32_t>(grp) * kGroupBytesB));
  };

  // The tile's scales, kChunkGroups groups at a time, as [group][row] and [group][column]: a thread reads one of
  // each a chunk ahead (16 consecutive groups of a row are half a cache line) and puts them into the buffer that
  // the chunk before the current one used, during the current chunk's last round (a barrier after every round
  // separates that from the buffer's last reader and from its first).
  static_assert(kThreads == kChunkGroups * kTM && kTM == kTN, "one activation scale and one weight scale a thread");
  float pre_sx, pre_sw;
  auto load_chunk = [&](int chunk) {
    // (groups past the end: clamped, so that the loads are unconditional; those values are never multiplied with)
    const int row = tid / kChunkGroups, grp = min(chunk * kChunkGroups + tid % kChunkGroups, g.G - 1);
    const int n = min(n0 + row, g.N - 1);
    pre_sx = g.sx[static_cast<int64_t>(min(m0 + row, g.M - 1)) * g.G + grp];
    pre_sw = g.sw[static_cast<int64_t>(g.out_group > 0 ? n / g.out_group : n) * g.G + grp];
  };
  auto store_chunk = [&](int chunk) {
    const int at = (chunk & 1) * kChunkGroups * kTM + (tid % kChunkGroups) * kTM + tid / kChunkGroups;
    s_sx[at] = pre_sx;
    // (the unpacked nibbles are 16 x their codes: the 16 leaves here, exactly)
    s_sw[at] = BITS == 4 ? pre_sw * 0.0625f : pre_sw;
  };

  // One group's terms into this wave's slot. The slot (4 KB) first serves as the wave's staging area, for the
  // activations and then for the weights: the packets go in as whole rows (16-byte pieces XOR-swizzled by row, so
  // that neither the writes nor the operand reads collide on banks) and come back out in operand layout: lane
  // (row or column `col`, k-half `half`) reads its pieces. LDS serves a wave's accesses in order; the wave
  // barriers keep the compiler from moving them.
  // Result register r of the 32 x 32 product is row 8 (r / 4) + 4 half + r % 4, column col; the slot keeps the
  // terms as [r / 2][lane][r % 2]: the pair of registers that one wave adds lies contiguous over the lanes, so
  // that both the stores here and the adders' 8-byte reads spread over all banks.
  auto produce = [&](const Operands<BITS>& o, int grp, float* round_slots) {
    unsigned char* stage = reinterpret_cast<unsigned char*>(round_slots + wv * kSlotFloats);
    // piece `piece` of 128-byte line `line`, XOR-swizzled
    // (by line / 2: the sixteen lanes that LDS serves together read one piece of sixteen different lines, or of
    // eight lines and two pieces four apart (packed weights), and a line's parity is already a bank bit)
    auto piece_at = [](int line, int piece) { return line * 128 + ((piece ^ ((line >> 1) & 7)) << 4); };
    // packet 64 i + lane is piece lane % 8 of line 8 i + lane / 8: one address; eight lines on, the swizzle's third
    // bit has flipped
    auto put_at = [&](int i) { return stage + ((piece_at(lane >> 3, lane & 7) ^ ((i & 1) << 6)) + i * 1024); };
    v4i fa[4];
    if constexpr (TILED_A) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        fa[ks] = v4i{static_cast<int>(o.ra[ks].x), static_cast<int>(o.ra[ks].y), static_cast<int>(o.ra[ks].z), static_cast<int>(o.ra[ks].w)};
    } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) store16(put_at(i), o.ra[i]);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const u32x4 d = load16(stage + piece_at(col, 4 * half + ks));
      if constexpr (BITS == 8) {
        fa[ks] = v4i{static_cast<int>(d.x), static_cast<int>(d.y), static_cast<int>(d.z), static_cast<int>(d.w)};
      } else {
        // even bytes, odd bytes of each pair of words: the order the unpacked nibbles come in
        fa[ks] = v4i{static_cast<int>(__builtin_amdgcn_perm(d.y, d.x, 0x06040200u)),
                     static_cast<int>(__builtin_amdgcn_perm(d.y, d.x, 0x07050301u)),
                     static_cast<int>(__builtin_amdgcn_perm(d.w, d.z, 0x06040200u)),
                     static_cast<int>(__builtin_amdgcn_perm(d.w, d.z, 0x07050301u))};
      }
    }
    __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int i = 0; i < kBPackets; ++i) store16(put_at(i), o.rb[i]);   // int4: 64-byte rows, two to a line
    __builtin_amdgcn_wave_barrier();
    v4i fb[4];
    if constexpr (BITS == 8) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const u32x4 w = load16(stage + piece_at(col, 4 * half + ks));
        fb[ks] = v4i{static_cast<int>(w.x), static_cast<int>(w.y), static_cast<int>(w.z), static_cast<int>(w.w)};
      }
    } else {
      // the lane's column: packets 4 col + 2 half + {0, 1} of the staged tile (neighbours in one line: the second
      // address is the first with bit 4 flipped)
      const int q = col * 4 + 2 * half;
      const int at = piece_at(q >> 3, q & 7);
      const u32x4 lo = load16(stage + at), hi = load16(stage + (at ^ 16));
      const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const uint32_t w0 = w[2 * ks], w1 = w[2 * ks + 1];
        fb[ks] = v4i{static_cast<int>(((w0 << 4) & 0xf0f0f0f0u) ^ 0x80808080u), static_cast<int>((w0 & 0xf0f0f0f0u) ^ 0x80808080u),
                     static_cast<int>(((w1 << 4) & 0xf0f0f0f0u) ^ 0x80808080u), static_cast<int>((w1 & 0xf0f0f0f0u) ^ 0x80808080u)};
      }
    }
    // every operand is in registers: the staging area becomes the slot
    __builtin_amdgcn_wave_barrier();
    v16i d = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) d = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks], fb[ks], d, 0, 0, 0);
    float* slot = round_slots + wv * kSlotFloats;
    const int gl = grp & (2 * kChunkGroups - 1);   // (chunk parity, group in the chunk)
    const float sw = s_sw[gl * kTN + col];
#pragma unroll
    for (int r4 = 0; r4 < 4; ++r4) {
      const u32x4 s4 = *reinterpret_cast<const u32x4*>(&s_sx[gl * kTM + 8 * r4 + 4 * half]);
      const float sx4[4] = {__builtin_bit_cast(float, s4.x), __builtin_bit_cast(float, s4.y),
                            __builtin_bit_cast(float, s4.z), __builtin_bit_cast(float, s4.w)};
      float p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float f = static_cast<float>(d[4 * r4 + i]);
        f = f * sw;
        p[i] = f * sx4[i];
      }
      *reinterpret_cast<u32x2*>(slot + ((2 * r4) * kWave + lane) * 2) =
          u32x2{__builtin_bit_cast(uint32_t, p[0]), __builtin_bit_cast(uint32_t, p[1])};
      *reinterpret_cast<u32x2*>(slot + ((2 * r4 + 1) * kWave + lane) * 2) =
          u32x2{__builtin_bit_cast(uint32_t, p[2]), __builtin_bit_cast(uint32_t, p[3])};
    }
  };

  // this wave's eighth of the tile in the additions: result registers 4 (wv / 2) + 2 (wv % 2) + {0, 1} of every lane
  float total[2] = {0.0f, 0.0f};
  const int my_pair = (wv * kWave + lane) * 2;
  auto add_round = [&](const float* round_slots, int valid) {
    for (int s = 0; s < valid; ++s) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(round_slots + s * kSlotFloats + my_pair);
      total[0] = total[0] + __builtin_bit_cast(float, v.x);
      total[1] = total[1] + __builtin_bit_cast(float, v.y);
    }
  };

  const int rounds = (g.G + kWays - 1) >> kWaysLog2;
  const int full = g.G >> kWaysLog2;   // rounds in which every wave has a group
  constexpr int kRoundsPerChunk = kChunkGroups / kWays;
  Operands<BITS> cur, nxt;
  if (wv < g.G) load(cur, wv);
  load_chunk(0);
  store_chunk(0);
  load_chunk(1);   // (past the last group: clamped loads whose values are never stored)
  __syncthreads();   // the first chunk's scales are in place
  // in the last round of a chunk the next chunk goes into the other buffer, and the one after it is requested
  auto turn_chunk = [&](int r) {
    if ((r + 1) % kRoundsPerChunk == 0 && r + 1 < rounds) {
      store_chunk((r + 1) / kRoundsPerChunk);
      load_chunk((r + 1) / kRoundsPerChunk + 1);
    }
  };
  auto slots_of = [&](int r) { return slots + (r & 1) * kWays * kSlotFloats; };
  int r = 0;
  // Round r: request the next round's operands, multiply this round's group into slots_of(r), add the terms of
  // round r - 1 out of slots_of(r - 1), one barrier. (The barrier publishes this round's terms and ends the reads of
  // the other set, which the next round overwrites.)
  // Steady state: this round's and the next round's group exist for every wave, so nothing branches around the
  // loads and the compiler's waits before the staging stores count exactly the loads that may stay in flight
  // (a branch around them makes it drain the next round's loads before this round's multiply). The operand set
  // is copied at the end of a round (two rounds per trip with the sets swapping roles needs 57 more registers).
  if (r + 1 < full) {   // the first round has nothing to add yet
    load(nxt, wv + kWays);
    produce(cur, wv, slots_of(0));
    turn_chunk(0);
    __syncthreads();
    cur = nxt;
    r = 1;
  }
  for (; r + 1 < full; ++r) {
    const int grp = r * kWays + wv;
    load(nxt, grp + kWays);
    produce(cur, grp, slots_of(r));
    add_round(slots_of(r - 1), kWays);
    turn_chunk(r);
    __syncthreads();
    cur = nxt;
  }
  for (; r < rounds; ++r) {
    const int grp = r * kWays + wv;
    const bool more = grp + kWays < g.G;
    if (more) load(nxt, grp + kWays);
    if (grp < g.G) produce(cur, grp, slots_of(r));
    if (r > 0) add_round(slots_of(r - 1), kWays);   // (a round before the last is a full one)
    turn_chunk(r);
    __syncthreads();
    if (more) cur = nxt;
  }
  if (rounds > 0) add_round(slots_of(rounds - 1), min(kWays, g.G - (rounds - 1) * kWays));

  T* __restrict__ out = static_cast<T*>(g.out);
  const int n = n0 + col;
  if (n < g.N) {
    const float b = g.bias != nullptr ? g.bias[n] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = m0 + 8 * (wv >> 1) + 4 * half + 2 * (wv & 1) + i;
      if (m < g.M) {
        const float v = g.bias != nullptr ? total[i] + b : total[i];
        out[static_cast<int64_t>(m) * g.N + n] = from_float<T>(v);
      }
    }
  }
}

// Packed int4 weights: held to 128 registers (eight spilled, all outside the steady loop's multiply), so that two
// workgroups (sixteen waves) share a CU and one's additions run under the other's multiplies: 128 x 4096 x 14336
// in 41 us against 47 us with one workgroup a CU. int8 weights would spill 31: that form runs one workgroup a CU.
template <typename T, bool TILED_A>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void wq_gemm_a8_groups_kernel4(const GroupArgs g) {
  groups_body<T, 4, TILED_A>(g);
}
template <typename T, bool TILED_A>
__global__ __launch_bounds__(kThreads) void wq_gemm_a8_groups_kernel8(const GroupArgs g) {
  groups_body<T, 8, TILED_A>(g);
}

// The activation quantizer of llmq_quant_group_codes (int8 codes, group 128: csrc/fake_quant.hip, quant_lanes_kernel:
// the same abs-max butterfly, IEEE division and round-half-even per group of 16 lanes) writing its codes in operand
// order. A lane holds eight consecutive values of a (row, group); EVEN_ODD: for packed int4 weights.
template <typename T, bool EVEN_ODD>
__global__ __launch_bounds__(256) void act_quant_tiled_kernel(const T* __restrict__ x, int8_t* __restrict__ codes,
                                                              float* __restrict__ scale_out, const int64_t total,
                                                              const uint32_t K) {
  const int64_t e0 = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  const bool active = e0 < total;   // total is a multiple of 128: the 16 lanes of a group are active or idle as one
  float f[8];
  if (active) {
    Pack<T>::unpack(load16(x + e0), f);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = 0.0f;
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(f[i]));
  amax = group_max<16>(amax);
  const float scale = scale_from_amax(amax, 127.0f);
  if (!active) return;
  const uint32_t G = K / kGroup;
  const uint32_t row = static_cast<uint32_t>(e0 / K), in_row = static_cast<uint32_t>(e0 - static_cast<int64_t>(row) * K);
  const uint32_t grp = in_row / kGroup, j = (in_row % kGroup) / 8;   // j: which eight of the group's 128
  if (j == 0) scale_out[static_cast<int64_t>(row) * G + grp] = scale;
  uint32_t c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = static_cast<uint32_t>(static_cast<int>(quant_code(f[i], scale, -128.0f, 127.0f))) & 0xffu;
  u32x2 w;
  if constexpr (EVEN_ODD) {
    w.x = c[0] | c[2] << 8 | c[4] << 16 | c[6] << 24;
    w.y = c[1] | c[3] << 8 | c[5] << 16 | c[7] << 24;
  } else {
    w.x = c[0] | c[1] << 8 | c[2] << 16 | c[3] << 24;
    w.y = c[4] | c[5] << 8 | c[6] << 16 | c[7] << 24;
  }
  // k = 8 j .. 8 j + 7: k-half j / 8, k-step (j % 8) / 2, first or second eight bytes of the lane's sixteen
  const int64_t block = (static_cast<int64_t>(row / kTM) * G + grp) * kBlockBytes;
  const uint32_t at = ((j & 7) >> 1) * 1024 + ((row % kTM) + 32 * (j >> 3)) * 16 + (j & 1) * 8;
  *reinterpret_cast<u32x2*>(codes + block + at) = w;
}

constexpr size_t kLdsBytes = 2 * (static_cast<size_t>(kWays) * kSlotFloats + kChunkGroups * (kTM + kTN)) * sizeof(float);

template <typename T, int BITS, bool TILED_A>
int launch(const GroupArgs& g, hipStream_t stream) {
  auto kernel = BITS == 4 ? wq_gemm_a8_groups_kernel4<T, TILED_A> : wq_gemm_a8_groups_kernel8<T, TILED_A>;
  static bool raised = false;  // per instantiation; worst case two threads both set it
  if (!raised) {
    const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (err != hipSuccess) {
      llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));
      return static_cast<int>(err);
    }
    raised = true;
  }
  const dim3 grid((g.N + kTN - 1) / kTN, (g.M + kTM - 1) / kTM), block(kThreads);
  hipLaunchKernelGGL(kernel, grid, block, kLdsBytes, stream, g);
  return llmq_host::check_launch("wq_gemm_a8_groups_kernel");
}

}  // namespace

namespace llmq_host {

// Whether the group-parallel form can take the problem: it addresses both operands with 32-bit byte offsets.
bool gemm_a8_groups_supported(int M, int N, int G) {
  const uint64_t k_total = static_cast<uint64_t>(G) * kGroup;
  return static_cast<uint64_t>(M) * k_total < (1ull << 32) && static_cast<uint64_t>(N) * k_total < (1ull << 32);
}

int gemm_a8_groups(const int8_t* a, const float* sx, const void* qweight, const float* wscale,
                   const float* bias_or_null, void* out, int M, int N, int G, int out_group, int wformat, int dtype,
                   hipStream_t stream, bool tiled_a) {
  GroupArgs g{a, sx, static_cast<const uint8_t*>(qweight), wscale, bias_or_null, out, M, N, G, out_group};
#define LLMQ_GO(T)                                                                                       \
  (tiled_a ? (wformat == LLMQ_W_INT8 ? launch<T, 8, true>(g, stream) : launch<T, 4, true>(g, stream))   \
           : (wformat == LLMQ_W_INT8 ? launch<T, 8, false>(g, stream) : launch<T, 4, false>(g, stream)))
  switch (dtype) {
    case LLMQ_F32: return LLMQ_GO(float);
    case LLMQ_F16: return LLMQ_GO(f16_t);
    case LLMQ_BF16: return LLMQ_GO(bf16_t);
  }
#undef LLMQ_GO
  return fail_invalid("out must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

}  // namespace llmq_host

extern "C" size_t llmq_act_codes_tiled_bytes(int M, int K) {
  if (M <= 0 || K <= 0) return 0;
  return static_cast<size_t>((M + kTM - 1) / kTM) * kTM * static_cast<size_t>(K);
}

extern "C" int llmq_quant_act_codes_tiled(const void* x, void* codes, float* scale, int M, int K, int wformat,
                                          int dtype, llmq_stream_t stream) {
  if (M < 0 || K <= 0 || K % kGroup) return llmq_host::fail_invalid("bad shape M=%d K=%d (K a multiple of %d)", M, K, kGroup);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (dtype != LLMQ_BF16 && dtype != LLMQ_F16)
    return llmq_host::fail_invalid("x must be bfloat16 or float16, got dtype code %d", dtype);
  if (M == 0) return 0;
  if (!x || !codes || !scale) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(codes)) & 15u)
    return llmq_host::fail_invalid("x and codes must be 16-byte aligned");
  if (!llmq_host::gemm_a8_groups_supported(M + kTM, 1, K / kGroup))
    return llmq_host::fail_invalid("activation of %d x %d codes is beyond the kernel's 32-bit offsets", M, K);
  const int64_t total = static_cast<int64_t>(M) * K;
  const dim3 grid(static_cast<unsigned>((total / 8 + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool even_odd = wformat == LLMQ_W_INT4_PACKED;
#define LLMQ_GO(T)                                                                                               \
  if (even_odd) hipLaunchKernelGGL((act_quant_tiled_kernel<T, true>), grid, block, 0, s, static_cast<const T*>(x), \
                                   static_cast<int8_t*>(codes), scale, total, static_cast<uint32_t>(K));          \
  else hipLaunchKernelGGL((act_quant_tiled_kernel<T, false>), grid, block, 0, s, static_cast<const T*>(x),         \
                          static_cast<int8_t*>(codes), scale, total, static_cast<uint32_t>(K))
  if (dtype == LLMQ_BF16) { LLMQ_GO(bf16_t); } else { LLMQ_GO(f16_t); }
#undef LLMQ_GO
  return llmq_host::check_launch("act_quant_tiled_kernel");
}

extern "C" int llmq_wq_gemm_a8_tiled(const void* codes_tiled, const float* sx, const void* qweight, const float* wscale,
                                     const float* bias_or_null, void* out, int M, int N, int G, int gs, int out_group,
                                     int wformat, int dtype, llmq_stream_t stream) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs != kGroup) return llmq_host::fail_invalid("the integer GEMM needs group_size 128, got %d", gs);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!codes_tiled || !sx || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(codes_tiled) | reinterpret_cast<uintptr_t>(qweight)) & 15u)
    return llmq_host::fail_invalid("codes and qweight must be 16-byte aligned");
  if (!llmq_host::gemm_a8_groups_supported(M + kTM, N, G))
    return llmq_host::fail_invalid("operands of %d x %d and %d x %d codes are beyond the kernel's 32-bit offsets", M,
                                   G * kGroup, N, G * kGroup);
  return llmq_host::gemm_a8_groups(static_cast<const int8_t*>(codes_tiled), sx, qweight, wscale, bias_or_null, out, M, N,
                                   G, out_group, wformat, dtype, static_cast<hipStream_t>(stream), true);
}
