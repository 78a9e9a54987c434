// Weight-only quantized GEMM for a handful to a few dozen activation rows, gfx950: the codes go from
// HBM to the matrix cores without a dense copy of the weight in between.
//
// KernelQuantLinear takes more than KERNEL_MAX_ROWS rows by rebuilding the whole weight in the
// activation dtype and handing it to a dense matmul (llmquant/quantizers/kernel.py:68-79, 88-91): for
// 4-bit codes that is nine times the codes' bytes through HBM (read codes, write 16-bit values, read
// them again), whatever the row count. Here, for 16-bit activations,
//
//   out[m, n] = sum over g of  wscale[sr(n), g] * sum_k x[m, g*128 + k] * code[n, g, k]
//
// the form of RealQuantLinear's weight-only branch (llmquant/quantizers/real.py:84-91): the codes
// are small integers and exact in bf16 / fp16, so the products are exact in the fp32 accumulator of
// v_mfma_f32_16x16x32_{bf16,f16} and the scale is applied once per group. (The reference's dense
// branch rounds code*scale to the activation dtype first; its own test holds the two branches
// together only within a tolerance, tests/test_kernel_linear.py:62-78.)
//
// A workgroup owns 16 or 32 weight rows; its waves split the groups of the reduction axis between them
// (wave w takes groups w, w + waves, ...) and meet in LDS at the end. Per group a wave reads
//   weights   16 rows x 64 B (4-bit) or 128 B (8-bit), 16 or 32 bytes per lane, straight from HBM
//             in operand layout: lane = (row j = lane % 16, block = lane / 16) holds k = 32 block ..
//             32 block + 31, eight of them per MFMA step
//   x         the group's 128 values of every activation row, through the wave's own LDS tile: whole rows
//             go there straight from L2 (global_load_lds_dwordx4: four rows of 256 bytes per instruction, eight
//             cache lines; as operand loads, 64 bytes per lane at a row each, the same bytes were 64 lines per
//             instruction and the address unit, not memory, set the pace), 16-byte slots XOR-swizzled by row,
//             and come out as operands: the 32 k of row (lane % 16) that the lane's codes belong to
// and issues 4 MFMAs per activation tile. The next group's transfer and codes are requested once this group's
// operands are in registers. Rows past M or N are clamped for the loads and dropped at the store, so the load
// sequence is the same for every lane.
#include "llmq_device.h"

namespace {

using namespace llmq;

constexpr int kGroup = 128;
constexpr int kTileN = 16;
constexpr int kTileM = 16;
constexpr int kMaxWaves = 8;
constexpr int kSlabRows = 64;  // activation rows one launch takes (four tiles of 16)

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

struct A16Args {
  const void* x;
  const uint8_t* qw;
  const float* ws;
  void* out;
  int M, N, G, out_group;
  int64_t row_bytes;
};

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  using Vec = v8bf;
  using Elem = __bf16;
  static __device__ __forceinline__ v4f run(Vec a, Vec b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  using Vec = v8h;
  using Elem = _Float16;
  static __device__ __forceinline__ v4f run(Vec a, Vec b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// Eight codes -> eight values of the operand type (exact: |code| <= 128), the signed code itself.
template <typename T, int BITS>
__device__ __forceinline__ typename Mfma16<T>::Vec codes_to_operand(const uint32_t* raw, int step) {
  using E = typename Mfma16<T>::Elem;
  typename Mfma16<T>::Vec v;
  if constexpr (BITS == 4) {
    const uint32_t w = raw[step];  // nibble i: even i is the low nibble of byte i/2, +8 biased
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<E>(static_cast<float>(static_cast<int>((w >> (4 * i)) & 0xfu) - 8));
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[i] = static_cast<E>(static_cast<float>(static_cast<int8_t>(raw[2 * step + i / 4] >> (8 * (i % 4)))));
    }
  }
  return v;
}

template <typename T, int BITS, int MT, int NT>
__global__ __launch_bounds__(kMaxWaves * kWave) void wq_gemm_a16_kernel(const A16Args a) {
  using Vec = typename Mfma16<T>::Vec;
  constexpr int kRaw = BITS == 4 ? 4 : 8;  // dwords of codes per lane per group and row tile
  constexpr bool kBiased = BITS == 4 && MT <= 2;   // codes as biased operands (see multiply)
  constexpr int kRows = NT * kTileN;       // weight rows of the workgroup
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* part = reinterpret_cast<float*>(smem);  // [waves][MT * 16][NT * 16]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wv = tid / kWave;
  const int wk = blockDim.x / kWave;
  const int j = lane & 15;
  const int blk = lane >> 4;
  const int G = a.G;
  const int64_t K = static_cast<int64_t>(G) * kGroup;

  const int n0 = blockIdx.x * kRows;
  const uint8_t* wrow[NT];
  const float* srow[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = min(n0 + nt * kTileN + j, a.N - 1);
    wrow[nt] = a.qw + static_cast<int64_t>(n) * a.row_bytes + blk * (BITS == 4 ? 16 : 32);
    srow[nt] = a.ws + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * G;
  }
  // ---- x of one group: [16 MT rows][16 slots of 16 bytes], slot p of row r holds chunk p ^ (r & 15) ------------
  // transfer i of the wave covers rows 4 i .. 4 i + 3; lane = (row 4 i + lane / 16, slot lane % 16)
  constexpr int kXInstr = MT * 4;
  constexpr int kXTileBytes = MT * kTileM * kGroup * 2;
  unsigned char* xtile = smem + wv * kXTileBytes;
  const unsigned char* xsrc[kXInstr];
#pragma unroll
  for (int i = 0; i < kXInstr; ++i) {
    const int row = 4 * i + (lane >> 4), chunk = (lane & 15) ^ (row & 15);
    xsrc[i] = reinterpret_cast<const unsigned char*>(static_cast<const T*>(a.x) + static_cast<int64_t>(min(row, a.M - 1)) * K +
                                                     chunk * 8);
  }
  auto request_rows = [&](int g) {
#pragma unroll
    for (int i = 0; i < kXInstr; ++i) {
      // (four rows past the activation's end are not fetched: what the tile holds there feeds only result rows
      // that are dropped at the store)
      if (4 * i < a.M) {
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(xsrc[i] + static_cast<int64_t>(g) * (kGroup * 2)),
                                         reinterpret_cast<u32x4*>(xtile + 1024 * i), 16, 0, 0);
      }
    }
  };
  // operand of step s, tile mt: row 16 mt + j, chunk 4 blk + s
  uint32_t x_at[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) x_at[mt] = static_cast<uint32_t>((mt * kTileM + j) * (kGroup * 2));

  struct Weights {
    uint32_t raw[NT][kRaw];
    float scale[NT];
  };
  struct Rows {
    u32x4 xa[MT][4];
  };
  auto load_weights = [&](int g, Weights& W) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const uint8_t* p = wrow[nt] + static_cast<int64_t>(g) * (kGroup * BITS / 8);
#pragma unroll
      for (int q = 0; q < kRaw / 4; ++q) {
        const u32x4 r = load16(p + 16 * q);
        W.raw[nt][4 * q] = r.x; W.raw[nt][4 * q + 1] = r.y; W.raw[nt][4 * q + 2] = r.z; W.raw[nt][4 * q + 3] = r.w;
      }
      W.scale[nt] = srow[nt][g];
    }
  };
  auto read_rows = [&](Rows& X) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(xtile + x_at[mt] + (((4 * blk + s) ^ j) << 4));
        X.xa[mt][s] = kBiased ? interleave_halves(v) : v;
      }
    }
  };

  v4f acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  // int4 codes, up to 32 activation rows: the codes become operands without a conversion per element (BiasedCodes:
  // a nibble placed in the mantissa of 16.0 is the value 16 + n; converting the signed code takes five vector
  // instructions per code, 160 per row tile and group). The matrix core then sums x (code + bias); bias * sum_k x
  // comes out per group through four more MFMAs per activation tile against a vector of ones, shared by the
  // workgroup's row tiles. Measured, 14336 x 4096 int4, M = 8 / 16 / 32: 16.0 / 16.4 / 21.9 -> 13.9 / 14.8 /
  // 20.9 us; with three or four activation tiles the extra MFMAs take back what the conversion saves, and int8
  // codes (a v_cvt_f32_ubyte each for bf16) gain nothing: those keep the signed conversion.
  using Codes = BiasedCodes<T, BITS>;
  uint32_t magic = Codes::kMagic;
  asm volatile("" : "+v"(magic));   // (in a vector register: see and_or)
  const uint32_t one = __builtin_bit_cast(uint16_t, from_float<T>(1.0f));
  const u32x4 ones = {one | (one << 16), one | (one << 16), one | (one << 16), one | (one << 16)};
  auto multiply = [&](const Weights& W, const Rows& X) {
    v4f xsum[MT];   // sum_k x of the group: rows 4 blk + r of tile mt, the same in every column
    if constexpr (kBiased) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        xsum[mt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          xsum[mt] = Mfma16<T>::run(__builtin_bit_cast(Vec, X.xa[mt][s]), __builtin_bit_cast(Vec, ones), xsum[mt]);
        }
      }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      Vec b[4];
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if constexpr (kBiased) b[s] = __builtin_bit_cast(Vec, Codes::operand(W.raw[nt], s, magic));
        else b[s] = codes_to_operand<T, BITS>(W.raw[nt], s);
      }
      const float scale = W.scale[nt];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        v4f d = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < 4; ++s) d = Mfma16<T>::run(__builtin_bit_cast(Vec, X.xa[mt][s]), b[s], d);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float sum = kBiased ? fmaf(-Codes::kBias, xsum[mt][r], d[r]) : d[r];
          acc[nt][mt][r] = fmaf(sum, scale, acc[nt][mt][r]);
        }
      }
    }
  };

  // The wave's groups wv, wv + wk, ...: this group's rows and codes have arrived (nothing else of the wave is in
  // flight), the rows go from the tile to registers, and with the tile free again the next group's transfer
  // and codes are requested, to arrive under this group's multiplications.
  Weights W0, W1;
  if (wv < G) {
    request_rows(wv);
    load_weights(wv, W0);
  }
  auto step = [&](int g, const Weights& now, Weights& next) {
    Rows X;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    read_rows(X);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (g + wk < G) {
      request_rows(g + wk);
      load_weights(g + wk, next);
    }
    multiply(now, X);
  };
  for (int g = wv; g < G; g += 2 * wk) {   // (two groups a round: the register sets swap by name)
    step(g, W0, W1);
    if (g + wk < G) step(g + wk, W1, W0);
  }
  __syncthreads();   // every wave is done with its tile: the partial sums take the same memory

  // ---- waves meet: part[wave][m][n], summed in wave order ---------------------------------------
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        part[(wv * MT * kTileM + mt * kTileM + 4 * blk + r) * kRows + nt * kTileN + j] = acc[nt][mt][r];
      }
  __syncthreads();
  T* __restrict__ out = static_cast<T*>(a.out);
  const int live = min(wk, G);
  for (int e = tid; e < MT * kTileM * kRows; e += blockDim.x) {
    const int m = e / kRows, jj = e % kRows;
    float total = 0.0f;
    for (int w = 0; w < live; ++w) total += part[(w * MT * kTileM + m) * kRows + jj];
    if (m < a.M && n0 + jj < a.N) out[static_cast<int64_t>(m) * a.N + n0 + jj] = from_float<T>(total);
  }
}

template <typename T, int BITS, int MT, int NT>
int launch_tile(const A16Args& a, int wk, hipStream_t stream) {
  const int grid = (a.N + NT * kTileN - 1) / (NT * kTileN);
  // the waves' activation tiles, then (the same memory) their partial sums
  const int part = wk * MT * kTileM * NT * kTileN * static_cast<int>(sizeof(float));
  const int tiles = wk * MT * kTileM * kGroup * 2;
  const int lds = part > tiles ? part : tiles;
  auto kernel = wq_gemm_a16_kernel<T, BITS, MT, NT>;
  if (lds > 64 * 1024) {
    static bool raised = false;  // per instantiation; worst case two threads both set it
    if (!raised) {
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kMaxWaves * MT * kTileM * kGroup * 2);
      if (err != hipSuccess) {
        llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));
        return static_cast<int>(err);
      }
      raised = true;
    }
  }
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(wk * kWave), lds, stream, a);
  return llmq_host::check_launch("wq_gemm_a16_kernel");
}

template <typename T, int BITS>
int launch_typed(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G, int out_group,
                 hipStream_t stream) {
  const int64_t K = static_cast<int64_t>(G) * kGroup;
  int wk = G < kMaxWaves ? G : kMaxWaves;
  // rows of few groups: two groups per wave at least
  if (G >= 4 && wk * 2 > G) wk = G / 2;
  // Two row tiles per workgroup share the activation rows a wave loads (the activation comes from L2
  // once per workgroup: 16 rows per workgroup make that traffic four times the codes' at M = 16),
  // as long as a workgroup per CU and more is left. Measured, M = 8 / 64, 14336 x 4096 int4:
  // 21 / 86 us with one tile, 17 / 48 us with two; 4096 x 4096: 7 / 23 against 9 / 24.
  const bool wide = N >= 2 * kTileN * 256;
  // (Sixteen waves for few row tiles of long rows, down_proj, measured no faster than eight.)
  for (int m0 = 0; m0 < M; m0 += kSlabRows) {
    A16Args a{};
    a.x = static_cast<const T*>(x) + static_cast<int64_t>(m0) * K;
    a.qw = static_cast<const uint8_t*>(qw);
    a.ws = ws;
    a.out = static_cast<T*>(out) + static_cast<int64_t>(m0) * N;
    a.M = M - m0 < kSlabRows ? M - m0 : kSlabRows;
    a.N = N; a.G = G; a.out_group = out_group;
    a.row_bytes = K * BITS / 8;
    const int mt = (a.M + kTileM - 1) / kTileM;
    int rc;
    if (wide) {
      switch (mt) {
        case 1: rc = launch_tile<T, BITS, 1, 2>(a, wk, stream); break;
        case 2: rc = launch_tile<T, BITS, 2, 2>(a, wk, stream); break;
        case 3: rc = launch_tile<T, BITS, 3, 2>(a, wk, stream); break;
        default: rc = launch_tile<T, BITS, 4, 2>(a, wk, stream); break;
      }
    } else {
      switch (mt) {
        case 1: rc = launch_tile<T, BITS, 1, 1>(a, wk, stream); break;
        case 2: rc = launch_tile<T, BITS, 2, 1>(a, wk, stream); break;
        case 3: rc = launch_tile<T, BITS, 3, 1>(a, wk, stream); break;
        default: rc = launch_tile<T, BITS, 4, 1>(a, wk, stream); break;
      }
    }
    if (rc) return rc;
  }
  return 0;
}

}  // namespace

extern "C" int llmq_wq_gemm_a16(const void* x, const void* qweight, const float* wscale, void* out, int M, int N,
                                int G, int gs, int out_group, int wformat, int dtype, llmq_stream_t stream) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs != kGroup) return llmq_host::fail_invalid("the fused GEMM needs group_size 128, got %d", gs);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("the fused GEMM takes float16 or bfloat16 activations, got dtype code %d", dtype);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!x || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qweight)) & 15u)
    return llmq_host::fail_invalid("x and qweight must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == LLMQ_BF16) {
    return wformat == LLMQ_W_INT8 ? launch_typed<bf16_t, 8>(x, qweight, wscale, out, M, N, G, out_group, s)
                                  : launch_typed<bf16_t, 4>(x, qweight, wscale, out, M, N, G, out_group, s);
  }
  return wformat == LLMQ_W_INT8 ? launch_typed<f16_t, 8>(x, qweight, wscale, out, M, N, G, out_group, s)
                                : launch_typed<f16_t, 4>(x, qweight, wscale, out, M, N, G, out_group, s);
}
