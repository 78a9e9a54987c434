// Weight-only quantized GEMM for a few dozen activation rows, the reduction axis split across
// workgroups: the form that keeps the bytes a CU pulls in close to the codes' own.
//
// Same sum as llmq_wq_gemm_a16 (wq_gemm_a16.hip):
//   out[m, n] = sum over g of  wscale[sr(n), g] * sum_k x[m, g*128 + k] * code[n, g, k]
// There a workgroup owns 16-32 weight rows and the whole reduction axis, so every workgroup reads
// all of x from L2: at M = 16 that is twice the bytes of 4-bit codes, at M = 64 eight times, and the
// time follows the bytes the CUs pull in (~6 TB/s), not HBM. Here a workgroup owns 128 weight rows
// (8 waves x 16) and a slice of four groups (512 k) of the reduction axis:
//   1  every wave requests its codes of the four groups (16 or 32 bytes per lane and group, MFMA
//      operand layout straight from HBM) -- all of the workgroup's HBM traffic, in flight at once
//   2  the workgroup copies its slice of x, [16 MT rows][512] 16-bit values, into LDS once (16-byte
//      slots, XOR-swizzled by row so that the operand reads below are conflict-free)
//   3  per group: codes -> operand type (as unsigned integers for up to 32 rows, see codes_to_operand),
//      activation operands from LDS, 4 (+ 4) MFMAs per activation tile, acc += (d - bias * sum x) * scale
//   4  the slice's fp32 sums go to a workspace [slices][M][N]; a second launch adds the slices in
//      order and casts (a fixed order: the result does not depend on which workgroup finished
//      first). One slice: the result is written directly and there is no second launch.
// x traffic falls from (N/32) M K 2 bytes to (N/128) M K 2, and a launch has N/128 * G/4
// workgroups whatever the shape (896 for both Llama-3-8B MLP shapes).
#include "llmq_device.h"

namespace {

using namespace llmq;

constexpr int kGroup = 128;
constexpr int kTileN = 16;
constexpr int kTileM = 16;
constexpr int kWaves = 8;
constexpr int kRowsPerBlock = kWaves * kTileN;  // 128 weight rows
constexpr int kSliceGroups = 4;                 // groups of the reduction axis per workgroup
constexpr int kSliceSlots = kSliceGroups * kGroup / 8;  // 16-byte slots per activation row and slice: 64
constexpr int kSlabRows = 64;

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

struct SplitArgs {
  const void* x;
  const uint8_t* qw;
  const float* ws;
  void* out;
  float* partial;  // [slices][M][N], unused with one slice
  int M, N, G, out_group, n_slices;
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

// Eight codes -> eight values of the operand type, as UNSIGNED integers: a 4-bit code is stored with a
// bias of 8 (0..15), an 8-bit code is taken with its sign bit flipped (code + 128, 0..255). Both are
// exact in bf16 and fp16, and unsigned bytes convert in one instruction each (v_cvt_f32_ubyteN)
// where the signed form costs a sign extension or a subtraction per element; the bias is taken out
// after the multiplication, sum_k x_k (u_k - B) = sum_k x_k u_k - B sum_k x_k, with sum_k x_k from
// one more MFMA against a vector of ones (the matrix cores are idle most of the time here, the
// vector ALU is not). The bias is small beside the codes' own spread, so the subtraction costs
// no precision to speak of.
template <int BITS> constexpr float kCodeBias = BITS == 4 ? 8.0f : 128.0f;

template <typename T> __device__ __forceinline__ uint32_t pack_exact(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack_exact<bf16_t>(float lo, float hi) {
  // integers below 256: the upper halves of the two floats are the bf16 values, exactly
  return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x07060302u);
}
template <> __device__ __forceinline__ uint32_t pack_exact<f16_t>(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));  // exact below 2048
}

// (With three or four activation tiles the extra MFMAs cost more than the conversion saves -- measured,
// 14336 x 4096 at M = 64: 43.8 us against 36.6 us -- so those sizes convert the signed code itself.)
template <int MT> constexpr bool kBiasedCodes = MT <= 2;

template <typename T, int BITS, bool BIASED>
__device__ __forceinline__ typename Mfma16<T>::Vec codes_to_operand(const uint32_t* raw, int step) {
  if constexpr (!BIASED) {
    using E = typename Mfma16<T>::Elem;
    typename Mfma16<T>::Vec v;
    if constexpr (BITS == 4) {
      const uint32_t w = raw[step];
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
  uint32_t out[4];
  if constexpr (BITS == 4) {
    const uint32_t w = raw[step];  // nibble i: even i is the low nibble of byte i/2
    const uint32_t even = w & 0x0f0f0f0fu, odd = (w >> 4) & 0x0f0f0f0fu;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      out[p] = pack_exact<T>(static_cast<float>((even >> (8 * p)) & 0xffu), static_cast<float>((odd >> (8 * p)) & 0xffu));
    }
  } else {
    const uint32_t w0 = raw[2 * step] ^ 0x80808080u, w1 = raw[2 * step + 1] ^ 0x80808080u;
    out[0] = pack_exact<T>(static_cast<float>(w0 & 0xffu), static_cast<float>((w0 >> 8) & 0xffu));
    out[1] = pack_exact<T>(static_cast<float>((w0 >> 16) & 0xffu), static_cast<float>(w0 >> 24));
    out[2] = pack_exact<T>(static_cast<float>(w1 & 0xffu), static_cast<float>((w1 >> 8) & 0xffu));
    out[3] = pack_exact<T>(static_cast<float>((w1 >> 16) & 0xffu), static_cast<float>(w1 >> 24));
  }
  return __builtin_bit_cast(typename Mfma16<T>::Vec, u32x4{out[0], out[1], out[2], out[3]});
}

template <typename T> __device__ __forceinline__ typename Mfma16<T>::Vec ones_operand() {
  const uint32_t one2 = pack_exact<T>(1.0f, 1.0f);
  return __builtin_bit_cast(typename Mfma16<T>::Vec, u32x4{one2, one2, one2, one2});
}

template <typename T, int BITS, int MT>
__global__ __launch_bounds__(kWaves * kWave) void wq_gemm_a16_split_kernel(const SplitArgs a) {
  using Vec = typename Mfma16<T>::Vec;
  constexpr int kRaw = BITS == 4 ? 4 : 8;  // dwords of codes per lane per group
  constexpr int kRowsM = MT * kTileM;
  __shared__ __attribute__((aligned(16))) u32x4 xs[kRowsM * kSliceSlots];  // 16 KB per activation tile

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wv = tid / kWave;
  const int j = lane & 15;
  const int blk = lane >> 4;
  const int G = a.G;
  const int64_t K = static_cast<int64_t>(G) * kGroup;
  const int g0 = blockIdx.y * kSliceGroups;
  const int groups = min(kSliceGroups, G - g0);  // >= 1 by the grid

  // ---- 1: the wave's codes and scales of the slice -------------------------------------------------
  const int n0 = (blockIdx.x * kWaves + wv) * kTileN;
  const int n = min(n0 + j, a.N - 1);
  const uint8_t* wrow = a.qw + static_cast<int64_t>(n) * a.row_bytes + blk * (BITS == 4 ? 16 : 32);
  const float* srow = a.ws + static_cast<int64_t>(a.out_group > 0 ? n / a.out_group : n) * G;
  uint32_t raw[kSliceGroups][kRaw];
  float scale[kSliceGroups];
#pragma unroll
  for (int gi = 0; gi < kSliceGroups; ++gi) {
    const int g = min(g0 + gi, G - 1);  // (a slice past the row's end repeats its last group, weighted by zero)
    const uint8_t* p = wrow + static_cast<int64_t>(g) * (kGroup * BITS / 8);
#pragma unroll
    for (int q = 0; q < kRaw / 4; ++q) {
      const u32x4 r = load16(p + 16 * q);
      raw[gi][4 * q] = r.x; raw[gi][4 * q + 1] = r.y; raw[gi][4 * q + 2] = r.z; raw[gi][4 * q + 3] = r.w;
    }
    scale[gi] = srow[g];
  }

  // ---- 2: the slice of x into LDS, slot s of row r at position s ^ (r & 15) ---------------------------
  const T* xbase = static_cast<const T*>(a.x) + static_cast<int64_t>(g0) * kGroup;
  const int slots_here = groups * (kGroup / 8);
#pragma unroll
  for (int i = 0; i < kRowsM * kSliceSlots / (kWaves * kWave); ++i) {
    const int idx = i * (kWaves * kWave) + tid;
    const int row = idx / kSliceSlots, slot = idx % kSliceSlots;
    u32x4 v{0u, 0u, 0u, 0u};
    if (slot < slots_here) v = load16(xbase + static_cast<int64_t>(min(row, a.M - 1)) * K + slot * 8);
    xs[row * kSliceSlots + (slot ^ (row & 15))] = v;
  }
  __syncthreads();

  // ---- 3: multiply ------------------------------------------------------------------------------------
  v4f acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  const Vec ones = ones_operand<T>();
#pragma unroll
  for (int gi = 0; gi < kSliceGroups; ++gi) {
    Vec b[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) b[s] = codes_to_operand<T, BITS, kBiasedCodes<MT>>(raw[gi], s);
    const float sc = gi < groups ? scale[gi] : 0.0f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int row = mt * kTileM + j;
      v4f d = v4f{0.0f, 0.0f, 0.0f, 0.0f}, xsum = v4f{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        // lane (j, blk), step s: x[row][32 blk + 8 s .. + 7] of group gi = slot 16 gi + 4 blk + s
        const u32x4 xa = xs[row * kSliceSlots + ((gi * 16 + blk * 4 + s) ^ (row & 15))];
        d = Mfma16<T>::run(__builtin_bit_cast(Vec, xa), b[s], d);
        if constexpr (kBiasedCodes<MT>) xsum = Mfma16<T>::run(__builtin_bit_cast(Vec, xa), ones, xsum);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float sum = kBiasedCodes<MT> ? fmaf(-kCodeBias<BITS>, xsum[r], d[r]) : d[r];
        acc[mt][r] = fmaf(sum, sc, acc[mt][r]);
      }
    }
  }

  // ---- 4: lane (j, blk) holds rows 4 blk + r of each activation tile, column n0 + j ------------------
  if (n0 + j < a.N) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = mt * kTileM + 4 * blk + r;
        if (m < a.M) {
          const int64_t at = static_cast<int64_t>(m) * a.N + n0 + j;
          if (a.n_slices == 1) static_cast<T*>(a.out)[at] = from_float<T>(acc[mt][r]);
          else a.partial[static_cast<int64_t>(blockIdx.y) * a.M * a.N + at] = acc[mt][r];
        }
      }
    }
  }
}

// out[i] = T(sum over the slices, in order, of partial[s][i]); four elements per thread.
template <typename T>
__global__ __launch_bounds__(256) void wq_gemm_a16_reduce_kernel(const float* __restrict__ partial, T* __restrict__ out,
                                                                  const int64_t count, const int n_slices) {
  const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i0 >= count) return;
  if (i0 + 4 <= count) {  // count * 4 bytes and the slices' offsets keep 16-byte alignment when count % 4 == 0
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if ((count & 3) == 0) {
      // eight slices' loads in flight at a time (a loop that waits for each costs a round trip per
      // slice: 28 of them for a 14336-wide reduction axis); added in slice order all the same
      for (int k0 = 0; k0 < n_slices; k0 += 8) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load16(partial + min(k0 + u, n_slices - 1) * count + i0);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (k0 + u < n_slices) {
            s[0] += __builtin_bit_cast(float, v[u].x); s[1] += __builtin_bit_cast(float, v[u].y);
            s[2] += __builtin_bit_cast(float, v[u].z); s[3] += __builtin_bit_cast(float, v[u].w);
          }
        }
      }
    } else {
      for (int k = 0; k < n_slices; ++k) {
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] += partial[k * count + i0 + e];
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) out[i0 + e] = from_float<T>(s[e]);
    return;
  }
  for (int64_t i = i0; i < count; ++i) {
    float s = 0.0f;
    for (int k = 0; k < n_slices; ++k) s += partial[k * count + i];
    out[i] = from_float<T>(s);
  }
}

int slices_of(int G) { return (G + kSliceGroups - 1) / kSliceGroups; }

template <typename T, int BITS>
int launch_typed(const void* x, const void* qw, const float* ws, void* out, float* workspace, int M, int N, int G,
                 int out_group, hipStream_t stream) {
  const int64_t K = static_cast<int64_t>(G) * kGroup;
  const int n_slices = slices_of(G);
  const dim3 grid((N + kRowsPerBlock - 1) / kRowsPerBlock, n_slices), block(kWaves * kWave);
  for (int m0 = 0; m0 < M; m0 += kSlabRows) {
    SplitArgs a{};
    a.x = static_cast<const T*>(x) + static_cast<int64_t>(m0) * K;
    a.qw = static_cast<const uint8_t*>(qw);
    a.ws = ws;
    a.out = static_cast<T*>(out) + static_cast<int64_t>(m0) * N;
    a.partial = workspace;
    a.M = M - m0 < kSlabRows ? M - m0 : kSlabRows;
    a.N = N; a.G = G; a.out_group = out_group; a.n_slices = n_slices;
    a.row_bytes = K * BITS / 8;
    switch ((a.M + kTileM - 1) / kTileM) {
      case 1: hipLaunchKernelGGL((wq_gemm_a16_split_kernel<T, BITS, 1>), grid, block, 0, stream, a); break;
      case 2: hipLaunchKernelGGL((wq_gemm_a16_split_kernel<T, BITS, 2>), grid, block, 0, stream, a); break;
      case 3: hipLaunchKernelGGL((wq_gemm_a16_split_kernel<T, BITS, 3>), grid, block, 0, stream, a); break;
      default: hipLaunchKernelGGL((wq_gemm_a16_split_kernel<T, BITS, 4>), grid, block, 0, stream, a); break;
    }
    if (int rc = llmq_host::check_launch("wq_gemm_a16_split_kernel")) return rc;
    if (n_slices > 1) {
      const int64_t count = static_cast<int64_t>(a.M) * N;
      const int blocks = static_cast<int>((count + 1023) / 1024);
      hipLaunchKernelGGL((wq_gemm_a16_reduce_kernel<T>), dim3(blocks), dim3(256), 0, stream, workspace,
                         static_cast<T*>(a.out), count, n_slices);
      if (int rc = llmq_host::check_launch("wq_gemm_a16_reduce_kernel")) return rc;
    }
  }
  return 0;
}

}  // namespace

extern "C" size_t llmq_wq_gemm_a16_workspace_bytes(int M, int N, int G) {
  if (M <= 0 || N <= 0 || G <= 0) return 0;
  const int n_slices = slices_of(G);
  if (n_slices == 1) return 0;
  const size_t rows = M < kSlabRows ? M : kSlabRows;
  return static_cast<size_t>(n_slices) * rows * static_cast<size_t>(N) * sizeof(float);
}

extern "C" int llmq_wq_gemm_a16_split(const void* x, const void* qweight, const float* wscale, void* out,
                                      void* workspace, size_t workspace_bytes, int M, int N, int G, int gs,
                                      int out_group, int wformat, int dtype, llmq_stream_t stream) {
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
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return llmq_host::fail_invalid("x, qweight and the workspace must be 16-byte aligned");
  const size_t need = llmq_wq_gemm_a16_workspace_bytes(M, N, G);
  if (need > 0 && (!workspace || workspace_bytes < need))
    return llmq_host::fail_invalid("the workspace holds %zu bytes, %zu are needed (llmq_wq_gemm_a16_workspace_bytes)",
                                   workspace ? workspace_bytes : static_cast<size_t>(0), need);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* wsp = static_cast<float*>(workspace);
  if (dtype == LLMQ_BF16) {
    return wformat == LLMQ_W_INT8 ? launch_typed<bf16_t, 8>(x, qweight, wscale, out, wsp, M, N, G, out_group, s)
                                  : launch_typed<bf16_t, 4>(x, qweight, wscale, out, wsp, M, N, G, out_group, s);
  }
  return wformat == LLMQ_W_INT8 ? launch_typed<f16_t, 8>(x, qweight, wscale, out, wsp, M, N, G, out_group, s)
                                : launch_typed<f16_t, 4>(x, qweight, wscale, out, wsp, M, N, G, out_group, s);
}
