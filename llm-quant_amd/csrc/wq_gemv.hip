// Weight-only quantized GEMV for decode (M small), gfx950.
//
//   out[m, n] = sum_g wscale[sr(n), g] * sum_{k in g} x[m, k] * q[n, g, k]
//
// Same algebra as the reference's wq_gemv kernel (llmquant/cuda/csrc/wq_gemv.cu:45-130):
// integer codes multiplied by the activation in fp32, the group scale applied to the
// per-lane partial, one cross-lane reduction at the very end. What differs is the shape.
//
// The weight is the only large operand, so everything is arranged around streaming it with
// 128-bit loads. A row of the canonical [N, G, gs] weight is cut into 16-byte chunks (16
// int8 codes or 32 packed int4 codes); a chunk never straddles a group. A wave owns a
// fixed K-segment of 64 chunks -- lane L owns chunk L of the segment -- so the slice of x a
// lane needs is the same for every row: it is loaded into registers once and rows are
// streamed past it, R rows per step so R 16-byte loads are in flight per lane. Waves of a
// workgroup split first the K-segments of a row (WK of them), then rows (WR). Partial sums
// cross lanes once per row batch (wave butterfly) and cross waves through LDS.
//
// Codes are converted with v_cvt_f32_ubyte*, which wants unsigned bytes: int8 is XORed
// with 0x80 (code + 128) and int4 nibbles are used as stored (code + 8); the bias comes
// back out as  bias * sum_{k in lane} x[k], computed once per x slice, not per row.
#include <stdlib.h>

#include <type_traits>

#include "llmq_device.h"

namespace {

using namespace llmq;

template <int BITS> struct Chunk {
  static constexpr int kVals = 128 / BITS;  // codes per 16-byte chunk
};

// Load the x values one chunk covers (kVals elements of row m starting at k0) as fp32.
template <typename T, int VALS>
__device__ __forceinline__ void load_x(const T* __restrict__ x, int64_t off, bool ok, float* f) {
  constexpr int V = Pack<T>::N;
#pragma unroll
  for (int p = 0; p < VALS / V; ++p) {
    if (ok) {
      Pack<T>::unpack(load16(x + off + p * V), f + p * V);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) f[p * V + i] = 0.0f;
    }
  }
}

template <int BITS, int M>
__device__ __forceinline__ void chunk_dot(const u32x4 w, const float (*xf)[M], float* p) {
  const uint32_t d[4] = {w.x, w.y, w.z, w.w};
  if constexpr (BITS == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t t = d[i] ^ 0x80808080u;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float u = static_cast<float>((t >> (8 * b)) & 0xffu);
#pragma unroll
        for (int m = 0; m < M; ++m) p[m] = fmaf(u, xf[4 * i + b][m], p[m]);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = d[i] & 0x0f0f0f0fu;         // codes at even k
      const uint32_t hi = (d[i] >> 4) & 0x0f0f0f0fu;  // codes at odd k
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const float ul = static_cast<float>((lo >> (8 * b)) & 0xffu);
        const float uh = static_cast<float>((hi >> (8 * b)) & 0xffu);
#pragma unroll
        for (int m = 0; m < M; ++m) {
          p[m] = fmaf(ul, xf[8 * i + 2 * b][m], p[m]);
          p[m] = fmaf(uh, xf[8 * i + 2 * b + 1][m], p[m]);
        }
      }
    }
  }
}

struct GemvArgs {
  const void* x;
  const uint8_t* qw;
  const float* ws;
  void* out;
  int N, G;
  int chunks_per_row;    // 16-byte chunks in one weight row
  int chunks_per_group;  // of one scale group
  int k_total;           // G * gs, row stride of x in elements
  int out_group;
  int wk, wr;            // waves along K and along rows in one workgroup
  int n_batches;         // row batches of wr*R rows
};

constexpr int kMaxWaves = 4;

template <typename T, int BITS, int M, int R>
__global__ __launch_bounds__(256) void wq_gemv_kernel(const GemvArgs a) {
  constexpr int VALS = Chunk<BITS>::kVals;
  constexpr float kBias = BITS == 8 ? 128.0f : 8.0f;
  __shared__ float s_part[kMaxWaves][R][M];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int wk = wave % a.wk;
  const int wr = wave / a.wk;
  const T* __restrict__ x = static_cast<const T*>(a.x);
  T* __restrict__ out = static_cast<T*>(a.out);
  const int n_seg = (a.chunks_per_row + kWave - 1) / kWave;
  const bool one_seg = n_seg <= a.wk;  // this wave's x slice never changes

  float xf[VALS][M];
  float xsum[M];
  auto fetch_x = [&](int seg) {
    const int c = seg * kWave + lane;
    const bool ok = c < a.chunks_per_row;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float tmp[VALS];
      load_x<T, VALS>(x, static_cast<int64_t>(m) * a.k_total + static_cast<int64_t>(c) * VALS, ok, tmp);
      float s = 0.0f;
#pragma unroll
      for (int i = 0; i < VALS; ++i) {
        xf[i][m] = tmp[i];
        s += tmp[i];
      }
      xsum[m] = s * kBias;
    }
  };
  if (one_seg) fetch_x(wk);  // wk >= n_seg leaves zeros: that wave contributes nothing

  for (int batch = blockIdx.x; batch < a.n_batches; batch += gridDim.x) {
    const int n0 = (batch * a.wr + wr) * R;
    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

    for (int seg = wk; seg < n_seg; seg += a.wk) {
      if (!one_seg) fetch_x(seg);
      const int c = seg * kWave + lane;
      const bool ok = c < a.chunks_per_row;
      const int g = ok ? c / a.chunks_per_group : 0;
      u32x4 w[R];
      float sc[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = min(n0 + r, a.N - 1);  // rows past the end are computed and dropped
        const int64_t row = static_cast<int64_t>(n) * a.chunks_per_row;
        w[r] = ok ? load16(a.qw + (row + c) * 16) : u32x4{0, 0, 0, 0};
        const int srow = a.out_group > 0 ? n / a.out_group : n;
        sc[r] = ok ? a.ws[static_cast<int64_t>(srow) * a.G + g] : 0.0f;
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float p[M];
#pragma unroll
        for (int m = 0; m < M; ++m) p[m] = 0.0f;
        chunk_dot<BITS, M>(w[r], xf, p);
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = fmaf(p[m] - xsum[m], sc[r], acc[r][m]);
      }
    }

#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[r][m] = wave_sum(acc[r][m]);

    if (a.wk == 1) {
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (n0 + r < a.N) {
#pragma unroll
            for (int m = 0; m < M; ++m) out[static_cast<int64_t>(m) * a.N + n0 + r] = from_float<T>(acc[r][m]);
          }
        }
      }
    } else {
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < M; ++m) s_part[wave][r][m] = acc[r][m];
      }
      __syncthreads();
      // one thread per (row group, r, m) adds the K-split partials in wave order
      const int items = a.wr * R * M;
      for (int it = threadIdx.x; it < items; it += blockDim.x) {
        const int m = it % M;
        const int r = (it / M) % R;
        const int rw = it / (M * R);
        float total = 0.0f;
        for (int k = 0; k < a.wk; ++k) total += s_part[rw * a.wk + k][r][m];
        const int n = (batch * a.wr + rw) * R + r;
        if (n < a.N) out[static_cast<int64_t>(m) * a.N + n] = from_float<T>(total);
      }
      __syncthreads();
    }
  }
}

// Fallback for layouts the chunked kernel cannot take (a group that is not a whole number
// of 16-byte chunks, or misaligned pointers): one wave per row, element at a time.
template <typename T, int BITS>
__global__ __launch_bounds__(256) void wq_gemv_scalar_kernel(
    const T* __restrict__ x, const uint8_t* __restrict__ qw, const float* __restrict__ ws,
    T* __restrict__ out, int M, int N, int G, int gs, int out_group) {
  const int lane = threadIdx.x & (kWave - 1);
  const int n = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (n >= N) return;  // whole waves leave together; no barrier follows
  const int64_t k_total = static_cast<int64_t>(G) * gs;
  const int srow = out_group > 0 ? n / out_group : n;
  for (int m = 0; m < M; ++m) {
    float acc = 0.0f;
    for (int g = 0; g < G; ++g) {
      float part = 0.0f;
      for (int k = lane; k < gs; k += kWave) {
        const int64_t idx = static_cast<int64_t>(n) * k_total + static_cast<int64_t>(g) * gs + k;
        int code;
        if constexpr (BITS == 8) {
          code = static_cast<int8_t>(qw[idx]);
        } else {
          const uint8_t byte = qw[idx >> 1];
          code = static_cast<int>((idx & 1) ? (byte >> 4) : (byte & 0xf)) - 8;
        }
        part = fmaf(static_cast<float>(code), to_float(x[m * k_total + g * gs + k]), part);
      }
      acc = fmaf(part, ws[static_cast<int64_t>(srow) * G + g], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[static_cast<int64_t>(m) * N + n] = from_float<T>(acc);
  }
}

// The batched form of the fallback: plan entry blockIdx.y names an expert and a run of rows.
template <typename T, int BITS>
__global__ __launch_bounds__(256) void wq_gemv_batched_scalar_kernel(
    const T* __restrict__ x, const uint8_t* __restrict__ qw, const float* __restrict__ ws, T* __restrict__ out,
    const int32_t* __restrict__ block_expert, const int32_t* __restrict__ block_row0,
    const int32_t* __restrict__ block_rows, int n_rows, int n_experts, int N, int G, int gs, int out_group) {
  const int b = blockIdx.y;
  const int rows = block_rows[b];
  if (rows <= 0) return;
  const int e = block_expert[b], row0 = block_row0[b];
  if (e < 0 || e >= n_experts || row0 < 0 || row0 + rows > n_rows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int n = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (n >= N) return;
  const int64_t k_total = static_cast<int64_t>(G) * gs;
  const int64_t scale_rows = out_group > 0 ? (N + out_group - 1) / out_group : N;
  const int srow = out_group > 0 ? n / out_group : n;
  const float* wse = ws + (static_cast<int64_t>(e) * scale_rows + srow) * G;
  const int64_t w0 = (static_cast<int64_t>(e) * N + n) * k_total;  // in codes
  for (int m = row0; m < row0 + rows; ++m) {
    float acc = 0.0f;
    for (int g = 0; g < G; ++g) {
      float part = 0.0f;
      for (int k = lane; k < gs; k += kWave) {
        const int64_t idx = w0 + static_cast<int64_t>(g) * gs + k;
        int code;
        if constexpr (BITS == 8) {
          code = static_cast<int8_t>(qw[idx]);
        } else {
          const uint8_t byte = qw[idx >> 1];
          code = static_cast<int>((idx & 1) ? (byte >> 4) : (byte & 0xf)) - 8;
        }
        part = fmaf(static_cast<float>(code), to_float(x[m * k_total + g * gs + k]), part);
      }
      acc = fmaf(part, wse[g], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[static_cast<int64_t>(m) * N + n] = from_float<T>(acc);
  }
}

template <typename T, int BITS>
int launch_batched_scalar(const void* x, const void* qw, const float* ws, void* out, const int32_t* be,
                          const int32_t* b0, const int32_t* br, int n_blocks, int n_rows, int n_experts, int N,
                          int G, int gs, int out_group, hipStream_t stream) {
  const dim3 g((N + 3) / 4, n_blocks), b(256);
  hipLaunchKernelGGL((wq_gemv_batched_scalar_kernel<T, BITS>), g, b, 0, stream, static_cast<const T*>(x),
                     static_cast<const uint8_t*>(qw), ws, static_cast<T*>(out), be, b0, br, n_rows, n_experts, N, G,
                     gs, out_group);
  return llmq_host::check_launch("wq_gemv_batched_scalar_kernel");
}

template <typename T, int BITS, int M>
int launch_rows(const GemvArgs& base, int N, hipStream_t stream) {
  GemvArgs a = base;
  const int n_seg = (a.chunks_per_row + kWave - 1) / kWave;
  a.wk = n_seg < 4 ? (n_seg < 2 ? 1 : 2) : 4;
  a.wr = 4 / a.wk;
  // rows per wave step: as many as keeps >= ~2 workgroups per CU
  int R = 8;
  while (R > 1 && (static_cast<int64_t>(N) + a.wr * R - 1) / (a.wr * R) < 512) R >>= 1;
  if (M >= 3 && R == 8) R = 4;  // register budget
  a.n_batches = (N + a.wr * R - 1) / (a.wr * R);
  const int grid = a.n_batches < 2048 ? a.n_batches : 2048;
  const dim3 g(grid), b(kWave * a.wk * a.wr);
  if constexpr (M <= 2) {
    if (R == 8) {
      hipLaunchKernelGGL((wq_gemv_kernel<T, BITS, M, 8>), g, b, 0, stream, a);
      return llmq_host::check_launch("wq_gemv_kernel");
    }
  }
  switch (R) {
    case 4: hipLaunchKernelGGL((wq_gemv_kernel<T, BITS, M, 4>), g, b, 0, stream, a); break;
    case 2: hipLaunchKernelGGL((wq_gemv_kernel<T, BITS, M, 2>), g, b, 0, stream, a); break;
    default: hipLaunchKernelGGL((wq_gemv_kernel<T, BITS, M, 1>), g, b, 0, stream, a); break;
  }
  return llmq_host::check_launch("wq_gemv_kernel");
}

template <typename T, int BITS>
int launch_typed(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                 int gs, int out_group, hipStream_t stream) {
  constexpr int VALS = Chunk<BITS>::kVals;
  const int64_t k_total = static_cast<int64_t>(G) * gs;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(qw)) & 15u) == 0;
  const bool chunked = aligned && gs % VALS == 0 && (k_total * sizeof(T)) % 16 == 0;
  constexpr int kRows = 4;  // activation rows one launch keeps in registers
  for (int m0 = 0; m0 < M; m0 += kRows) {
    const int rows = M - m0 < kRows ? M - m0 : kRows;
    const T* xm = static_cast<const T*>(x) + static_cast<int64_t>(m0) * k_total;
    T* om = static_cast<T*>(out) + static_cast<int64_t>(m0) * N;
    if (llmq_host::gemv_mfma_supported(xm, qw, ws, rows, G, gs, BITS == 8 ? LLMQ_W_INT8 : LLMQ_W_INT4_PACKED) &&
        !llmq_host::gemv_force_alu()) {
      const int dtype = sizeof(T) == 4 ? LLMQ_F32 : (std::is_same<T, f16_t>::value ? LLMQ_F16 : LLMQ_BF16);
      if (int rc = llmq_host::gemv_mfma_launch(xm, qw, ws, om, rows, N, G, out_group,
                                               BITS == 8 ? LLMQ_W_INT8 : LLMQ_W_INT4_PACKED, dtype, stream))
        return rc;
      continue;
    }
    if (!chunked) {
      const dim3 g((N + 3) / 4), b(256);
      hipLaunchKernelGGL((wq_gemv_scalar_kernel<T, BITS>), g, b, 0, stream, xm,
                         static_cast<const uint8_t*>(qw), ws, om, rows, N, G, gs, out_group);
      if (int rc = llmq_host::check_launch("wq_gemv_scalar_kernel")) return rc;
      continue;
    }
    GemvArgs a{};
    a.x = xm; a.qw = static_cast<const uint8_t*>(qw); a.ws = ws; a.out = om;
    a.N = N; a.G = G;
    a.chunks_per_row = static_cast<int>(k_total / VALS);
    a.chunks_per_group = gs / VALS;
    a.k_total = static_cast<int>(k_total);
    a.out_group = out_group;
    int rc = 0;
    switch (rows) {
      case 1: rc = launch_rows<T, BITS, 1>(a, N, stream); break;
      case 2: rc = launch_rows<T, BITS, 2>(a, N, stream); break;
      case 3: rc = launch_rows<T, BITS, 3>(a, N, stream); break;
      default: rc = launch_rows<T, BITS, 4>(a, N, stream); break;
    }
    if (rc) return rc;
  }
  return 0;
}

template <int BITS>
int launch_bits(const void* x, const void* qw, const float* ws, void* out, int M, int N, int G,
                int gs, int out_group, int dtype, hipStream_t stream) {
  switch (dtype) {
    case LLMQ_F32: return launch_typed<float, BITS>(x, qw, ws, out, M, N, G, gs, out_group, stream);
    case LLMQ_F16: return launch_typed<f16_t, BITS>(x, qw, ws, out, M, N, G, gs, out_group, stream);
    case LLMQ_BF16: return launch_typed<bf16_t, BITS>(x, qw, ws, out, M, N, G, gs, out_group, stream);
  }
  return llmq_host::fail_invalid("x must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

}  // namespace

namespace llmq_host {
// LLMQ_GEMV_ALU=1 in the environment routes every GEMV to the vector-ALU kernel (used by the
// tests to cover that kernel on shapes the matrix-core kernel would otherwise take).
bool gemv_force_alu() {
  static const bool forced = [] {
    const char* v = getenv("LLMQ_GEMV_ALU");
    return v != nullptr && v[0] == '1';
  }();
  return forced;
}
}  // namespace llmq_host

extern "C" int llmq_wq_gemv(const void* x, const void* qweight, const float* wscale, void* out,
                            int M, int N, int G, int gs, int out_group, int wformat, int dtype,
                            llmq_stream_t stream) {
  if (M < 0 || N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension M=%d N=%d G=%d", M, N, G);
  if (gs <= 0) return llmq_host::fail_invalid("group_size must be positive, got %d", gs);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (wformat == LLMQ_W_INT8 && gs % 4)
    return llmq_host::fail_invalid("group_size must be a multiple of 4, got %d", gs);
  if (wformat == LLMQ_W_INT4_PACKED && gs % 8)
    return llmq_host::fail_invalid("group_size must be a multiple of 8 for packed int4, got %d", gs);
  if (M == 0 || N == 0) return 0;
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!x || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  return wformat == LLMQ_W_INT8
             ? launch_bits<8>(x, qweight, wscale, out, M, N, G, gs, out_group, dtype, s)
             : launch_bits<4>(x, qweight, wscale, out, M, N, G, gs, out_group, dtype, s);
}

extern "C" int llmq_wq_gemv_fused(const void* x, const void* qweight, const float* wscale, void* out,
                                  int N, int G, int out_group, int wformat, int dtype, int prologue,
                                  const void* norm_weight, float eps, int in_head_dim,
                                  const void* residual_or_null, llmq_stream_t stream) {
  if (N < 0 || G <= 0) return llmq_host::fail_invalid("bad dimension N=%d G=%d", N, G);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (prologue != LLMQ_PRO_NONE && prologue != LLMQ_PRO_RMSNORM && prologue != LLMQ_PRO_SILU_MUL)
    return llmq_host::fail_invalid("unknown prologue %d", prologue);
  if (prologue == LLMQ_PRO_RMSNORM && norm_weight == nullptr)
    return llmq_host::fail_invalid("the RMSNorm prologue needs its weight");
  if (in_head_dim < 0 || in_head_dim > 128 || in_head_dim % 8)
    return llmq_host::fail_invalid("in_head_dim must be a multiple of 8 in [0, 128], got %d", in_head_dim);
  if (in_head_dim > 0 && prologue != LLMQ_PRO_NONE)
    return llmq_host::fail_invalid("head padding cannot be combined with a prologue");
  if (N == 0) return 0;
  if (!x || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if (!llmq_host::gemv_mfma_supported(x, qweight, wscale, 1, G, 128, wformat))
    return llmq_host::fail_invalid("the fused GEMV needs group size 128, a multiple of 4 groups "
                                   "and 16-byte aligned operands");
  return llmq_host::gemv_mfma_launch_fused(x, qweight, wscale, out, 1, N, G, out_group, wformat, dtype, prologue,
                                           norm_weight, eps, in_head_dim, residual_or_null,
                                           static_cast<hipStream_t>(stream));
}

extern "C" int llmq_wq_gemv_attn_merge(const float* partials, int n_splits, int head_dim, const void* qweight,
                                       const float* wscale, void* out, int N, int G, int out_group, int wformat,
                                       int dtype, int in_head_dim, const void* residual_or_null,
                                       llmq_stream_t stream) {
  if (N < 0 || G <= 0) return llmq_host::fail_invalid("bad dimension N=%d G=%d", N, G);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (n_splits < 1 || n_splits > 256) return llmq_host::fail_invalid("n_splits must be in [1, 256], got %d", n_splits);
  if (head_dim <= 0 || head_dim % 8) return llmq_host::fail_invalid("head_dim must be a positive multiple of 8, got %d", head_dim);
  if (in_head_dim < 0 || in_head_dim > 128 || in_head_dim % 8)
    return llmq_host::fail_invalid("in_head_dim must be a multiple of 8 in [0, 128], got %d", in_head_dim);
  const int k_real = G * (in_head_dim > 0 ? in_head_dim : 128);
  if (k_real % head_dim)
    return llmq_host::fail_invalid("the Linear's input width %d is not a whole number of heads of %d", k_real, head_dim);
  if (N == 0) return 0;
  if (!partials || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if (!llmq_host::gemv_mfma_supported(partials, qweight, wscale, 1, G, 128, wformat))
    return llmq_host::fail_invalid("the fused GEMV needs group size 128, a multiple of 4 groups "
                                   "and 16-byte aligned operands");
  return llmq_host::gemv_mfma_launch_fused(partials, qweight, wscale, out, 1, N, G, out_group, wformat, dtype,
                                           LLMQ_PRO_ATTN_MERGE, nullptr, 0.0f, in_head_dim, residual_or_null,
                                           static_cast<hipStream_t>(stream), n_splits, head_dim);
}

extern "C" int llmq_wq_gemv_gate_up_silu(const void* x, const void* qweight, const float* wscale, void* out,
                                        int intermediate, int G, int wformat, int dtype, int prologue,
                                        const void* norm_weight, float eps, llmq_stream_t stream) {
  if (intermediate < 0 || G <= 0) return llmq_host::fail_invalid("bad dimension intermediate=%d G=%d", intermediate, G);
  if (intermediate % 8) return llmq_host::fail_invalid("the intermediate width must be a multiple of 8, got %d", intermediate);
  if (intermediate > (1 << 29)) return llmq_host::fail_invalid("intermediate width %d is too large", intermediate);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (prologue != LLMQ_PRO_NONE && prologue != LLMQ_PRO_RMSNORM)
    return llmq_host::fail_invalid("the gate|up GEMV takes no prologue or RMSNorm, got %d", prologue);
  if (prologue == LLMQ_PRO_RMSNORM && norm_weight == nullptr)
    return llmq_host::fail_invalid("the RMSNorm prologue needs its weight");
  if (intermediate == 0) return 0;
  if (!x || !qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if (!llmq_host::gemv_mfma_supported(x, qweight, wscale, 1, G, 128, wformat))
    return llmq_host::fail_invalid("the fused GEMV needs group size 128, a multiple of 4 groups "
                                   "and 16-byte aligned operands");
  return llmq_host::gemv_mfma_launch_fused(x, qweight, wscale, out, 1, 2 * intermediate, G, 0, wformat, dtype,
                                           prologue, norm_weight, eps, 0, nullptr,
                                           static_cast<hipStream_t>(stream), 0, 0, intermediate);
}

extern "C" int llmq_wq_gemv_batched_max_rows(void) { return 8; }

extern "C" int llmq_wq_gemv_batched(const void* x, const void* qweight, const float* wscale, void* out,
                                    const int32_t* block_expert, const int32_t* block_row0,
                                    const int32_t* block_rows, int n_blocks, int n_rows, int n_experts, int N,
                                    int G, int gs, int out_group, int wformat, int dtype, llmq_stream_t stream) {
  if (n_blocks < 0 || n_rows < 0 || n_experts < 0 || N < 0 || G < 0)
    return llmq_host::fail_invalid("negative dimension blocks=%d rows=%d experts=%d N=%d G=%d", n_blocks, n_rows,
                                   n_experts, N, G);
  if (gs <= 0) return llmq_host::fail_invalid("group_size must be positive, got %d", gs);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (wformat == LLMQ_W_INT4_PACKED && gs % 2)
    return llmq_host::fail_invalid("group_size must be even for packed int4, got %d", gs);
  if (n_blocks == 0 || n_rows == 0 || N == 0 || n_experts == 0) return 0;
  if (n_blocks > 65535) return llmq_host::fail_invalid("at most 65535 plan entries per launch, got %d", n_blocks);
  if (G == 0) return llmq_host::fail_invalid("a weight with no groups has no reduction axis");
  if (!x || !qweight || !wscale || !out || !block_expert || !block_row0 || !block_rows)
    return llmq_host::fail_invalid("null tensor pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // every expert's weight must be as aligned as the first one's
  const int64_t weight_stride = static_cast<int64_t>(N) * G * gs * (wformat == LLMQ_W_INT8 ? 2 : 1) / 2;
  if (weight_stride % 16 == 0 && llmq_host::gemv_batched_mfma_supported(x, qweight, wscale, G, gs, wformat)) {
    return llmq_host::gemv_batched_mfma_launch(x, qweight, wscale, out, block_expert, block_row0, block_rows,
                                               n_blocks, n_rows, n_experts, N, G, out_group, wformat, dtype, s);
  }
#define LLMQ_SCALAR(T)                                                                                        \
  (wformat == LLMQ_W_INT8                                                                                     \
       ? launch_batched_scalar<T, 8>(x, qweight, wscale, out, block_expert, block_row0, block_rows, n_blocks, \
                                     n_rows, n_experts, N, G, gs, out_group, s)                               \
       : launch_batched_scalar<T, 4>(x, qweight, wscale, out, block_expert, block_row0, block_rows, n_blocks, \
                                     n_rows, n_experts, N, G, gs, out_group, s))
  switch (dtype) {
    case LLMQ_F32: return LLMQ_SCALAR(float);
    case LLMQ_F16: return LLMQ_SCALAR(f16_t);
    case LLMQ_BF16: return LLMQ_SCALAR(bf16_t);
  }
#undef LLMQ_SCALAR
  return llmq_host::fail_invalid("x must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

extern "C" int llmq_wq_gemv_batched_fused(const void* x, int64_t x_row_stride, const void* qweight,
                                         const float* wscale, void* out, const int32_t* block_expert,
                                         const int32_t* block_row0, const int32_t* block_rows, int n_blocks,
                                         int n_rows, int n_experts, int N, int G, int wformat, int dtype,
                                         int act_pair, llmq_stream_t stream) {
  if (n_blocks < 0 || n_rows < 0 || n_experts < 0 || N < 0 || G <= 0)
    return llmq_host::fail_invalid("bad dimension blocks=%d rows=%d experts=%d N=%d G=%d", n_blocks, n_rows,
                                   n_experts, N, G);
  if (x_row_stride < 0) return llmq_host::fail_invalid("x_row_stride must be >= 0");
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (act_pair && N % 16) return llmq_host::fail_invalid("gate|up needs halves that are multiples of 8 rows, got N=%d", N);
  if (n_blocks == 0 || n_rows == 0 || N == 0 || n_experts == 0) return 0;
  if (n_blocks > 65535) return llmq_host::fail_invalid("at most 65535 plan entries per launch, got %d", n_blocks);
  if (!x || !qweight || !wscale || !out || !block_expert || !block_row0 || !block_rows)
    return llmq_host::fail_invalid("null tensor pointer");
  const int64_t weight_stride = static_cast<int64_t>(N) * G * 128 * (wformat == LLMQ_W_INT8 ? 2 : 1) / 2;
  if (weight_stride % 16 || (x_row_stride * (dtype == LLMQ_F32 ? 4 : 2)) % 16 ||
      !llmq_host::gemv_batched_mfma_supported(x, qweight, wscale, G, 128, wformat))
    return llmq_host::fail_invalid("the fused batched GEMV needs group size 128, a multiple of 4 groups and "
                                   "16-byte aligned operands and rows");
  return llmq_host::gemv_batched_mfma_launch(x, qweight, wscale, out, block_expert, block_row0, block_rows, n_blocks,
                                             n_rows, n_experts, N, G, 0, wformat, dtype,
                                             static_cast<hipStream_t>(stream), x_row_stride, act_pair ? N / 2 : 0);
}
