// GEMV over an UNQUANTIZED 16-bit weight for one activation row, with the decode step's prologues and
// epilogues, gfx950.
//
//   out[n] = sum_k x'[k] * W[n, k]       W: [N, K] fp16 / bf16 row-major, fp32 accumulation
//
// This is the baseline's kernel, not the product's: it lets a bf16 model run through the same five-launch
// decode step as the quantized one (RMSNorm -> q|k|v, attention records merged -> o_proj + residual,
// RMSNorm -> gate|up storing act(gate) * up, down + residual, RMSNorm -> lm_head), so that what weight
// quantization buys is measured with everything else held equal -- the reference compares its two sides under
// one runtime as well (llmquant/eval/verify.py:44-47). The prologues and epilogues are those of the quantized
// GEMV (llmq_wq_gemv_fused), with the same rounding points.
//
// Shape: a workgroup of four waves stages x' once in LDS (as T, 16-byte packets), then every wave walks
// rows: R rows at a time, lane l taking packets l, l + 64, ... of each, sixteen 16-byte loads in flight per
// lane, products accumulated in fp32 and summed across the wave with DPP row operations. HBM-bound:
// algorithmic bytes N * K * 2 + K * 2 + N * 2.
#include "llmq_device.h"

namespace {

using namespace llmq;

struct DenseArgs {
  const void* x;
  const void* w;
  void* out;
  int N, K;
  int prologue;             // LLMQ_PRO_NONE, LLMQ_PRO_RMSNORM or LLMQ_PRO_ATTN_MERGE
  const void* norm_weight;  // [K] for LLMQ_PRO_RMSNORM
  float eps;
  const void* residual;     // [N] or null
  int pair_half;            // > 0: W is gate rows [0, pair_half) over up rows [pair_half, 2 pair_half); out [pair_half]
  int attn_splits, attn_head_dim;
};

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

// x' into LDS as packets of eight T. Every thread of the workgroup calls it; the caller synchronises.
template <typename T, bool MERGE>
__device__ __forceinline__ void stage(const DenseArgs& a, u32x4* xs, float* red) {
  const int tid = threadIdx.x;
  const int packets = a.K / 8;
  const T* x = static_cast<const T*>(a.x);
  if constexpr (MERGE) {
    // x holds the partial records of split attention: packet p covers elements 8p .. 8p + 7 of one head
    const int hd = a.attn_head_dim;
    for (int p = tid; p < packets; p += kThreads) {
      const int head = p * 8 / hd, d0 = p * 8 - head * hd;
      float f[8];
      merge_partials8(reinterpret_cast<const float*>(a.x) +
                          static_cast<int64_t>(head) * a.attn_splits * (hd + kAttnRecordHeader),
                      a.attn_splits, hd, d0, f);
      xs[p] = Pack<T>::pack(f);
    }
    return;
  }
  if (a.prologue == LLMQ_PRO_RMSNORM) {
    // transformers' LlamaRMSNorm.forward: variance in fp32, x * rsqrt rounded to T, times the weight, rounded
    float ss = 0.0f;
    for (int p = tid; p < packets; p += kThreads) {
      float f[8];
      Pack<T>::unpack(load16(x + p * 8), f);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
    }
    ss = wave_sum(ss);
    if ((tid & (kWave - 1)) == 0) red[tid / kWave] = ss;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < kWaves; ++w) total += red[w];
    const float inv_rms = rsqrtf(total / static_cast<float>(a.K) + a.eps);
    const T* nw = static_cast<const T*>(a.norm_weight);
    for (int p = tid; p < packets; p += kThreads) {
      float f[8], w[8];
      Pack<T>::unpack(load16(x + p * 8), f);
      Pack<T>::unpack(load16(nw + p * 8), w);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = w[e] * round_through<T>(f[e] * inv_rms);
      xs[p] = Pack<T>::pack(f);
    }
    return;
  }
  for (int p = tid; p < packets; p += kThreads) xs[p] = load16(x + p * 8);
}

// R rows per wave step, U packets per row requested together: R * U = 16 loads in flight per lane.
template <typename T, int R, int U, bool MERGE>
__global__ __launch_bounds__(kThreads) void dense_gemv_kernel(const DenseArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u32x4* xs = reinterpret_cast<u32x4*>(smem);
  float* red = reinterpret_cast<float*>(smem + static_cast<size_t>(a.K) * 2);
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  stage<T, MERGE>(a, xs, red);
  __syncthreads();

  const int packets = a.K / 8;                 // per row
  const int rounds = (packets + kWave * U - 1) / (kWave * U);
  const T* w = static_cast<const T*>(a.w);
  T* out = static_cast<T*>(a.out);
  const bool paired = a.pair_half > 0;
  // a step's R rows: consecutive rows, or (paired) R / 2 gate rows and the up rows that go with them
  const int rows_per_step = paired && R >= 2 ? R / 2 : R;
  const int n_out = paired ? a.pair_half : a.N;
  const int steps = (n_out + rows_per_step - 1) / rows_per_step;
  for (int step = blockIdx.x * kWaves + wv; step < steps; step += gridDim.x * kWaves) {
    const int n0 = step * rows_per_step;
    const T* row[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // rows past the end are clamped: loaded, never stored
      const int n = paired ? min(n0 + (r >> 1), a.pair_half - 1) + ((r & 1) ? a.pair_half : 0) : min(n0 + r, a.N - 1);
      row[r] = w + static_cast<int64_t>(n) * a.K;
    }
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
    for (int round = 0; round < rounds; ++round) {
      u32x4 wp[R][U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = min((round * U + u) * kWave + lane, packets - 1);   // clamped: weighted by zero below
#pragma unroll
        for (int r = 0; r < R; ++r) wp[r][u] = load16(row[r] + p * 8);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int p = (round * U + u) * kWave + lane;
        float xf[8];
        Pack<T>::unpack(xs[min(p, packets - 1)], xf);
        if (p >= packets) {
#pragma unroll
          for (int e = 0; e < 8; ++e) xf[e] = 0.0f;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float wf[8];
          Pack<T>::unpack(wp[r][u], wf);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[r] = fmaf(wf[e], xf[e], acc[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
      if (paired) {
        if constexpr (R >= 2) {
#pragma unroll
          for (int r = 0; r < R; r += 2) {
            const int n = n0 + (r >> 1);
            if (n < a.pair_half) {
              // LlamaMLP: act_fn(gate) * up on the two Linears' rounded outputs
              const float g = round_through<T>(acc[r]), up = round_through<T>(acc[r + 1]);
              const float silu = g / (1.0f + expf(-g));
              out[n] = from_float<T>(round_through<T>(silu) * up);
            }
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int n = n0 + r;
          if (n < a.N) {
            out[n] = a.residual == nullptr
                         ? from_float<T>(acc[r])
                         : from_float<T>(to_float(static_cast<const T*>(a.residual)[n]) + round_through<T>(acc[r]));
          }
        }
      }
    }
  }
}

template <typename T, int R, int U>
int launch_ru(const DenseArgs& a, hipStream_t stream) {
  const int rows_per_step = a.pair_half > 0 && R >= 2 ? R / 2 : R;
  const int n_out = a.pair_half > 0 ? a.pair_half : a.N;
  const int steps = (n_out + rows_per_step - 1) / rows_per_step;
  int grid = (steps + kWaves - 1) / kWaves;
  if (grid > 1280) grid = 1280;   // five workgroups per CU: what is resident at this kernel's register count
  const size_t lds = static_cast<size_t>(a.K) * 2 + 64;
  if (a.prologue == LLMQ_PRO_ATTN_MERGE) {
    hipLaunchKernelGGL((dense_gemv_kernel<T, R, U, true>), dim3(grid), dim3(kThreads), lds, stream, a);
  } else {
    hipLaunchKernelGGL((dense_gemv_kernel<T, R, U, false>), dim3(grid), dim3(kThreads), lds, stream, a);
  }
  return llmq_host::check_launch("dense_gemv_kernel");
}

template <typename T>
int launch_typed(const DenseArgs& a, hipStream_t stream) {
  const int per_lane = (a.K / 8 + kWave - 1) / kWave;   // packets of a row per lane
  if (per_lane <= 4) return launch_ru<T, 4, 4>(a, stream);
  if (per_lane <= 8 || a.pair_half > 0) return launch_ru<T, 2, 8>(a, stream);
  return launch_ru<T, 1, 16>(a, stream);
}

}  // namespace

extern "C" int llmq_dense_gemv_fused(const void* x, const void* weight, void* out, int N, int K, int dtype,
                                     int prologue, const void* norm_weight, float eps, const void* residual,
                                     int pair_half, int attn_splits, int attn_head_dim, llmq_stream_t stream) {
  if (N < 0 || K < 0) return llmq_host::fail_invalid("negative dimension N=%d K=%d", N, K);
  if (dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("the dense GEMV takes float16 or bfloat16 weights and activations, got dtype code %d", dtype);
  if (K % 8 || K > 28672) return llmq_host::fail_invalid("K must be a multiple of 8 and at most 28672, got %d", K);
  if (prologue != LLMQ_PRO_NONE && prologue != LLMQ_PRO_RMSNORM && prologue != LLMQ_PRO_ATTN_MERGE)
    return llmq_host::fail_invalid("prologue must be none, RMSNorm or the attention merge, got %d", prologue);
  if (prologue == LLMQ_PRO_RMSNORM && !norm_weight) return llmq_host::fail_invalid("the RMSNorm prologue needs norm_weight");
  if (prologue == LLMQ_PRO_ATTN_MERGE &&
      (attn_splits < 1 || attn_head_dim < 8 || attn_head_dim % 8 || K % attn_head_dim))
    return llmq_host::fail_invalid("attention merge: %d splits, heads of %d in a row of %d", attn_splits, attn_head_dim, K);
  if (pair_half < 0 || (pair_half > 0 && (N != 2 * pair_half || residual != nullptr)))
    return llmq_host::fail_invalid("a gate|up weight has 2 * pair_half rows and no residual (N=%d, pair_half=%d)", N, pair_half);
  if (N == 0) return 0;
  if (K == 0) return llmq_host::fail_invalid("a weight with no columns has no reduction axis");
  if (!x || !weight || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(norm_weight)) & 15u)
    return llmq_host::fail_invalid("activation, weight and norm weight pointers must be 16-byte aligned");
  DenseArgs a{x, weight, out, N, K, prologue, norm_weight, eps, residual, pair_half, attn_splits, attn_head_dim};
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dtype == LLMQ_F16 ? launch_typed<f16_t>(a, s) : launch_typed<bf16_t>(a, s);
}
