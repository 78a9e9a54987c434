// The elementwise pieces of a prompt pass, one launch each, gfx950.
//
// Walking a decoder layer over a prompt the way transformers does costs ~45 PyTorch kernels per
// layer beside the matmuls: LlamaRMSNorm alone is seven (to fp32, pow, mean, add, rsqrt, mul, cast,
// mul), apply_rotary_pos_emb ten, and on a 512-token prompt of a 1B model they add up to more time
// than the matmuls. Each of the three below is one pass over its tensor with the rounding points of
// the PyTorch sequence it replaces, the same ones the decode kernels use.
//
//   rmsnorm    out = w * T(x_f32 * rsqrt(mean(x_f32^2) + eps))        (LlamaRMSNorm.forward), optionally
//              on x = T(x + delta), the residual add in front of it, which is stored as well
//   rope_qk    out = T(T(x * cos) + T(rotate_half(x) * sin))           (apply_rotary_pos_emb), q and k
//   silu_mul   out = T(T(silu(gate)) * up)                             (LlamaMLP: act_fn(gate) * up)
#include "llmq_device.h"

namespace {

using namespace llmq;

constexpr int kNormThreads = 256;

// One workgroup per row. The row is read twice (the second time from cache). With `delta` the row is
// first replaced by T(x + delta), which is also stored to `sum_out`: the residual add in front of a
// norm (hidden = hidden + branch; normed = norm(hidden)) in the same launch.
template <typename T, bool ADD>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ delta,
                                                              const T* __restrict__ w, T* __restrict__ sum_out,
                                                              T* __restrict__ out, const int hidden, const float eps) {
  constexpr int V = Pack<T>::N;
  __shared__ float red[kNormThreads / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * hidden;
  const T* row = x + base;
  T* orow = out + base;
  const int tid = threadIdx.x;
  float ss = 0.0f;
  for (int i = tid * V; i < hidden; i += kNormThreads * V) {
    float f[V];
    Pack<T>::unpack(load16(row + i), f);
    if constexpr (ADD) {
      float d[V];
      Pack<T>::unpack(load16(delta + base + i), d);
#pragma unroll
      for (int e = 0; e < V; ++e) f[e] = round_through<T>(f[e] + d[e]);
      store16(sum_out + base + i, Pack<T>::pack(f));
    }
#pragma unroll
    for (int e = 0; e < V; ++e) ss = fmaf(f[e], f[e], ss);
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
  for (int i = tid * V; i < hidden; i += kNormThreads * V) {
    float f[V], g[V];
    Pack<T>::unpack(load16(src + i), f);
    Pack<T>::unpack(load16(w + i), g);
#pragma unroll
    for (int e = 0; e < V; ++e) f[e] = g[e] * round_through<T>(f[e] * inv_rms);
    store16(orow + i, Pack<T>::pack(f));
  }
}

// x: [tokens, heads, D] with a row stride (elements between tokens), cos/sin: [tokens, D]. One thread
// per Pack of the first half of a head: it produces element i and element i + D/2, which read the
// same two inputs.
template <typename T>
__global__ __launch_bounds__(256) void rope_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                   const T* __restrict__ cos_t, const T* __restrict__ sin_t,
                                                   T* __restrict__ q_out, T* __restrict__ k_out, const int tokens,
                                                   const int q_heads, const int kv_heads, const int D,
                                                   const int64_t q_stride, const int64_t k_stride) {
  constexpr int V = Pack<T>::N;
  const int per_head = D / 2 / V;
  const int heads = q_heads + kv_heads;
  const int64_t item = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (item >= static_cast<int64_t>(tokens) * heads * per_head) return;
  const int p = static_cast<int>(item % per_head);
  const int h = static_cast<int>((item / per_head) % heads);
  const int t = static_cast<int>(item / (static_cast<int64_t>(per_head) * heads));
  const bool is_k = h >= q_heads;
  const T* src = is_k ? k + t * k_stride + static_cast<int64_t>(h - q_heads) * D : q + t * q_stride + static_cast<int64_t>(h) * D;
  T* dst = is_k ? k_out + (static_cast<int64_t>(t) * kv_heads + (h - q_heads)) * D
                : q_out + (static_cast<int64_t>(t) * q_heads + h) * D;
  const int i = p * V;
  float lo[V], hi[V], c_lo[V], c_hi[V], s_lo[V], s_hi[V];
  Pack<T>::unpack(load16(src + i), lo);
  Pack<T>::unpack(load16(src + i + D / 2), hi);
  Pack<T>::unpack(load16(cos_t + static_cast<int64_t>(t) * D + i), c_lo);
  Pack<T>::unpack(load16(cos_t + static_cast<int64_t>(t) * D + i + D / 2), c_hi);
  Pack<T>::unpack(load16(sin_t + static_cast<int64_t>(t) * D + i), s_lo);
  Pack<T>::unpack(load16(sin_t + static_cast<int64_t>(t) * D + i + D / 2), s_hi);
  float o_lo[V], o_hi[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    // rotate_half: first half pairs with -second half, second half with +first half
    o_lo[e] = round_through<T>(round_through<T>(lo[e] * c_lo[e]) + round_through<T>(-hi[e] * s_lo[e]));
    o_hi[e] = round_through<T>(round_through<T>(hi[e] * c_hi[e]) + round_through<T>(lo[e] * s_hi[e]));
  }
  store16(dst + i, Pack<T>::pack(o_lo));
  store16(dst + i + D / 2, Pack<T>::pack(o_hi));
}

// gate, up: [rows, width] with row strides (two column blocks of one projection output, or two tensors).
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                       T* __restrict__ out, const int64_t packets, const int per_row,
                                                       const int64_t gate_stride, const int64_t up_stride) {
  constexpr int V = Pack<T>::N;
  const int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (p >= packets) return;
  const int64_t row = p / per_row;
  const int col = static_cast<int>(p - row * per_row) * V;
  float g[V], u[V];
  Pack<T>::unpack(load16(gate + row * gate_stride + col), g);
  Pack<T>::unpack(load16(up + row * up_stride + col), u);
#pragma unroll
  for (int e = 0; e < V; ++e) g[e] = round_through<T>(g[e] / (1.0f + expf(-g[e]))) * u[e];
  store16(out + p * V, Pack<T>::pack(g));
}

bool aligned16(const void* a, const void* b = nullptr, const void* c = nullptr) {
  return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 15u) == 0;
}

int packet_of(int dtype) { return dtype == LLMQ_F32 ? 4 : 8; }

}  // namespace

#define LLMQ_BY_DTYPE(CALL)                                                                                  \
  switch (dtype) {                                                                                           \
    case LLMQ_F32: { using T = float; CALL; } break;                                                         \
    case LLMQ_F16: { using T = llmq::f16_t; CALL; } break;                                                   \
    case LLMQ_BF16: { using T = llmq::bf16_t; CALL; } break;                                                 \
    default: return llmq_host::fail_invalid("dtype code %d is not float32, float16 or bfloat16", dtype);      \
  }

extern "C" int llmq_add_rmsnorm(const void* x, const void* delta_or_null, const void* weight, void* sum_out_or_null,
                                void* out, int rows, int hidden, float eps, int dtype, llmq_stream_t stream) {
  if (rows < 0 || hidden <= 0) return llmq_host::fail_invalid("bad dimension rows=%d hidden=%d", rows, hidden);
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("dtype code %d is not float32, float16 or bfloat16", dtype);
  if (hidden % packet_of(dtype)) return llmq_host::fail_invalid("hidden must be a multiple of %d, got %d", packet_of(dtype), hidden);
  if (rows == 0) return 0;
  if (!x || !weight || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((delta_or_null == nullptr) != (sum_out_or_null == nullptr))
    return llmq_host::fail_invalid("delta and sum_out go together");
  if (!aligned16(x, weight, out) || !aligned16(delta_or_null, sum_out_or_null))
    return llmq_host::fail_invalid("tensors must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (delta_or_null) {
    LLMQ_BY_DTYPE(hipLaunchKernelGGL((rmsnorm_kernel<T, true>), dim3(rows), dim3(kNormThreads), 0, s,
                                     static_cast<const T*>(x), static_cast<const T*>(delta_or_null),
                                     static_cast<const T*>(weight), static_cast<T*>(sum_out_or_null),
                                     static_cast<T*>(out), hidden, eps));
  } else {
    LLMQ_BY_DTYPE(hipLaunchKernelGGL((rmsnorm_kernel<T, false>), dim3(rows), dim3(kNormThreads), 0, s,
                                     static_cast<const T*>(x), static_cast<const T*>(nullptr),
                                     static_cast<const T*>(weight), static_cast<T*>(nullptr), static_cast<T*>(out),
                                     hidden, eps));
  }
  return llmq_host::check_launch("rmsnorm_kernel");
}

extern "C" int llmq_rmsnorm(const void* x, const void* weight, void* out, int rows, int hidden, float eps, int dtype,
                            llmq_stream_t stream) {
  return llmq_add_rmsnorm(x, nullptr, weight, nullptr, out, rows, hidden, eps, dtype, stream);
}

extern "C" int llmq_rope_qk(const void* q, const void* k, const void* cos_rows, const void* sin_rows, void* q_out,
                            void* k_out, int tokens, int q_heads, int kv_heads, int head_dim, int64_t q_row_stride,
                            int64_t k_row_stride, int dtype, llmq_stream_t stream) {
  if (tokens < 0 || q_heads < 0 || kv_heads < 0 || head_dim <= 0)
    return llmq_host::fail_invalid("bad dimension tokens=%d q_heads=%d kv_heads=%d head_dim=%d", tokens, q_heads, kv_heads, head_dim);
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("dtype code %d is not float32, float16 or bfloat16", dtype);
  const int v = packet_of(dtype);
  if (head_dim % (2 * v)) return llmq_host::fail_invalid("head_dim must be a multiple of %d, got %d", 2 * v, head_dim);
  if (q_row_stride % v || k_row_stride % v) return llmq_host::fail_invalid("row strides must be multiples of %d elements", v);
  if (tokens == 0 || q_heads + kv_heads == 0) return 0;
  if (!cos_rows || !sin_rows || (q_heads && (!q || !q_out)) || (kv_heads && (!k || !k_out)))
    return llmq_host::fail_invalid("null tensor pointer");
  if (!aligned16(q, k, cos_rows) || !aligned16(sin_rows, q_out, k_out))
    return llmq_host::fail_invalid("tensors must be 16-byte aligned");
  const int64_t items = static_cast<int64_t>(tokens) * (q_heads + kv_heads) * (head_dim / 2 / v);
  const dim3 grid(static_cast<unsigned>((items + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  LLMQ_BY_DTYPE(hipLaunchKernelGGL(rope_kernel<T>, grid, block, 0, s, static_cast<const T*>(q), static_cast<const T*>(k),
                                   static_cast<const T*>(cos_rows), static_cast<const T*>(sin_rows),
                                   static_cast<T*>(q_out), static_cast<T*>(k_out), tokens, q_heads, kv_heads, head_dim,
                                   q_row_stride, k_row_stride));
  return llmq_host::check_launch("rope_kernel");
}

extern "C" int llmq_silu_mul_rows(const void* gate, const void* up, void* out, int64_t rows, int width,
                                  int64_t gate_row_stride, int64_t up_row_stride, int dtype, llmq_stream_t stream) {
  if (rows < 0 || width < 0) return llmq_host::fail_invalid("negative dimension");
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("dtype code %d is not float32, float16 or bfloat16", dtype);
  const int v = packet_of(dtype);
  if (width % v || gate_row_stride % v || up_row_stride % v)
    return llmq_host::fail_invalid("the width and the row strides must be multiples of %d elements", v);
  if (rows == 0 || width == 0) return 0;
  if (!gate || !up || !out) return llmq_host::fail_invalid("null tensor pointer");
  if (!aligned16(gate, up, out)) return llmq_host::fail_invalid("gate, up and out must be 16-byte aligned");
  const int per_row = width / v;
  const int64_t packets = rows * per_row;
  const dim3 grid(static_cast<unsigned>((packets + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  LLMQ_BY_DTYPE(hipLaunchKernelGGL(silu_mul_kernel<T>, grid, block, 0, s, static_cast<const T*>(gate),
                                   static_cast<const T*>(up), static_cast<T*>(out), packets, per_row, gate_row_stride,
                                   up_row_stride));
  return llmq_host::check_launch("silu_mul_kernel");
}

extern "C" int llmq_silu_mul(const void* gate, const void* up, void* out, int64_t count, int dtype, llmq_stream_t stream) {
  if (count < 0) return llmq_host::fail_invalid("negative element count");
  const int v = dtype == LLMQ_F32 ? 4 : 8;
  if (count % v) return llmq_host::fail_invalid("the element count must be a multiple of %d", v);
  return llmq_silu_mul_rows(gate, up, out, count / v, v, v, v, dtype, stream);  // rows of one packet each
}
