// Quantized weight -> dense matrix in the activation dtype, gfx950: what KernelQuantLinear
// multiplies by when more rows arrive than the GEMV takes (llmquant/quantizers/kernel.py:68-79,
// `(qweight * scale).to(dtype)`), as one pass: read the codes once, write each value once.
//
//   out[n, g * keep + k] = (dtype)(code[n, g, k] * wscale[sr(n), g])        k < keep <= group_size
//
// keep < group_size drops the zero padding of head-aligned groups (o_proj with head_dim 64 in
// groups of 128), so the dense matrix has the layer's real input width and the activation
// needs no padding either.
//
//
// A lane produces eight consecutive values per step (from 4 or 8 bytes of int4 / int8 codes) and
// stores them as one 16-byte packet (two for fp32), so a wave's store is a contiguous KiB; the write
// is four fifths of the traffic and is what has to be coalesced. Four steps are in flight per lane.
#include "llmq_device.h"

namespace {

using namespace llmq;

constexpr int kDqInFlight = 4;

template <typename T, int BITS>
__global__ __launch_bounds__(256) void dequant_weight_kernel(
    const uint8_t* __restrict__ qw, const float* __restrict__ ws, T* __restrict__ out, const int64_t n_out_packets,
    const int G, const int gs, const int keep, const int out_group) {
  constexpr int V = 8;                  // values per step
  constexpr int kBytes = V * BITS / 8;  // code bytes behind them
  const int64_t n_threads = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const int64_t tid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int per_group = keep / V;  // output packets per group (keep is a multiple of V here)
  for (int64_t p0 = tid; p0 < n_out_packets; p0 += kDqInFlight * n_threads) {
    uint32_t raw[kDqInFlight][kBytes / 4];
    float scale[kDqInFlight];
#pragma unroll
    for (int u = 0; u < kDqInFlight; ++u) {
      const int64_t p = p0 + u * n_threads;
      if (p >= n_out_packets) break;
      const int64_t group = p / per_group;  // n * G + g
      const int k0 = static_cast<int>(p - group * per_group) * V;
      const int64_t n = group / G;
      const int g = static_cast<int>(group - n * G);
      const uint8_t* src = qw + (group * gs + k0) * BITS / 8;
#pragma unroll
      for (int w = 0; w < kBytes / 4; ++w) raw[u][w] = reinterpret_cast<const uint32_t*>(src)[w];
      scale[u] = ws[(out_group > 0 ? n / out_group : n) * G + g];
    }
#pragma unroll
    for (int u = 0; u < kDqInFlight; ++u) {
      const int64_t p = p0 + u * n_threads;
      if (p >= n_out_packets) break;
      float f[V];
      if constexpr (BITS == 8) {
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = static_cast<float>(static_cast<int8_t>(raw[u][i / 4] >> (8 * (i % 4)))) * scale[u];
      } else {
        // nibble i of the little-endian word: even i is the low nibble of byte i/2, +8 biased
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = static_cast<float>(static_cast<int>((raw[u][i / 8] >> (4 * (i % 8))) & 0xfu) - 8) * scale[u];
      }
      if constexpr (Pack<T>::N == 8) {
        store16(out + p * V, Pack<T>::pack(f));
      } else {
        store16(out + p * V, Pack<T>::pack(f));
        store16(out + p * V + 4, Pack<T>::pack(f + 4));
      }
    }
  }
}

// Any keep (not a multiple of the packet width): one thread per (row, group), element at a time.
template <typename T, int BITS>
__global__ __launch_bounds__(256) void dequant_weight_ragged_kernel(
    const uint8_t* __restrict__ qw, const float* __restrict__ ws, T* __restrict__ out, const int64_t n_groups,
    const int G, const int gs, const int keep, const int out_group) {
  const int64_t group = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (group >= n_groups) return;
  const int64_t n = group / G;
  const int g = static_cast<int>(group - n * G);
  const float scale = ws[(out_group > 0 ? n / out_group : n) * G + g];
  for (int k = 0; k < keep; ++k) {
    const int64_t idx = group * gs + k;
    int code;
    if constexpr (BITS == 8) {
      code = static_cast<int8_t>(qw[idx]);
    } else {
      const uint8_t byte = qw[idx >> 1];
      code = static_cast<int>((idx & 1) ? (byte >> 4) : (byte & 0xf)) - 8;
    }
    out[group * keep + k] = from_float<T>(static_cast<float>(code) * scale);
  }
}

template <typename T, int BITS>
int launch_bits(const void* qw, const float* ws, void* out, int64_t N, int G, int gs, int keep, int out_group,
                hipStream_t stream) {
  const uint8_t* q = static_cast<const uint8_t*>(qw);
  T* o = static_cast<T*>(out);
  if (keep % 8 == 0) {
    const int64_t n_out_packets = N * G * (keep / 8);
    int64_t blocks = (n_out_packets + 256 * kDqInFlight - 1) / (256 * kDqInFlight);
    if (blocks > 256 * 32) blocks = 256 * 32;  // the rest is walked in stripes
    hipLaunchKernelGGL((dequant_weight_kernel<T, BITS>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, q,
                       ws, o, n_out_packets, G, gs, keep, out_group);
    return llmq_host::check_launch("dequant_weight_kernel");
  }
  const int64_t n_groups = N * G;
  const int64_t blocks = (n_groups + 255) / 256;
  if (blocks > 0x7fffffff) return llmq_host::fail_invalid("weight too large for one launch");
  hipLaunchKernelGGL((dequant_weight_ragged_kernel<T, BITS>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     stream, q, ws, o, n_groups, G, gs, keep, out_group);
  return llmq_host::check_launch("dequant_weight_ragged_kernel");
}

template <typename T>
int launch_typed(const void* qw, const float* ws, void* out, int64_t N, int G, int gs, int keep, int out_group,
                 int wformat, hipStream_t stream) {
  return wformat == LLMQ_W_INT8 ? launch_bits<T, 8>(qw, ws, out, N, G, gs, keep, out_group, stream)
                                : launch_bits<T, 4>(qw, ws, out, N, G, gs, keep, out_group, stream);
}

}  // namespace

extern "C" int llmq_dequant_weight(const void* qweight, const float* wscale, void* out, int N, int G, int gs,
                                   int keep_per_group, int out_group, int wformat, int dtype,
                                   llmq_stream_t stream) {
  if (N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension N=%d G=%d", N, G);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  if (gs <= 0 || gs % 8)
    return llmq_host::fail_invalid("group_size must be a positive multiple of 8, got %d", gs);
  if (keep_per_group <= 0 || keep_per_group > gs)
    return llmq_host::fail_invalid("keep_per_group must be in [1, %d], got %d", gs, keep_per_group);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (N == 0 || G == 0) return 0;
  if (!qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(out)) & 15u)
    return llmq_host::fail_invalid("weight and output pointers must be 16-byte aligned");
  if (keep_per_group % 8 == 0 && (static_cast<int64_t>(G) * keep_per_group) % 8)
    return llmq_host::fail_invalid("internal: row width not a multiple of 8");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case LLMQ_F32: return launch_typed<float>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
    case LLMQ_F16: return launch_typed<f16_t>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
    case LLMQ_BF16: return launch_typed<bf16_t>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
  }
  return llmq_host::fail_invalid("out must be float32, float16 or bfloat16, got dtype code %d", dtype);
}
