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
// One 16-byte packet of codes per lane (16 int8 codes or 32 nibbles); a wave covers 1 KB of
// contiguous codes and writes 2 KB / 4 KB of contiguous bf16 when nothing is dropped.
#include "llmq_device.h"

namespace {

using namespace llmq;

template <typename T, int BITS>
__global__ __launch_bounds__(256) void dequant_weight_kernel(
    const uint8_t* __restrict__ qw, const float* __restrict__ ws, T* __restrict__ out, const int64_t n_packets,
    const int G, const int gs, const int keep, const int out_group) {
  constexpr int kCodes = BITS == 8 ? 16 : 32;  // codes per packet
  const int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (p >= n_packets) return;
  const int per_group = gs / kCodes;  // packets per group
  const int64_t group = p / per_group;  // n * G + g
  const int k0 = static_cast<int>(p - group * per_group) * kCodes;
  if (k0 >= keep) return;
  const int64_t n = group / G;
  const int g = static_cast<int>(group - n * G);
  const float scale = ws[(out_group > 0 ? n / out_group : n) * G + g];
  const u32x4 raw = load16(qw + p * 16);
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
  float f[kCodes];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    if constexpr (BITS == 8) {
#pragma unroll
      for (int b = 0; b < 4; ++b) f[4 * d + b] = static_cast<float>(static_cast<int8_t>(w[d] >> (8 * b))) * scale;
    } else {
      // byte b holds codes 2b (low nibble) and 2b + 1 (high nibble), each biased by +8
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int byte = (w[d] >> (8 * b)) & 0xff;
        f[8 * d + 2 * b] = static_cast<float>((byte & 15) - 8) * scale;
        f[8 * d + 2 * b + 1] = static_cast<float>((byte >> 4) - 8) * scale;
      }
    }
  }
  T* dst = out + (n * G + g) * keep + k0;
  constexpr int kPer = Pack<T>::N;  // elements per 16-byte store
  if (keep % kPer == 0) {
#pragma unroll
    for (int i = 0; i < kCodes; i += kPer) {
      if (k0 + i < keep) store16(dst + i, Pack<T>::pack(f + i));
    }
  } else {
#pragma unroll
    for (int i = 0; i < kCodes; ++i) {
      if (k0 + i < keep) dst[i] = from_float<T>(f[i]);
    }
  }
}

template <typename T>
int launch_typed(const void* qw, const float* ws, void* out, int64_t N, int G, int gs, int keep, int out_group,
                 int wformat, hipStream_t stream) {
  const int codes_per_packet = wformat == LLMQ_W_INT8 ? 16 : 32;
  const int64_t n_packets = N * G * (gs / codes_per_packet);
  const int64_t blocks = (n_packets + 255) / 256;
  if (blocks > 0x7fffffff) return llmq_host::fail_invalid("weight too large for one launch");
  if (wformat == LLMQ_W_INT8) {
    hipLaunchKernelGGL((dequant_weight_kernel<T, 8>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                       static_cast<const uint8_t*>(qw), ws, static_cast<T*>(out), n_packets, G, gs, keep, out_group);
  } else {
    hipLaunchKernelGGL((dequant_weight_kernel<T, 4>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                       static_cast<const uint8_t*>(qw), ws, static_cast<T*>(out), n_packets, G, gs, keep, out_group);
  }
  return llmq_host::check_launch("dequant_weight_kernel");
}

}  // namespace

extern "C" int llmq_dequant_weight(const void* qweight, const float* wscale, void* out, int N, int G, int gs,
                                   int keep_per_group, int out_group, int wformat, int dtype,
                                   llmq_stream_t stream) {
  if (N < 0 || G < 0) return llmq_host::fail_invalid("negative dimension N=%d G=%d", N, G);
  if (wformat != LLMQ_W_INT8 && wformat != LLMQ_W_INT4_PACKED)
    return llmq_host::fail_invalid("unsupported weight format %d, expected 8 or 4", wformat);
  const int codes_per_packet = wformat == LLMQ_W_INT8 ? 16 : 32;
  if (gs <= 0 || gs % codes_per_packet)
    return llmq_host::fail_invalid("group_size must be a positive multiple of %d, got %d", codes_per_packet, gs);
  if (keep_per_group <= 0 || keep_per_group > gs)
    return llmq_host::fail_invalid("keep_per_group must be in [1, %d], got %d", gs, keep_per_group);
  if (out_group < 0) return llmq_host::fail_invalid("out_group must be >= 0, got %d", out_group);
  if (N == 0 || G == 0) return 0;
  if (!qweight || !wscale || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(qweight) | reinterpret_cast<uintptr_t>(out)) & 15u)
    return llmq_host::fail_invalid("weight and output pointers must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case LLMQ_F32: return launch_typed<float>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
    case LLMQ_F16: return launch_typed<f16_t>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
    case LLMQ_BF16: return launch_typed<bf16_t>(qweight, wscale, out, N, G, gs, keep_per_group, out_group, wformat, s);
  }
  return llmq_host::fail_invalid("out must be float32, float16 or bfloat16, got dtype code %d", dtype);
}
