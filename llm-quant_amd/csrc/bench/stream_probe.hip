// Measurement aid for bench.py, built into its own small library (libllmq_bench_probe.so) and not part
// of the product library or its header: a plain streaming read of a buffer with
// non-temporal 128-bit loads, eight in flight per lane, one workgroup per CU (of the grid sizes
// and load flavours tried, 256 x 256 threads with eight loads in flight read fastest on MI355X:
// 6.2 TB/s, against 4.7-5.9 TB/s for 1024-8192 workgroups). Its rate is what this GPU's
// memory system delivers to a kernel that does nothing but read, i.e. the ceiling the GEMV's
// bytes-per-second figure is to be compared with beside the published peak.
#include "../llmq_device.h"

namespace {

using namespace llmq;

constexpr int kInFlight = 8;

__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ p, const size_t n16,
                                                          uint32_t* __restrict__ sink) {
  const size_t tid = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  uint32_t acc = 0;
  size_t i = tid;
  for (; i + (kInFlight - 1) * stride < n16; i += kInFlight * stride) {
    u32x4 v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const u32x4* q = p + i + u * stride;
      v[u].x = __builtin_nontemporal_load(&q->x);
      v[u].y = __builtin_nontemporal_load(&q->y);
      v[u].z = __builtin_nontemporal_load(&q->z);
      v[u].w = __builtin_nontemporal_load(&q->w);
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const u32x4 v = p[i];
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  // the loads must not be optimised away; the store itself practically never happens
  if (acc == 0x9e3779b9u) sink[0] = acc;
}

}  // namespace

// Returns 0 or a hipError_t.
extern "C" int bench_stream_read_probe(const void* buffer, size_t bytes, uint32_t* sink, void* stream) {
  if (bytes == 0) return 0;
  if (!buffer || !sink || (reinterpret_cast<uintptr_t>(buffer) & 15u)) return static_cast<int>(hipErrorInvalidValue);
  hipLaunchKernelGGL(stream_read_kernel, dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(buffer), bytes / 16, sink);
  return static_cast<int>(hipGetLastError());
}
