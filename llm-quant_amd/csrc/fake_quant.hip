// Symmetric RTN group quantizer for gfx950: quantize-dequantize (fake quant) and the
// codes-emitting variant used for int8 activations.
//
// Arithmetic contract (llmquant/core/observers.py:74-98, llmquant/core/quant_ops.py:13-37,
// restated by the reference's CUDA kernel at llmquant/cuda/csrc/fake_quant.cu:50-84):
//   amax  = max |x| over the group                      (exact in any order)
//   scale = max(amax / qmax, 1e-8)                      fp32, true IEEE division
//   q     = clamp(rint(x / scale), -qmax-1, qmax)       round half to even
//   out   = cast(q * scale)                             round to nearest even
// Nothing here may be contracted, reordered or approximated: the file is built with
// -ffp-contract=off and without fast-math.
//
// Shape of the kernel. The input is read ONCE (the reference's kernel reads it twice): a
// lane owns one 16-byte packet (8 half-width or 4 fp32 elements) and keeps it in registers
// between the abs-max reduction and the quantize step. A group of `gs` elements is
// gs / packet lanes wide -- 16 lanes for the default 128-wide bf16 group, exactly one DPP
// row -- so the reduction is a short butterfly inside the wave and a wave covers a
// contiguous 1 KiB of the tensor per step, fully coalesced. Groups too wide for one wave
// (or not a power-of-two number of packets, or misaligned) take the block-per-group kernel,
// which holds up to 16 elements per thread and rereads only beyond that.
#include "llmq_device.h"

namespace {

using namespace llmq;

enum OutMode { kQdq = 0, kCodes8 = 1, kCodes4 = 2 };

template <typename T, int LPG, int MODE>
__global__ __launch_bounds__(256) void quant_lanes_kernel(
    const T* __restrict__ x, void* __restrict__ out, float* __restrict__ scale_out,
    const int64_t total, const int group_size, const float qmin, const float qmax) {
  constexpr int V = Pack<T>::N;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * blockDim.x / kWave;
  const int64_t per_wave = static_cast<int64_t>(kWave) * V;

  for (int64_t base = wave * per_wave; base < total; base += n_waves * per_wave) {
    const int64_t e0 = base + static_cast<int64_t>(lane) * V;
    const bool active = e0 < total;  // whole lane groups fall on one side: LPG*V == group_size
    float f[V];
    if (active) {
      Pack<T>::unpack(load16(x + e0), f);
    } else {
#pragma unroll
      for (int i = 0; i < V; ++i) f[i] = 0.0f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < V; ++i) amax = fmaxf(amax, fabsf(f[i]));
    amax = group_max<LPG>(amax);
    const float scale = scale_from_amax(amax, qmax);
    if (!active) continue;
    if (scale_out != nullptr && (lane & (LPG - 1)) == 0) scale_out[e0 / group_size] = scale;

    float q[V];
#pragma unroll
    for (int i = 0; i < V; ++i) q[i] = quant_code(f[i], scale, qmin, qmax);

    if constexpr (MODE == kQdq) {
#pragma unroll
      for (int i = 0; i < V; ++i) q[i] = q[i] * scale;
      store16(static_cast<T*>(out) + e0, Pack<T>::pack(q));
    } else if constexpr (MODE == kCodes8) {
      uint32_t w[V / 4];
#pragma unroll
      for (int i = 0; i < V / 4; ++i) {
        w[i] = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w[i] |= (static_cast<uint32_t>(static_cast<int>(q[4 * i + j])) & 0xffu) << (8 * j);
        }
      }
      int8_t* dst = static_cast<int8_t*>(out) + e0;
      if constexpr (V == 8) {
        *reinterpret_cast<u32x2*>(dst) = u32x2{w[0], w[1]};
      } else {
        *reinterpret_cast<uint32_t*>(dst) = w[0];
      }
    } else {
      // nibble packing of llmquant/packing/packing.py:20-33: +8 bias, even index low
      uint32_t w = 0;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        w |= (static_cast<uint32_t>(static_cast<int>(q[i]) + 8) & 0xfu) << (4 * i);
      }
      uint8_t* dst = static_cast<uint8_t*>(out) + e0 / 2;
      if constexpr (V == 8) {
        *reinterpret_cast<uint32_t*>(dst) = w;
      } else {
        *reinterpret_cast<uint16_t*>(dst) = static_cast<uint16_t>(w);
      }
    }
  }
}

// One 256-thread block per group, any group size, any alignment.
constexpr int kBlockThreads = 256;
constexpr int kHeld = 16;  // elements a thread keeps in registers between the two passes

template <typename T, int MODE>
__global__ __launch_bounds__(kBlockThreads) void quant_block_kernel(
    const T* __restrict__ x, void* __restrict__ out, float* __restrict__ scale_out,
    const int group_size, const float qmin, const float qmax) {
  __shared__ float s_part[kBlockThreads / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * group_size;
  const int tid = threadIdx.x;

  float held[kHeld];
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < kHeld; ++j) {
    const int i = tid + j * kBlockThreads;
    held[j] = i < group_size ? to_float(x[base + i]) : 0.0f;
    amax = fmaxf(amax, fabsf(held[j]));
  }
  for (int i = tid + kHeld * kBlockThreads; i < group_size; i += kBlockThreads) {
    amax = fmaxf(amax, fabsf(to_float(x[base + i])));
  }
  amax = group_max<kWave>(amax);
  if ((tid & (kWave - 1)) == 0) s_part[tid / kWave] = amax;
  __syncthreads();
  amax = s_part[0];
#pragma unroll
  for (int w = 1; w < kBlockThreads / kWave; ++w) amax = fmaxf(amax, s_part[w]);

  const float scale = scale_from_amax(amax, qmax);
  if (scale_out != nullptr && tid == 0) scale_out[blockIdx.x] = scale;

  auto emit = [&](int i, float v) {
    const float q = quant_code(v, scale, qmin, qmax);
    if constexpr (MODE == kQdq) {
      static_cast<T*>(out)[base + i] = from_float<T>(q * scale);
    } else {
      static_cast<int8_t*>(out)[base + i] = static_cast<int8_t>(static_cast<int>(q));
    }
  };
#pragma unroll
  for (int j = 0; j < kHeld; ++j) {
    const int i = tid + j * kBlockThreads;
    if (i < group_size) emit(i, held[j]);
  }
  for (int i = tid + kHeld * kBlockThreads; i < group_size; i += kBlockThreads) {
    emit(i, to_float(x[base + i]));
  }
}

// Packed-nibble output for the block kernel: a thread owns element pairs.
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void quant_block_pack4_kernel(
    const T* __restrict__ x, uint8_t* __restrict__ out, float* __restrict__ scale_out,
    const int group_size, const float qmin, const float qmax) {
  __shared__ float s_part[kBlockThreads / kWave];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * group_size;
  const int tid = threadIdx.x;
  float amax = 0.0f;
  for (int i = tid; i < group_size; i += kBlockThreads) {
    amax = fmaxf(amax, fabsf(to_float(x[base + i])));
  }
  amax = group_max<kWave>(amax);
  if ((tid & (kWave - 1)) == 0) s_part[tid / kWave] = amax;
  __syncthreads();
  amax = s_part[0];
#pragma unroll
  for (int w = 1; w < kBlockThreads / kWave; ++w) amax = fmaxf(amax, s_part[w]);
  const float scale = scale_from_amax(amax, qmax);
  if (scale_out != nullptr && tid == 0) scale_out[blockIdx.x] = scale;
  for (int p = tid; p < group_size / 2; p += kBlockThreads) {
    const int lo = static_cast<int>(quant_code(to_float(x[base + 2 * p]), scale, qmin, qmax)) + 8;
    const int hi = static_cast<int>(quant_code(to_float(x[base + 2 * p + 1]), scale, qmin, qmax)) + 8;
    out[base / 2 + p] = static_cast<uint8_t>((lo & 0xf) | ((hi & 0xf) << 4));
  }
}

template <typename T, int MODE>
int launch_typed(const void* x, void* out, float* scale, int64_t n_groups, int group_size,
                 float qmin, float qmax, hipStream_t stream) {
  constexpr int V = Pack<T>::N;
  const int64_t total = n_groups * group_size;
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int lpg = group_size / V;
  const bool lanes_ok = aligned && group_size % V == 0 && lpg >= 1 && lpg <= kWave &&
                        (lpg & (lpg - 1)) == 0;
  if (lanes_ok) {
    const int64_t per_wave = static_cast<int64_t>(kWave) * V;
    const int64_t waves = (total + per_wave - 1) / per_wave;
    int64_t blocks = (waves + 3) / 4;
    const int64_t cap = 256 * 32;  // enough resident waves to cover HBM latency; rest strides
    if (blocks > cap) blocks = cap;
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    const T* xp = static_cast<const T*>(x);
#define LLMQ_LANES(L)                                                                        \
  case L:                                                                                    \
    hipLaunchKernelGGL((quant_lanes_kernel<T, L, MODE>), grid, block, 0, stream, xp, out,    \
                       scale, total, group_size, qmin, qmax);                                \
    break;
    switch (lpg) {
      LLMQ_LANES(1) LLMQ_LANES(2) LLMQ_LANES(4) LLMQ_LANES(8)
      LLMQ_LANES(16) LLMQ_LANES(32) LLMQ_LANES(64)
    }
#undef LLMQ_LANES
    return llmq_host::check_launch("quant_lanes_kernel");
  }
  if (n_groups > 2147483647LL) {
    return llmq_host::fail_invalid("too many groups for a 1D grid: %lld", (long long)n_groups);
  }
  const dim3 grid(static_cast<unsigned>(n_groups)), block(kBlockThreads);
  if constexpr (MODE == kCodes4) {
    hipLaunchKernelGGL((quant_block_pack4_kernel<T>), grid, block, 0, stream,
                       static_cast<const T*>(x), static_cast<uint8_t*>(out), scale, group_size,
                       qmin, qmax);
  } else {
    hipLaunchKernelGGL((quant_block_kernel<T, MODE>), grid, block, 0, stream,
                       static_cast<const T*>(x), out, scale, group_size, qmin, qmax);
  }
  return llmq_host::check_launch("quant_block_kernel");
}

template <int MODE>
int launch(const void* x, void* out, float* scale, int64_t n_groups, int group_size,
           int num_bits, int dtype, hipStream_t stream) {
  const float qmax = static_cast<float>((1 << (num_bits - 1)) - 1);
  const float qmin = -qmax - 1.0f;
  switch (dtype) {
    case LLMQ_F32:
      return launch_typed<float, MODE>(x, out, scale, n_groups, group_size, qmin, qmax, stream);
    case LLMQ_F16:
      return launch_typed<f16_t, MODE>(x, out, scale, n_groups, group_size, qmin, qmax, stream);
    case LLMQ_BF16:
      return launch_typed<bf16_t, MODE>(x, out, scale, n_groups, group_size, qmin, qmax, stream);
  }
  return llmq_host::fail_invalid("x must be float32, float16 or bfloat16, got dtype code %d", dtype);
}

int check_common(const void* x, const void* out, int64_t n_groups, int group_size, int num_bits) {
  if (n_groups < 0) return llmq_host::fail_invalid("n_groups must be >= 0, got %lld", (long long)n_groups);
  if (group_size <= 0) return llmq_host::fail_invalid("group_size must be positive, got %d", group_size);
  if (num_bits < 2 || num_bits > 8) return llmq_host::fail_invalid("num_bits must be in [2, 8], got %d", num_bits);
  if (n_groups > 0 && (x == nullptr || out == nullptr)) return llmq_host::fail_invalid("null tensor pointer");
  return 0;
}

}  // namespace

extern "C" int llmq_fake_quant_group(const void* x, void* out, float* scale_or_null,
                                     int64_t n_groups, int group_size, int num_bits, int dtype,
                                     llmq_stream_t stream) {
  if (int rc = check_common(x, out, n_groups, group_size, num_bits)) return rc;
  if (n_groups == 0) return 0;
  return launch<kQdq>(x, out, scale_or_null, n_groups, group_size, num_bits, dtype,
                      static_cast<hipStream_t>(stream));
}

extern "C" int llmq_quant_group_codes(const void* x, void* codes, float* scale, int64_t n_groups,
                                      int group_size, int num_bits, int pack4, int dtype,
                                      llmq_stream_t stream) {
  if (int rc = check_common(x, codes, n_groups, group_size, num_bits)) return rc;
  if (pack4 && num_bits > 4) return llmq_host::fail_invalid("nibble packing needs num_bits <= 4, got %d", num_bits);
  if (pack4 && group_size % 2) return llmq_host::fail_invalid("group_size %d must be even to pack into nibbles", group_size);
  if (n_groups == 0) return 0;
  if (scale == nullptr) return llmq_host::fail_invalid("scale output is required");
  hipStream_t s = static_cast<hipStream_t>(stream);
  return pack4 ? launch<kCodes4>(x, codes, scale, n_groups, group_size, num_bits, dtype, s)
               : launch<kCodes8>(x, codes, scale, n_groups, group_size, num_bits, dtype, s);
}
