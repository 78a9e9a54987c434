// Quantized KV cache for decode, gfx950: quantize-on-append, dequantize-on-read inside
// single-token grouped-query attention.
//
// What is stored is what FakeQuantCache (llmquant/quantizers/fake.py:39-55) computes and then
// throws away: the integer codes and the one fp32 scale per (token, head) that its group-128
// rule yields for head_dim <= 128. Reading a cached element back gives (dtype)(code * scale),
// the very value the reference keeps in its bf16 cache, so attention sees the same K and V;
// only the bytes in HBM differ: head_dim (+4) per token-head instead of 2*head_dim.
//
// Layout, one layer: codes [kv_heads, t_max, head_dim] int8 (8 bit) or
// [kv_heads, t_max, head_dim/2] nibble-packed uint8 (4 bit, +8 bias, even index low), scales
// [kv_heads, t_max] fp32. The write position and the valid length live on the device, so a
// decode step is the same sequence of launches every token and can be replayed from a graph.
#include <mutex>

#include "llmq_device.h"

namespace {

using namespace llmq;

// ---- append -------------------------------------------------------------------------------------
// One wave per (tensor, head, token): lane l holds elements l and l + 64 of the head vector.
template <typename T, int BITS>
__global__ __launch_bounds__(256) void kv_append_kernel(
    const T* __restrict__ k_new, const T* __restrict__ v_new, const int64_t head_stride,
    const int64_t token_stride, uint8_t* __restrict__ k_codes, uint8_t* __restrict__ v_codes,
    float* __restrict__ k_scale, float* __restrict__ v_scale, T* __restrict__ dq_k, T* __restrict__ dq_v,
    const int32_t* __restrict__ pos_dev, const int n_new, const int kv_heads, const int head_dim,
    const int t_max) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t per_tensor = static_cast<int64_t>(kv_heads) * n_new;
  if (wave >= 2 * per_tensor) return;  // whole waves leave together; no barrier follows
  const bool is_v = wave >= per_tensor;
  const int64_t idx = is_v ? wave - per_tensor : wave;
  const int head = static_cast<int>(idx / n_new);
  const int tok = static_cast<int>(idx - static_cast<int64_t>(head) * n_new);
  const int pos = pos_dev[0] + tok;
  if (pos < 0 || pos >= t_max) return;

  const T* src = (is_v ? v_new : k_new) + head * head_stride + tok * token_stride;
  const float qmax = static_cast<float>((1 << (BITS - 1)) - 1);
  const float qmin = -qmax - 1.0f;
  float f[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int d = lane + e * kWave;
    f[e] = d < head_dim ? to_float(src[d]) : 0.0f;
  }
  float amax = fmaxf(fabsf(f[0]), fabsf(f[1]));
  amax = group_max<kWave>(amax);
  const float scale = scale_from_amax(amax, qmax);
  const int64_t slot = static_cast<int64_t>(head) * t_max + pos;
  if (lane == 0) (is_v ? v_scale : k_scale)[slot] = scale;
  uint8_t* codes = is_v ? v_codes : k_codes;
  T* dq = is_v ? dq_v : dq_k;
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int d = lane + e * kWave;
    const float q = quant_code(f[e], scale, qmin, qmax);
    if (dq != nullptr && d < head_dim) {
      dq[(static_cast<int64_t>(head) * n_new + tok) * head_dim + d] = from_float<T>(q * scale);
    }
    const int code = static_cast<int>(q);
    if constexpr (BITS == 8) {
      if (d < head_dim) codes[slot * head_dim + d] = static_cast<uint8_t>(code);
    } else {
      // pair the even lane's code with its odd neighbour's
      const int mine = (code + 8) & 0xf;
      const int other = dpp<kDppXor1>(mine);
      if ((lane & 1) == 0 && d < head_dim) {
        codes[slot * (head_dim / 2) + d / 2] = static_cast<uint8_t>(mine | (other << 4));
      }
    }
  }
}

// ---- prompt pass: RoPE on q and k, then the append, in one launch -----------------------------------
// One wave per (token, head) over the query, key and value heads of a token, heads of a token side
// by side so that a row of the q|k|v projection is read in order. Lane l holds elements l and
// l + 64 of the head vector, as in kv_append_kernel; the RoPE partner of element i is i +- D/2, the
// same lane for D = 128 and lane l ^ 32 for D = 64. Query waves rotate and store; key waves rotate,
// round to T (the tensor the two-launch path hands to the append) and quantize; value waves quantize.
template <typename T, int BITS, int D>
__global__ __launch_bounds__(256) void rope_kv_append_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, const int64_t q_stride,
    const int64_t k_stride, const int64_t v_stride, const T* __restrict__ cos_rows,
    const T* __restrict__ sin_rows, T* __restrict__ q_out, uint8_t* __restrict__ k_codes,
    uint8_t* __restrict__ v_codes, float* __restrict__ k_scale, float* __restrict__ v_scale,
    T* __restrict__ dq_k, T* __restrict__ dq_v, const int32_t* __restrict__ pos_dev, const int tokens,
    const int q_heads, const int kv_heads, const int t_max) {
  static_assert(D == 64 || D == 128, "lane layout below");
  constexpr int E = D / kWave;  // elements per lane
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int heads = q_heads + 2 * kv_heads;
  if (wave >= static_cast<int64_t>(tokens) * heads) return;  // whole waves leave together
  const int tok = static_cast<int>(wave / heads);
  const int h = static_cast<int>(wave - static_cast<int64_t>(tok) * heads);
  const bool is_q = h < q_heads;
  const bool is_v = h >= q_heads + kv_heads;
  const int head = is_q ? h : (is_v ? h - q_heads - kv_heads : h - q_heads);
  const T* src = is_q   ? q + tok * q_stride + static_cast<int64_t>(head) * D
                 : is_v ? v + tok * v_stride + static_cast<int64_t>(head) * D
                        : k + tok * k_stride + static_cast<int64_t>(head) * D;
  float f[2] = {0.0f, 0.0f};
#pragma unroll
  for (int e = 0; e < E; ++e) f[e] = to_float(src[lane + e * kWave]);

  if (!is_v) {
    float rot[2] = {0.0f, 0.0f};
    if constexpr (D == 128) {
      rot[0] = -f[1];
      rot[1] = f[0];
    } else {
      const float other = __shfl_xor(f[0], 32, kWave);
      rot[0] = lane < 32 ? -other : other;
    }
    const T* cos_row = cos_rows + static_cast<int64_t>(tok) * D;
    const T* sin_row = sin_rows + static_cast<int64_t>(tok) * D;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float a = round_through<T>(f[e] * to_float(cos_row[lane + e * kWave]));
      const float b = round_through<T>(rot[e] * to_float(sin_row[lane + e * kWave]));
      f[e] = round_through<T>(a + b);
    }
  }
  if (is_q) {
    T* dst = q_out + (static_cast<int64_t>(tok) * q_heads + head) * D;
#pragma unroll
    for (int e = 0; e < E; ++e) dst[lane + e * kWave] = from_float<T>(f[e]);
    return;
  }

  const int pos = pos_dev[0] + tok;
  if (pos < 0 || pos >= t_max) return;
  const float qmax = static_cast<float>((1 << (BITS - 1)) - 1);
  const float qmin = -qmax - 1.0f;
  float amax = fmaxf(fabsf(f[0]), fabsf(f[1]));
  amax = group_max<kWave>(amax);
  const float scale = scale_from_amax(amax, qmax);
  const int64_t slot = static_cast<int64_t>(head) * t_max + pos;
  if (lane == 0) (is_v ? v_scale : k_scale)[slot] = scale;
  uint8_t* codes = is_v ? v_codes : k_codes;
  T* dq = is_v ? dq_v : dq_k;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int d = lane + e * kWave;
    const float qv = quant_code(f[e], scale, qmin, qmax);
    if (dq != nullptr) dq[(static_cast<int64_t>(head) * tokens + tok) * D + d] = from_float<T>(qv * scale);
    const int code = static_cast<int>(qv);
    if constexpr (BITS == 8) {
      codes[slot * D + d] = static_cast<uint8_t>(code);
    } else {
      const int mine = (code + 8) & 0xf;
      const int other = dpp<kDppXor1>(mine);
      if ((lane & 1) == 0) codes[slot * (D / 2) + d / 2] = static_cast<uint8_t>(mine | (other << 4));
    }
  }
}

// ---- dequantize a range of the cache (what update() hands back outside of decode) ---------------
template <typename T, int BITS>
__global__ __launch_bounds__(256) void kv_dequant_kernel(
    const uint8_t* __restrict__ codes, const float* __restrict__ scale, T* __restrict__ out,
    const int kv_heads, const int head_dim, const int t_max, const int n_tokens) {
  const int64_t total = static_cast<int64_t>(kv_heads) * n_tokens * head_dim;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int d = static_cast<int>(i % head_dim);
    const int64_t ht = i / head_dim;
    const int t = static_cast<int>(ht % n_tokens);
    const int h = static_cast<int>(ht / n_tokens);
    const int64_t slot = static_cast<int64_t>(h) * t_max + t;
    int code;
    if constexpr (BITS == 8) {
      code = static_cast<int8_t>(codes[slot * head_dim + d]);
    } else {
      const uint8_t byte = codes[slot * (head_dim / 2) + d / 2];
      code = static_cast<int>((d & 1) ? (byte >> 4) : (byte & 0xf)) - 8;
    }
    out[i] = from_float<T>(static_cast<float>(code) * scale[slot]);
  }
}

// ---- decode attention ------------------------------------------------------------------------------
// Grid (splits, kv_heads). A workgroup owns one kv head and a fixed slice of token positions,
// and serves all `REP` query heads of that kv head, so codes are read once. Inside a wave a
// quad of lanes shares a token: lane (tk = lane / 4, dq = lane % 4) loads a quarter of the
// token's K row and V row (16-byte loads; 16 tokens = 1 KiB contiguous per wave-load for
// head_dim 64 int8). Every quad runs its own online softmax over its tokens (no cross-lane
// traffic in the loop besides the 2-step quad sum of the score); quads, waves and finally
// splits are merged with the usual (max, sum, weighted output) rule. The last workgroup of a
// kv head to arrive (device counter, reset by that workgroup) merges the splits and writes
// the output, so the whole attention is one launch.
constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / kWave;
constexpr int kTokPerIter = 16;  // tokens one wave handles per step (a quad per token)

// The code bytes of one token quarter (DPL codes), raw, and their conversion to floats.
template <int BITS, int DPL> struct RawCodes {
  static constexpr int kWords = DPL * BITS / 32;
  uint32_t w[kWords];
};

template <int BITS, int DPL>
__device__ __forceinline__ RawCodes<BITS, DPL> load_raw(const uint8_t* row, int dq) {
  RawCodes<BITS, DPL> r;
  const uint8_t* p = row + dq * (DPL * BITS / 8);
  if constexpr (RawCodes<BITS, DPL>::kWords % 4 == 0) {
#pragma unroll
    for (int i = 0; i < RawCodes<BITS, DPL>::kWords / 4; ++i) {
      const u32x4 v = load16(p + 16 * i);
      r.w[4 * i] = v.x; r.w[4 * i + 1] = v.y; r.w[4 * i + 2] = v.z; r.w[4 * i + 3] = v.w;
    }
  } else {
    const u32x2 v = *reinterpret_cast<const u32x2*>(p);
    r.w[0] = v.x; r.w[1] = v.y;
  }
  return r;
}

template <int BITS, int DPL>
__device__ __forceinline__ void decode_raw(const RawCodes<BITS, DPL>& r, float* c) {
  if constexpr (BITS == 8) {
#pragma unroll
    for (int i = 0; i < DPL / 4; ++i)
#pragma unroll
      for (int b = 0; b < 4; ++b) c[4 * i + b] = static_cast<float>(static_cast<int8_t>(r.w[i] >> (8 * b)));
  } else {
#pragma unroll
    for (int i = 0; i < DPL / 8; ++i)
#pragma unroll
      for (int b = 0; b < 8; ++b) c[8 * i + b] = static_cast<float>(static_cast<int>((r.w[i] >> (4 * b)) & 0xfu) - 8);
  }
}

// BITS == 16: the cache holds the values themselves in the model's 16-bit type T (the unquantized cache of a
// 16-bit baseline run through the same step); "decoding" is the conversion to float and the scale is 1.
template <typename T, int DPL>
__device__ __forceinline__ void decode_values16(const RawCodes<16, DPL>& r, float* c) {
#pragma unroll
  for (int i = 0; i < DPL / 8; ++i) {
    Pack<T>::unpack(u32x4{r.w[4 * i], r.w[4 * i + 1], r.w[4 * i + 2], r.w[4 * i + 3]}, c + 8 * i);
  }
}
template <typename T, int BITS, int DPL>
__device__ __forceinline__ void decode_cache_row(const RawCodes<BITS, DPL>& r, float* c) {
  if constexpr (BITS == 16) {
    static_assert(sizeof(T) == 2, "an unquantized cache holds 16-bit values");
    decode_values16<T, DPL>(r, c);
  } else {
    decode_raw<BITS, DPL>(r, c);
  }
}

// One step's operands of attend_range, for callers that can request the first steps early.
template <int BITS, int DPL> struct AttnPrefetch {
  RawCodes<BITS, DPL> k, v;
  float ks, vs;
};

template <int BITS, int DPL>
__device__ __forceinline__ AttnPrefetch<BITS, DPL> attn_prefetch(const uint8_t* kbase, const uint8_t* vbase,
                                                                 const float* ksc, const float* vsc, int t, int dq) {
  constexpr int ROWB = DPL * 4 * BITS / 8;
  AttnPrefetch<BITS, DPL> p;
  p.k = load_raw<BITS, DPL>(kbase + static_cast<int64_t>(t) * ROWB, dq);
  p.v = load_raw<BITS, DPL>(vbase + static_cast<int64_t>(t) * ROWB, dq);
  p.ks = ksc[t];
  p.vs = vsc[t];
  return p;
}

// Online-softmax attention of one wave over tokens t_first, t_first + t_step, ... (16 tokens per
// step, a quad of lanes per token), followed by the merge of the wave's 16 quads. On return
// lanes 0..3 (and every lane with the same dq, up to the order of the additions) hold the wave's
// (max, sum, weighted output quarter) per head.
// The loads of step i + NPRE are issued before step i is computed. `first`, when given, holds the
// operands of steps 0 .. NPRE-1 (token rows min(t_first + i t_step + tk, t_clamp)), requested by the
// caller before it knew t_end; every row up to t_clamp must be readable, what lies at or beyond
// t_end is loaded and dropped.
// ROW_PARTIALS: instead of the merged wave result, every lane returns the wave's maximum
// in m and, in l / o, the sums over the four quads of its own row of 16 lanes that share its dq,
// already scaled to that maximum: the caller adds the four rows (lanes 0..3, 16..19, 32..35, 48..51).
// One exponential and two DPP additions per value, against a rescaling exchange per step and two
// trips through the LDS permute path for the full merge.
template <typename T, int BITS, int D, int REP, int NPRE = 1, bool ROW_PARTIALS = false>
__device__ __forceinline__ void attend_range(const float (*qf)[D / 4], const uint8_t* kbase, const uint8_t* vbase,
                                             const float* ksc, const float* vsc, const int t_first,
                                             const int t_end, const int t_step, const int tk, const int dq,
                                             float* m, float* l, float (*o)[D / 4],
                                             const AttnPrefetch<BITS, D / 4>* first = nullptr, int t_clamp = -1) {
  constexpr int DPL = D / 4;
#pragma unroll
  for (int h = 0; h < REP; ++h) {
    m[h] = -INFINITY;
    l[h] = 0.0f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) o[h][i] = 0.0f;
  }

  if (t_clamp < 0) t_clamp = t_end - 1;  // clamp: loads stay in range, result dropped
  AttnPrefetch<BITS, DPL> ring[NPRE];
#pragma unroll
  for (int r = 0; r < NPRE; ++r) {
    if (first != nullptr) {
      ring[r] = first[r];
    } else if (t_first + r * t_step < t_end) {
      ring[r] = attn_prefetch<BITS, DPL>(kbase, vbase, ksc, vsc, min(t_first + r * t_step + tk, t_clamp), dq);
    }
  }
  for (int t_round = t_first; t_round < t_end; t_round += NPRE * t_step) {
#pragma unroll
  for (int r = 0; r < NPRE; ++r) {
    const int t0 = t_round + r * t_step;
    if (t0 >= t_end) break;
    const bool ok = t0 + tk < t_end;
    const RawCodes<BITS, DPL> k_now = ring[r].k, v_now = ring[r].v;
    const float ks = ring[r].ks, vs = ring[r].vs;
    if (t0 + NPRE * t_step < t_end) {
      ring[r] = attn_prefetch<BITS, DPL>(kbase, vbase, ksc, vsc, min(t0 + NPRE * t_step + tk, t_clamp), dq);
    }
    float kc[DPL], vc[DPL];
    decode_cache_row<T, BITS, DPL>(k_now, kc);
    decode_cache_row<T, BITS, DPL>(v_now, vc);
    float s[REP];
#pragma unroll
    for (int h = 0; h < REP; ++h) s[h] = 0.0f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const float kd = round_through<T>(kc[i] * ks);  // the value the reference's cache holds
#pragma unroll
      for (int h = 0; h < REP; ++h) s[h] = fmaf(qf[h][i], kd, s[h]);
    }
#pragma unroll
    for (int h = 0; h < REP; ++h) {
      s[h] += dpp<kDppXor1>(s[h]);  // the four lanes of a token's quad
      s[h] += dpp<kDppXor2>(s[h]);
    }
    if (ok) {
      float p[REP];
#pragma unroll
      for (int h = 0; h < REP; ++h) {
        const float m_new = fmaxf(m[h], s[h]);
        const float corr = exp2f(m[h] - m_new);  // exp2f(-inf) == 0 on the first token
        p[h] = exp2f(s[h] - m_new);
        // Once the running maxima have settled no lane of the wave raises its own any more and the
        // correction is exactly 1 everywhere: the rescaling is skipped (same bits, fewer multiplies).
        if (__builtin_amdgcn_ballot_w64(m_new != m[h]) != 0) {
          l[h] = l[h] * corr;
#pragma unroll
          for (int i = 0; i < DPL; ++i) o[h][i] *= corr;
        }
        l[h] = l[h] + p[h];
        m[h] = m_new;
      }
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const float vd = round_through<T>(vc[i] * vs);
#pragma unroll
        for (int h = 0; h < REP; ++h) o[h][i] = fmaf(p[h], vd, o[h][i]);
      }
    }
  }
  }

  if constexpr (ROW_PARTIALS) {
#pragma unroll
    for (int h = 0; h < REP; ++h) {
      const float m_wave = group_max<kWave>(m[h]);
      const float a = m[h] == -INFINITY ? 0.0f : exp2f(m[h] - m_wave);
      l[h] *= a;
      l[h] += dpp<kDppRor4>(l[h]);
      l[h] += dpp<kDppRor8>(l[h]);
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        float v = o[h][i] * a;
        v += dpp<kDppRor4>(v);
        v += dpp<kDppRor8>(v);
        o[h][i] = v;
      }
      m[h] = m_wave;
    }
    return;
  }
  // ---- merge the 16 quads of the wave (lanes with the same dq) ----------------------------------------
  // Inside a row of 16 lanes: rotate by 4, then by 8 (DPP, no LDS round trip); lane i then holds
  // quads i, i+4, i+8, i+12 of its row. Across the four rows: xor 16, xor 32.
  auto merge_with = [&](auto exchange) {
#pragma unroll
    for (int h = 0; h < REP; ++h) {
      const float m_o = exchange(m[h]);
      const float l_o = exchange(l[h]);
      const float m_new = fmaxf(m[h], m_o);
      const float a = m[h] == -INFINITY ? 0.0f : exp2f(m[h] - m_new);
      const float b = m_o == -INFINITY ? 0.0f : exp2f(m_o - m_new);
      l[h] = l[h] * a + l_o * b;
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const float o_o = exchange(o[h][i]);
        o[h][i] = o[h][i] * a + o_o * b;
      }
      m[h] = m_new;
    }
  };
  merge_with([](float v) { return dpp<kDppRor4>(v); });
  merge_with([](float v) { return dpp<kDppRor8>(v); });
  merge_with([](float v) { return __shfl_xor(v, 16, kWave); });
  merge_with([](float v) { return __shfl_xor(v, 32, kWave); });
}

template <typename T, int BITS, int D, int REP>
__global__ __launch_bounds__(kAttnThreads) void kv_decode_attn_kernel(
    const T* __restrict__ q, const uint8_t* __restrict__ k_codes, const uint8_t* __restrict__ v_codes,
    const float* __restrict__ k_scale, const float* __restrict__ v_scale, T* __restrict__ out,
    float* __restrict__ ws_part, int* __restrict__ ws_count, const int32_t* __restrict__ len_dev,
    const float sm_scale_log2, const int t_max, const int chunk) {
  constexpr int DPL = D / 4;           // head-dim elements per lane
  constexpr int ROWB = BITS == 8 ? D : D / 2;
  constexpr int REC = D + 2;           // floats per partial record: max, sum, weighted output
  __shared__ float s_rec[kAttnWaves][REP][REC];
  __shared__ int s_last;

  const int split = blockIdx.x, n_splits = gridDim.x, kvh = blockIdx.y;
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  const int tk = lane >> 2, dq = lane & 3;
  const int len = min(len_dev[0], t_max);
  const int t_begin = split * chunk, t_end = min(t_begin + chunk, len);

  // this lane's quarter of each query head, pre-scaled so exp2 can be used
  float qf[REP][DPL];
#pragma unroll
  for (int h = 0; h < REP; ++h)
#pragma unroll
    for (int i = 0; i < DPL; ++i)
      qf[h][i] = to_float(q[(static_cast<int64_t>(kvh) * REP + h) * D + dq * DPL + i]) * sm_scale_log2;

  float m[REP], l[REP], o[REP][DPL];
  attend_range<T, BITS, D, REP>(qf, k_codes + static_cast<int64_t>(kvh) * t_max * ROWB,
                                v_codes + static_cast<int64_t>(kvh) * t_max * ROWB,
                                k_scale + static_cast<int64_t>(kvh) * t_max,
                                v_scale + static_cast<int64_t>(kvh) * t_max, t_begin + wv * kTokPerIter, t_end,
                                kAttnWaves * kTokPerIter, tk, dq, m, l, o);
  if (tk == 0) {
#pragma unroll
    for (int h = 0; h < REP; ++h) {
      if (dq == 0) {
        s_rec[wv][h][0] = m[h];
        s_rec[wv][h][1] = l[h];
      }
#pragma unroll
      for (int i = 0; i < DPL; ++i) s_rec[wv][h][2 + dq * DPL + i] = o[h][i];
    }
  }
  __syncthreads();

  // ---- merge the waves; thread (h, d) for d < D ------------------------------------------------------
  float* my_part = ws_part + ((static_cast<int64_t>(kvh) * n_splits + split) * REP) * REC;
  for (int item = threadIdx.x; item < REP * D; item += kAttnThreads) {
    const int h = item / D, d = item % D;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) mm = fmaxf(mm, s_rec[w][h][0]);
    float ll = 0.0f, oo = 0.0f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float a = s_rec[w][h][0] == -INFINITY ? 0.0f : exp2f(s_rec[w][h][0] - mm);
      ll += s_rec[w][h][1] * a;
      oo += s_rec[w][h][2 + d] * a;
    }
    my_part[h * REC + 2 + d] = oo;
    if (d == 0) {
      my_part[h * REC] = mm;
      my_part[h * REC + 1] = ll;
    }
  }

  // ---- last workgroup of this kv head merges the splits ------------------------------------------------
  __threadfence();
  __syncthreads();
  if (threadIdx.x == 0) {
    const int arrived = atomicAdd(&ws_count[kvh], 1);
    s_last = arrived == n_splits - 1;
  }
  __syncthreads();
  if (!s_last) return;
  __threadfence();
  const float* parts = ws_part + static_cast<int64_t>(kvh) * n_splits * REP * REC;
  for (int item = threadIdx.x; item < REP * D; item += kAttnThreads) {
    const int h = item / D, d = item % D;
    float mm = -INFINITY;
    for (int s2 = 0; s2 < n_splits; ++s2) mm = fmaxf(mm, parts[(s2 * REP + h) * REC]);
    float ll = 0.0f, oo = 0.0f;
    for (int s2 = 0; s2 < n_splits; ++s2) {
      const float ms = parts[(s2 * REP + h) * REC];
      const float a = ms == -INFINITY ? 0.0f : exp2f(ms - mm);
      ll += parts[(s2 * REP + h) * REC + 1] * a;
      oo += parts[(s2 * REP + h) * REC + 2 + d] * a;
    }
    out[(static_cast<int64_t>(kvh) * REP + h) * D + d] = from_float<T>(ll > 0.0f ? oo / ll : 0.0f);
  }
  if (threadIdx.x == 0) ws_count[kvh] = 0;  // ready for the next launch
}

// ---- one decode step of attention in one launch ----------------------------------------------------
// RoPE on the new token's query and key, quantize-and-append of its key and value, and
// attention over the whole cache including that token. One workgroup of 16 waves per QUERY
// head: a wave step covers 16 tokens, so a workgroup covers 256 tokens per step and a context
// of a few thousand tokens is a handful of steps, each with the next step's loads already in
// flight. Nothing crosses workgroups: every workgroup rotates and quantizes the new token's
// key and value itself (64 values; the one whose query head is the first of its kv head also
// writes them to the cache) and attends to that token from LDS, to the older ones from the
// cache. The cache codes of a kv head are therefore read by its 4 query-head workgroups, from
// L2 after the first. RoPE follows transformers' apply_rotary_pos_emb with its rounding
// points: dtype(dtype(x * cos) + dtype(rotate_half(x) * sin)).
constexpr int kFusedWaves = 16;
constexpr int kFusedThreads = kFusedWaves * kWave;

template <typename T, int D>
__device__ __forceinline__ float rope_element(const T* x, const T* cos_row, const T* sin_row, int i) {
  const float xi = to_float(x[i]);
  const float rot = i < D / 2 ? -to_float(x[i + D / 2]) : to_float(x[i - D / 2]);
  const float a = round_through<T>(xi * to_float(cos_row[i]));
  const float b = round_through<T>(rot * to_float(sin_row[i]));
  return round_through<T>(a + b);
}

template <typename T, int BITS, int D>
__global__ __launch_bounds__(kFusedThreads) void kv_rope_append_attend_kernel(
    const T* __restrict__ qkv, const T* __restrict__ cos_table, const T* __restrict__ sin_table,
    uint8_t* __restrict__ k_codes, uint8_t* __restrict__ v_codes, float* __restrict__ k_scale,
    float* __restrict__ v_scale, T* __restrict__ out, const int32_t* __restrict__ pos_dev,
    const float sm_scale_log2, const int q_heads, const int kv_heads, const int t_max) {
  constexpr int DPL = D / 4;
  constexpr int ROWB = BITS == 8 ? D : D / 2;
  constexpr int REC = D + 2;
  __shared__ float s_q[D];
  __shared__ float s_new[2][D];  // the new token's key and value as the cache will return them
  __shared__ float s_rec[kFusedWaves][REC];

  const int qh = blockIdx.x;
  const int rep = q_heads / kv_heads;
  const int kvh = qh / rep;
  const bool writer = qh % rep == 0;
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  const int tk = lane >> 2, dq = lane & 3;
  const int pos = min(max(pos_dev[0], 0), t_max - 1);
  const T* cos_row = cos_table + static_cast<int64_t>(pos) * D;
  const T* sin_row = sin_table + static_cast<int64_t>(pos) * D;

  // the cache reads of the first attention step do not depend on phase A: request them now
  const uint8_t* kbase = k_codes + static_cast<int64_t>(kvh) * t_max * ROWB;
  const uint8_t* vbase = v_codes + static_cast<int64_t>(kvh) * t_max * ROWB;
  const float* ksc = k_scale + static_cast<int64_t>(kvh) * t_max;
  const float* vsc = v_scale + static_cast<int64_t>(kvh) * t_max;
  const int t_mine = wv * kTokPerIter;
  AttnPrefetch<BITS, DPL> first;
  if (t_mine < pos) first = attn_prefetch<BITS, DPL>(kbase, vbase, ksc, vsc, min(t_mine + tk, pos - 1), dq);

  // ---- phase A: wave 0 rotates the query, wave 1 rotates + quantizes K, wave 2 quantizes V ------------
  if (wv == 0) {
    const T* q = qkv + static_cast<int64_t>(qh) * D;
    for (int i = lane; i < D; i += kWave) s_q[i] = rope_element<T, D>(q, cos_row, sin_row, i) * sm_scale_log2;
  } else if (wv <= 2) {
    const bool is_v = wv == 2;
    const T* src = qkv + (static_cast<int64_t>(q_heads) + (is_v ? kv_heads : 0) + kvh) * D;
    const float qmax = static_cast<float>((1 << (BITS - 1)) - 1);
    const float qmin = -qmax - 1.0f;
    float f[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int d = lane + e * kWave;
      f[e] = 0.0f;
      if (d < D) f[e] = is_v ? to_float(src[d]) : rope_element<T, D>(src, cos_row, sin_row, d);
    }
    const int64_t slot = static_cast<int64_t>(kvh) * t_max + pos;
    uint8_t* codes = is_v ? v_codes : k_codes;
    if constexpr (BITS == 16) {
      // the unquantized cache: the rotated key / the value as the model's dtype holds them, scale 1
      if (writer && lane == 0) (is_v ? v_scale : k_scale)[slot] = 1.0f;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = lane + e * kWave;
        if (d < D) {
          s_new[is_v ? 1 : 0][d] = f[e];   // (already a value of T: RoPE rounds its result, V is read as T)
          if (writer) reinterpret_cast<T*>(codes)[slot * D + d] = from_float<T>(f[e]);
        }
      }
      return;
    }
    const float amax = group_max<kWave>(fmaxf(fabsf(f[0]), fabsf(f[1])));
    const float scale = scale_from_amax(amax, qmax);
    if (writer && lane == 0) (is_v ? v_scale : k_scale)[slot] = scale;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int d = lane + e * kWave;
      const float qv = quant_code(f[e], scale, qmin, qmax);
      if (d < D) s_new[is_v ? 1 : 0][d] = round_through<T>(qv * scale);
      const int code = static_cast<int>(qv);
      if constexpr (BITS == 8) {
        if (writer && d < D) codes[slot * D + d] = static_cast<uint8_t>(code);
      } else if constexpr (BITS == 4) {
        const int mine = (code + 8) & 0xf;
        const int other = dpp<kDppXor1>(mine);
        if (writer && (lane & 1) == 0 && d < D) codes[slot * (D / 2) + d / 2] = static_cast<uint8_t>(mine | (other << 4));
      }
    }
  }
  __syncthreads();

  // ---- phase B: tokens 0 .. pos-1 from the cache, token pos from LDS -------------------------------------
  float qf[1][DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) qf[0][i] = s_q[dq * DPL + i];
  float m[1], l[1], o[1][DPL];
  attend_range<T, BITS, D, 1>(qf, kbase, vbase, ksc, vsc, t_mine, pos, kFusedWaves * kTokPerIter, tk, dq, m, l, o,
                              &first);
  if (wv == kFusedWaves - 1) {
    // every lane with the same dq holds the same merged record; fold the new token into it
    float sc = 0.0f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) sc = fmaf(qf[0][i], s_new[0][dq * DPL + i], sc);
    sc += dpp<kDppXor1>(sc);
    sc += dpp<kDppXor2>(sc);
    const float m_new = fmaxf(m[0], sc);
    const float corr = m[0] == -INFINITY ? 0.0f : exp2f(m[0] - m_new);
    const float pnew = exp2f(sc - m_new);
    l[0] = l[0] * corr + pnew;
#pragma unroll
    for (int i = 0; i < DPL; ++i) o[0][i] = fmaf(pnew, s_new[1][dq * DPL + i], o[0][i] * corr);
    m[0] = m_new;
  }
  if (tk == 0) {
    if (dq == 0) {
      s_rec[wv][0] = m[0];
      s_rec[wv][1] = l[0];
    }
#pragma unroll
    for (int i = 0; i < DPL; ++i) s_rec[wv][2 + dq * DPL + i] = o[0][i];
  }
  __syncthreads();
  if (threadIdx.x < D) {
    const int d = threadIdx.x;
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kFusedWaves; ++w) mm = fmaxf(mm, s_rec[w][0]);
    float ll = 0.0f, oo = 0.0f;
#pragma unroll
    for (int w = 0; w < kFusedWaves; ++w) {
      const float a = s_rec[w][0] == -INFINITY ? 0.0f : exp2f(s_rec[w][0] - mm);
      ll += s_rec[w][1] * a;
      oo += s_rec[w][2 + d] * a;
    }
    out[static_cast<int64_t>(qh) * D + d] = from_float<T>(ll > 0.0f ? oo / ll : 0.0f);
  }
}

// ---- the same step spread over more of the chip ------------------------------------------------------
// One workgroup per (query head, split): split s of S takes the 64-token slabs s, s + S, ... of the
// cache (balanced at every context length, nothing to compute from the length), the last split
// also the new token. A workgroup is 4 waves, so with S = 8 a 32-head model fills 256 CUs with one
// workgroup each and the dequantization work of a head runs on 8 CUs instead of one. What leaves a
// workgroup is a partial record (max, sum, weighted output relative to that max) per (head, split);
// the records are merged by whoever consumes the attention output: llmq_kv_attend_merge, or the
// o_proj GEMV while it stages its activation (llmq_wq_gemv_attn_merge), which costs no launch.
constexpr int kSplitWaves = 4;
constexpr int kSplitThreads = kSplitWaves * kWave;
constexpr int kSplitSlab = kSplitWaves * kTokPerIter;  // 64 tokens per workgroup step
constexpr int kSplitPrefetch = 2;  // steps of cache rows a wave requests before it knows the position

// Phase A of a split attention step: the workgroup's waves rotate its query heads into s_q (times the softmax
// scale in log2 units; one head: wave 0), and in the last split waves 1 / 2 quantize the new token's K / V: the
// dequantized values go to s_new for the workgroup's own attention, the codes and scales (writer only: one
// workgroup per kv head) into the cache at `pos`.
template <typename T, int BITS, int D, int HEADS>
__device__ __forceinline__ void split_phase_a(const T* __restrict__ qkv, const T* __restrict__ cos_row,
                                              const T* __restrict__ sin_row, uint8_t* __restrict__ k_codes,
                                              uint8_t* __restrict__ v_codes, float* __restrict__ k_scale,
                                              float* __restrict__ v_scale, const float sm_scale_log2, const int q_heads,
                                              const int kv_heads, const int t_max, const int pos, const int qh0,
                                              const int kvh, const bool last_split, const bool writer, const int lane,
                                              const int wv, float (*s_q)[D], float (*s_new)[D]) {
  for (int h = wv; h < HEADS; h += kSplitWaves) {
    const T* q = qkv + static_cast<int64_t>(qh0 + h) * D;
    for (int i = lane; i < D; i += kWave) s_q[h][i] = rope_element<T, D>(q, cos_row, sin_row, i) * sm_scale_log2;
  }
  if (wv >= 1 && wv <= 2 && last_split) {
    const bool is_v = wv == 2;
    const T* src = qkv + (static_cast<int64_t>(q_heads) + (is_v ? kv_heads : 0) + kvh) * D;
    const float qmax = static_cast<float>((1 << (BITS - 1)) - 1);
    const float qmin = -qmax - 1.0f;
    float f[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int d = lane + e * kWave;
      f[e] = 0.0f;
      if (d < D) f[e] = is_v ? to_float(src[d]) : rope_element<T, D>(src, cos_row, sin_row, d);
    }
    const int64_t slot = static_cast<int64_t>(kvh) * t_max + pos;
    uint8_t* codes = is_v ? v_codes : k_codes;
    if constexpr (BITS == 16) {
      // the unquantized cache: the rotated key / the value as the model's dtype holds them, scale 1
      if (writer && lane == 0) (is_v ? v_scale : k_scale)[slot] = 1.0f;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int d = lane + e * kWave;
        if (d < D) {
          s_new[is_v ? 1 : 0][d] = f[e];   // (already a value of T: RoPE rounds its result, V is read as T)
          if (writer) reinterpret_cast<T*>(codes)[slot * D + d] = from_float<T>(f[e]);
        }
      }
      return;
    }
    const float amax = group_max<kWave>(fmaxf(fabsf(f[0]), fabsf(f[1])));
    const float scale = scale_from_amax(amax, qmax);
    if (writer && lane == 0) (is_v ? v_scale : k_scale)[slot] = scale;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int d = lane + e * kWave;
      const float qv = quant_code(f[e], scale, qmin, qmax);
      if (d < D) s_new[is_v ? 1 : 0][d] = round_through<T>(qv * scale);
      const int code = static_cast<int>(qv);
      if constexpr (BITS == 8) {
        if (writer && d < D) codes[slot * D + d] = static_cast<uint8_t>(code);
      } else if constexpr (BITS == 4) {
        const int mine = (code + 8) & 0xf;
        const int other = dpp<kDppXor1>(mine);
        if (writer && (lane & 1) == 0 && d < D) codes[slot * (D / 2) + d / 2] = static_cast<uint8_t>(mine | (other << 4));
      }
    }
  }
}

// HEADS: query heads of one kv head that a workgroup takes together (1, or 4 under grouped-query
// attention with long caches). Every cache row is then read and dequantized once for the four of
// them: beyond a few thousand tokens the step is bound by exactly that arithmetic, which one
// workgroup per query head repeats q_heads / kv_heads times.
template <typename T, int BITS, int D, int HEADS>
__global__ __launch_bounds__(kSplitThreads) void kv_rope_append_attend_split_kernel(
    const T* __restrict__ qkv, const T* __restrict__ cos_table, const T* __restrict__ sin_table,
    uint8_t* __restrict__ k_codes, uint8_t* __restrict__ v_codes, float* __restrict__ k_scale,
    float* __restrict__ v_scale, float* __restrict__ partials, const int32_t* __restrict__ pos_dev,
    const float sm_scale_log2, const int q_heads, const int kv_heads, const int t_max) {
  constexpr int DPL = D / 4;
  constexpr int ROWB = D * BITS / 8;
  constexpr int REC = D + 2;                    // per-wave record in LDS
  constexpr int GREC = D + kAttnRecordHeader;  // per-split record in global memory
  __shared__ float s_q[HEADS][D];
  __shared__ float s_new[2][D];
  __shared__ float s_rec[kSplitWaves][4][HEADS][REC];  // per wave and row of 16 lanes: (wave max, sum, output)
  __shared__ float s_new_score[HEADS];                 // the new token's scores (last split), else -inf

  const int qh0 = blockIdx.x * HEADS, split = blockIdx.y, n_splits = gridDim.y;  // heads qh0 .. qh0 + HEADS - 1
  const bool last_split = split == n_splits - 1;
  const int rep = q_heads / kv_heads;  // a multiple of HEADS
  const int kvh = qh0 / rep;
  const bool writer = last_split && qh0 % rep == 0;
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  const int tk = lane >> 2, dq = lane & 3;

  // The wave's first steps of cache rows do not depend on the position (rows up to t_max - 1 exist;
  // what lies at or beyond the position is dropped later): requested first, so that the position's
  // own round trip and phase A run under them.
  const uint8_t* kbase = k_codes + static_cast<int64_t>(kvh) * t_max * ROWB;
  const uint8_t* vbase = v_codes + static_cast<int64_t>(kvh) * t_max * ROWB;
  const float* ksc = k_scale + static_cast<int64_t>(kvh) * t_max;
  const float* vsc = v_scale + static_cast<int64_t>(kvh) * t_max;
  const int t_mine = split * kSplitSlab + wv * kTokPerIter;
  const int t_step = n_splits * kSplitSlab;
  AttnPrefetch<BITS, DPL> first[kSplitPrefetch];
#pragma unroll
  for (int r = 0; r < kSplitPrefetch; ++r) {
    first[r] = attn_prefetch<BITS, DPL>(kbase, vbase, ksc, vsc, min(t_mine + r * t_step + tk, t_max - 1), dq);
  }

  const int pos = min(max(pos_dev[0], 0), t_max - 1);
  const T* cos_row = cos_table + static_cast<int64_t>(pos) * D;
  const T* sin_row = sin_table + static_cast<int64_t>(pos) * D;

  // ---- phase A: the waves rotate the query heads (one head: wave 0); in the last split wave 1 / 2 also
  // prepare the new K / V ----------------------------------------------------------------------------
  split_phase_a<T, BITS, D, HEADS>(qkv, cos_row, sin_row, k_codes, v_codes, k_scale, v_scale, sm_scale_log2, q_heads,
                                   kv_heads, t_max, pos, qh0, kvh, last_split, writer, lane, wv, s_q, s_new);
  __syncthreads();

  // ---- phase B: this split's slabs of tokens 0 .. pos-1, and (last split) token pos from LDS ------------
  float qf[HEADS][DPL];
#pragma unroll
  for (int h = 0; h < HEADS; ++h)
#pragma unroll
    for (int i = 0; i < DPL; ++i) qf[h][i] = s_q[h][dq * DPL + i];
  float m[HEADS], l[HEADS], o[HEADS][DPL];
  attend_range<T, BITS, D, HEADS, kSplitPrefetch, true>(qf, kbase, vbase, ksc, vsc, t_mine, pos, t_step, tk, dq, m, l,
                                                        o, first, t_max - 1);
  if (wv == kSplitWaves - 1) {
    // the new token is a record of its own: scores here, its value is s_new[1]
#pragma unroll
    for (int h = 0; h < HEADS; ++h) {
      float sc = 0.0f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) sc = fmaf(qf[h][i], s_new[0][dq * DPL + i], sc);
      sc += dpp<kDppXor1>(sc);
      sc += dpp<kDppXor2>(sc);
      if (lane == 0) s_new_score[h] = last_split ? sc : -INFINITY;
    }
  }
  if ((tk & 3) == 0) {
    const int row = lane >> 4;
#pragma unroll
    for (int h = 0; h < HEADS; ++h) {
      if (dq == 0) {
        s_rec[wv][row][h][0] = m[h];
        s_rec[wv][row][h][1] = l[h];
      }
#pragma unroll
      for (int i = 0; i < DPL; ++i) s_rec[wv][row][h][2 + dq * DPL + i] = o[h][i];
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < HEADS * D; item += kSplitThreads) {
    const int h = item / D, d = item - h * D;
    const float new_score = s_new_score[h];
    float mm = new_score;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w) mm = fmaxf(mm, s_rec[w][0][h][0]);
    float ll = 0.0f, oo = 0.0f;
#pragma unroll
    for (int w = 0; w < kSplitWaves; ++w) {
      const float a = s_rec[w][0][h][0] == -INFINITY ? 0.0f : exp2f(s_rec[w][0][h][0] - mm);
      ll += ((s_rec[w][0][h][1] + s_rec[w][1][h][1]) + (s_rec[w][2][h][1] + s_rec[w][3][h][1])) * a;
      oo += ((s_rec[w][0][h][2 + d] + s_rec[w][1][h][2 + d]) + (s_rec[w][2][h][2 + d] + s_rec[w][3][h][2 + d])) * a;
    }
    if (new_score != -INFINITY) {
      const float b = exp2f(new_score - mm);
      ll += b;
      oo = fmaf(b, s_new[1][d], oo);
    }
    float* rec = partials + (static_cast<int64_t>(qh0 + h) * n_splits + split) * GREC;
    if (d == 0) {
      rec[0] = mm;
      rec[1] = ll;
    }
    rec[kAttnRecordHeader + d] = oo;
  }
}

// ---- the same step under grouped-query attention on the int8 matrix core (caches of 2048 rows and more) --------
// Beyond a few thousand tokens the step above is bound by the vector ALU: every code is converted to a float and
// multiplied there (~500 instructions per 16 tokens and four heads, 2.6 TB/s of cache bytes at best). Here the int8
// codes are matrix-core operands as they lie in the cache (v_mfma_i32_16x16x64_i8), for the four query heads of a
// kv head at once, and the vector ALU is left with the softmax: ~2 instructions per token and head.
//
//   scores   S[(head, digit)][token] = sum_d Q[(head, digit)][d] * Kcode[token][d]: the rotated, scaled query of a
//            head as a block-floating-point integer (22 bits below the head's abs-max) cut in three signed base-256
//            digits, one operand row each (the GEMV's trick); a lane ends up with the three digit sums of one
//            (token, head) and combines them: score = (S0 + 256 S1 + 65536 S2) * 2^-sh * kscale[token].
//   values   O[(head, digit)][d] = sum_t W[(head, digit)][t] * Vcode[t][d] with W = p * vscale[t], p the softmax
//            weight relative to the running maximum, as an integer below the largest W of the head in the 64-token
//            step: 14 bits in two digits (fp32 models: 22 in three). The weights reach operand layout (tokens along a lane's 16 bytes)
//            through 1 KB of LDS per wave; V's codes, token-major in the cache, are read from LDS transposed
//            (ds_read_b64_tr_b8: in a group of 16 lanes, byte j of result lane l is byte l % 8 of what lane
//            2 j + l / 8 points at).
//
// Both sums are exact integers; what differs from the step above is that K and V enter as code * scale without the
// rounding to the model's dtype in between, and the resolution of the weights (2^-14 beside a 16-bit output's 2^-8 or
// 2^-11; 2^-22, fp32's own, for fp32 models): within the tolerance the attention output is held to, and for fp32
// models at fp32's rounding level (rel-L2 1e-6 against the float64 oracle).
// A wave walks 64-token slabs (wave w of split s: slabs 4 s + w, 4 s + w + 4 S, ...) through two LDS stages of its
// own, both in flight while it computes, filled by DMA (codes of K and V with their 16-byte pieces XOR-swizzled by row for the operand reads and the
// transposed reads, and the two scale vectors): no barrier inside the loop. The records it leaves are those of the
// kernel above. Measured, 32 heads on 8 kv heads of 64, int8, per layer: 5.7 us at 2048 cached tokens (8 splits; the
// step above 6.6), 12 us at 32 000 (32 splits; 20.7), 33 us at 131 000 (64 splits; 55).
// 4-bit codes: a lane's eight packed bytes (16 codes) become two operand halves, the low nibbles (even dimensions) and
// the high ones (odd), with the query's digits laid out in the same order; V's packed bytes go through the same
// transposed read and split into the operand of an even and of an odd dimension. The nibbles are code + 8: the 8
// leaves through the C operand of the multiply (- 8 * the sum of the other operand's row, an integer the lane has).
typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef int v2i32 __attribute__((ext_vector_type(2)));

constexpr int kMfHeads = 4;   // query heads of one kv head per workgroup
constexpr int kMfSlab = 64;   // tokens of one wave step
// caches shorter than this keep the vector-ALU form, whose K and V pass through the model's dtype as the reference's
// cache holds them; the step is bound by latency there whichever form runs
constexpr int kMfMinCache = 2048;

template <int BITS, int D> struct MfLds {
  static constexpr int kRowBytes = D * BITS / 8;                  // a token's codes: 32, 64 or 128 bytes
  static constexpr int kPieces = kRowBytes / 16;                  // 16-byte pieces of a row of codes
  static constexpr int kTransfers = kMfSlab * kRowBytes / 1024;   // 1 KB DMA instructions per tensor and slab
  static constexpr int kCodes = kMfSlab * kRowBytes;              // bytes of a slab's K (or V) codes
  static constexpr int kStage = 2 * kCodes + 2 * kMfSlab * 4;     // K codes, V codes, K scales, V scales
  static constexpr int kP = 16 * kMfSlab;                         // the weights as operand rows: [16 rows][64 tokens] bytes
  static constexpr int kWaveBytes = 2 * kStage + kP + 512;        // two stages, the weights, per-head constants
  static constexpr int kRec = D + 2;                              // a wave's (max, sum, output) per head
  static constexpr int kHeaderFloats = kMfHeads * D + 2 * D + kSplitWaves * kMfHeads * kRec + 2 * kMfHeads;
  static constexpr int kHeaderBytes = (kHeaderFloats * 4 + 255) / 256 * 256;
  static constexpr int kBytes = kHeaderBytes + kSplitWaves * kWaveBytes;   // int8: 82 KB (D = 64), 150 KB (D = 128)
  // Slot of a row's 16-byte piece p in LDS is p ^ swizzle(row); both depend on the row's bytes only. K is read as
  // operands: 16 lanes read the same piece (or, 4-bit, the same eight bytes) of 16 consecutive rows and have to land
  // in different banks. V is read transposed: a lane points at 8 bytes of row 16 g + 8 half + s / 2 (s its index
  // among its 16 lanes), two such groups of lanes go together.
  static __device__ __forceinline__ int swizzle_k(int row) {
    return kRowBytes == 32 ? (row >> 3) & 1 : kRowBytes == 64 ? (row >> 2) & 3 : (row >> 1) & 7;
  }
  static __device__ __forceinline__ int swizzle_v(int row) {
    return kRowBytes == 32   ? (row >> 4) & 1
           : kRowBytes == 64 ? ((row >> 2) & 1) | (((row >> 4) & 1) << 1)
                             : ((row >> 1) & 3) | (((row >> 4) & 1) << 2);
  }
};

template <typename T, int BITS, int D>
__global__ __launch_bounds__(kSplitThreads, 2) void kv_rope_append_attend_split_mfma_kernel(
    const T* __restrict__ qkv, const T* __restrict__ cos_table, const T* __restrict__ sin_table,
    uint8_t* __restrict__ k_codes, uint8_t* __restrict__ v_codes, float* __restrict__ k_scale,
    float* __restrict__ v_scale, float* __restrict__ partials, const int32_t* __restrict__ pos_dev,
    const float sm_scale_log2, const int q_heads, const int kv_heads, const int t_max) {
  using L = MfLds<BITS, D>;
  constexpr int HEADS = kMfHeads;
  constexpr int RB = L::kRowBytes;
  constexpr uint32_t kNibbles = 0x0f0f0f0fu;
  constexpr int GREC = D + kAttnRecordHeader;
  constexpr int kKSteps = D / 64;    // matrix-core steps along a head's dimensions
  constexpr int kWDigits = sizeof(T) == 4 ? 3 : 2;   // base-256 digits of the softmax weights (see the loop)
  constexpr int kDTiles = D / 16;    // tiles of 16 dimensions of the output
  extern __shared__ __attribute__((aligned(16))) unsigned char mf_smem[];
  float (*s_q)[D] = reinterpret_cast<float (*)[D]>(mf_smem);
  float (*s_new)[D] = reinterpret_cast<float (*)[D]>(mf_smem + HEADS * D * 4);
  float* s_rec = reinterpret_cast<float*>(mf_smem + (HEADS + 2) * D * 4);   // [waves][HEADS][kRec]
  float* s_new_score = s_rec + kSplitWaves * HEADS * L::kRec;
  float* s_qmax = s_new_score + HEADS;   // abs-max of each rotated, scaled query head

  const int qh0 = blockIdx.x * HEADS, split = blockIdx.y, n_splits = gridDim.y;
  const bool last_split = split == n_splits - 1;
  const int rep = q_heads / kv_heads;  // a multiple of HEADS
  const int kvh = qh0 / rep;
  const bool writer = last_split && qh0 % rep == 0;
  const int lane = threadIdx.x & (kWave - 1);
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int j = lane & 15, g = lane >> 4;   // (column, row block) of the matrix core's lanes

  unsigned char* mine = mf_smem + L::kHeaderBytes + wv * L::kWaveBytes;
  unsigned char* pbuf = mine + 2 * L::kStage;
  float* qinv_of = reinterpret_cast<float*>(pbuf + L::kP);        // [4]: 2^-sh per head
  int* qpart_of = reinterpret_cast<int*>(pbuf + L::kP + 64);       // [4 blocks][16 rows]: sums of the query's digits

  const uint8_t* kbase = k_codes + static_cast<int64_t>(kvh) * t_max * RB;
  const uint8_t* vbase = v_codes + static_cast<int64_t>(kvh) * t_max * RB;
  const float* ksc = k_scale + static_cast<int64_t>(kvh) * t_max;
  const float* vsc = v_scale + static_cast<int64_t>(kvh) * t_max;
  // transfer i of a slab's codes lands in LDS bytes 1024 i + 16 lane: row (1024 / row bytes) i + lane / pieces, slot
  // lane % pieces
  auto request = [&](const int t0, const int stage) {
    unsigned char* st = mine + stage * L::kStage;
#pragma unroll
    for (int i = 0; i < L::kTransfers; ++i) {
      const int row = (1024 / RB) * i + lane / L::kPieces, slot = lane % L::kPieces;
      const int64_t t = min(t0 + row, t_max - 1);   // (rows past the cache's end: the last row again)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(kbase + t * RB + 16 * (slot ^ L::swizzle_k(row))),
                                       reinterpret_cast<u32x4*>(st + 1024 * i), 16, 0, 0);
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(vbase + t * RB + 16 * (slot ^ L::swizzle_v(row))),
                                       reinterpret_cast<u32x4*>(st + L::kCodes + 1024 * i), 16, 0, 0);
    }
    const int64_t ts = min(t0 + lane, t_max - 1);
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(ksc + ts),
                                     reinterpret_cast<uint32_t*>(st + 2 * L::kCodes), 4, 0, 0);
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint32_t*>(vsc + ts),
                                     reinterpret_cast<uint32_t*>(st + 2 * L::kCodes + kMfSlab * 4), 4, 0, 0);
  };
  constexpr int kRequestLoads = 2 * L::kTransfers + 2;

  // the wave's first slab does not depend on the position (rows up to t_max - 1 exist; what lies at or beyond the
  // position is masked later): requested first, so that the position's round trip and phase A run under it
  int t0 = (split * kSplitWaves + wv) * kMfSlab;
  const int t_step = n_splits * kSplitWaves * kMfSlab;
  request(t0, 0);

  const int pos = min(max(pos_dev[0], 0), t_max - 1);
  const T* cos_row = cos_table + static_cast<int64_t>(pos) * D;
  const T* sin_row = sin_table + static_cast<int64_t>(pos) * D;
  // two slabs in flight per wave from here on: the second goes out as soon as the position says it exists
  if (t0 + t_step < pos) request(t0 + t_step, 1);
  split_phase_a<T, BITS, D, HEADS>(qkv, cos_row, sin_row, k_codes, v_codes, k_scale, v_scale, sm_scale_log2, q_heads,
                                kv_heads, t_max, pos, qh0, kvh, last_split, writer, lane, wv, s_q, s_new);
  // operand rows the weights never reach (one or two of a head's four) stay zero
  for (int i = lane; i < L::kP / 4; i += kWave) reinterpret_cast<uint32_t*>(pbuf)[i] = 0u;
  {
    // the head this wave has just rotated (one per wave): its abs-max, for the digits below
    static_assert(HEADS == kSplitWaves, "a head per wave");
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < D / kWave; ++i) a = fmaxf(a, fabsf(s_q[wv][lane + i * kWave]));
    a = group_max<kWave>(a);
    if (lane == 0) s_qmax[wv] = a;
  }
  __syncthreads();

  // ---- the query heads as operand rows: lane (row = j = 4 head + digit, block g) holds d = 64 step + 16 g .. + 15
  // (4-bit codes: in the order the nibbles of eight bytes come apart, the even dimensions, then the odd ones)
  v4i32 qa[kKSteps];
  v4i32 q_bias = v4i32{0, 0, 0, 0};   // 4-bit: - 8 * (sum of the digits of rows 4 g .. 4 g + 3), the scores' C operand
  {
    const int h = j >> 2, digit = j & 3;
    const float amax = s_qmax[h];
    const uint32_t e = __builtin_bit_cast(uint32_t, amax) >> 23;   // amax = f 2^(e - 126), f in [0.5, 1)
    const bool usable = e >= 22u && e < 255u;                       // (below 2^-105 the head counts as zero)
    const float up = __builtin_bit_cast(float, (275u - e) << 23);  // 2^(148 - e): amax * up in [2^21, 2^22)
    const float down = __builtin_bit_cast(float, (e - 21u) << 23); // 2^(e - 148)
    // digit k of q = d0 + 256 d1 + 65536 d2 (each in [-128, 127]) is the sign-extended low byte of
    // (q + 128 + ... + 128 * 256^(k-1)) >> 8 k; the fourth row of a head is empty
    const int digit_add = digit == 1 ? 128 : digit == 2 ? 32896 : 0;
    const int digit_shift = 8 * (digit & 3);
    int digit_sum = 0;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      uint32_t words[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int b = 0; b < 16; ++b) {
        const int d_in_block = BITS == 8 ? b : (b < 8 ? 2 * b : 2 * (b - 8) + 1);
        const int qi = static_cast<int>(rintf(s_q[h][64 * ks + 16 * g + d_in_block] * up));
        const int digit_value = usable && digit < 3 ? static_cast<int>(static_cast<int8_t>((qi + digit_add) >> digit_shift)) : 0;
        words[b >> 2] |= static_cast<uint32_t>(digit_value & 0xff) << (8 * (b & 3));
        digit_sum += digit_value;
      }
      qa[ks] = v4i32{static_cast<int>(words[0]), static_cast<int>(words[1]), static_cast<int>(words[2]),
                     static_cast<int>(words[3])};
    }
    if (digit == 0 && g == 0) qinv_of[h] = usable ? down : 0.0f;
    if constexpr (BITS == 4) qpart_of[16 * g + j] = digit_sum;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  const float qinv = qinv_of[g];   // in the score tiles a lane's head is its row block
  if constexpr (BITS == 4) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = 4 * g + r;
      q_bias[r] = -8 * ((qpart_of[row] + qpart_of[16 + row]) + (qpart_of[32 + row] + qpart_of[48 + row]));
    }
  }

  // the rows this lane points at in a transposed read are 16 g + 8 half + j / 2: one swizzle for both halves
  const int swz_v_read = L::swizzle_v(16 * g + (j >> 1));
  float m_run = -INFINITY, l_part = 0.0f;
  float o_acc[kDTiles];   // head g, d = 16 tile + j
#pragma unroll
  for (int dt = 0; dt < kDTiles; ++dt) o_acc[dt] = 0.0f;
  int stage = 0;
  for (; t0 < pos; t0 += t_step, stage ^= 1) {
    // this slab is in `stage`; the next one, if there is one, has been requested into the other stage
    if (t0 + t_step < pos) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kRequestLoads) : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const unsigned char* st = mine + stage * L::kStage;
    const float* ks_of = reinterpret_cast<const float*>(st + 2 * L::kCodes);
    const float* vs_of = ks_of + kMfSlab;
    // ---- scores of the slab's four tiles of 16 tokens: lane = (token 16 c + j, head g)
    float sc[4], w[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int r = 16 * c + j;
      v4i32 acc = q_bias;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        v4i32 kb;
        if constexpr (BITS == 8) {
          kb = *reinterpret_cast<const v4i32*>(st + r * RB + 16 * ((4 * ks + g) ^ L::swizzle_k(r)));
        } else {
          // the lane's 16 codes are bytes 32 ks + 8 g .. + 7 of the row
          const u32x2 raw = *reinterpret_cast<const u32x2*>(st + r * RB + 16 * ((2 * ks + (g >> 1)) ^ L::swizzle_k(r)) +
                                                            8 * (g & 1));
          kb = v4i32{static_cast<int>(raw.x & kNibbles), static_cast<int>(raw.y & kNibbles),
                     static_cast<int>((raw.x >> 4) & kNibbles), static_cast<int>((raw.y >> 4) & kNibbles)};
        }
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(qa[ks], kb, acc, 0, 0, 0);
      }
      const float dot = fmaf(static_cast<float>(acc[2]), 65536.0f,
                             fmaf(static_cast<float>(acc[1]), 256.0f, static_cast<float>(acc[0])));
      sc[c] = t0 + r < pos ? dot * (ks_of[r] * qinv) : -INFINITY;
    }
    const float m_new = fmaxf(m_run, group_max<16>(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]))));
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);   // (the slab's first token is below pos: m_new is finite)
    float p_sum = 0.0f, w_max = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int r = 16 * c + j;
      const float p = __builtin_amdgcn_exp2f(sc[c] - m_new);
      p_sum += p;
      w[c] = t0 + r < pos ? p * vs_of[r] : 0.0f;
      w_max = fmaxf(w_max, w[c]);
    }
    l_part = fmaf(l_part, alpha, p_sum);
    m_run = m_new;
    // ---- the weights as integers below the head's largest in this slab: 14 bits in two digits for 16-bit models (whose
    // output keeps 8 or 11 bits), 22 bits in three digits, like the query's, for fp32 ones
    constexpr uint32_t kWBits = kWDigits == 3 ? 22u : 14u;
    w_max = group_max<16>(w_max);
    const uint32_t we = max(__builtin_bit_cast(uint32_t, w_max) >> 23, kWBits - 1u);   // w_max = f 2^(we - 126)
    const float w_up = __builtin_bit_cast(float, (253u + kWBits - we) << 23);   // 2^(126 + bits - we): w * w_up < 2^bits
    const float w_down = __builtin_bit_cast(float, (we + 1u - kWBits) << 23);   // 2^(we - 126 - bits)
    int w_sum0 = 0, w_sum1 = 0, w_sum2 = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int wi = static_cast<int>(rintf(w[c] * w_up));
      const int d0 = static_cast<int8_t>(wi);
      const int r1 = (wi + 128) >> 8;   // (wi - d0) / 256
      const int d1 = kWDigits == 3 ? static_cast<int>(static_cast<int8_t>(r1)) : r1;
      pbuf[(4 * g) * kMfSlab + 16 * c + j] = static_cast<unsigned char>(d0);
      pbuf[(4 * g + 1) * kMfSlab + 16 * c + j] = static_cast<unsigned char>(d1);
      w_sum0 += d0;
      w_sum1 += d1;
      if constexpr (kWDigits == 3) {
        const int d2 = (wi + 32896) >> 16;
        pbuf[(4 * g + 2) * kMfSlab + 16 * c + j] = static_cast<unsigned char>(d2);
        w_sum2 += d2;
      }
    }
    v4i32 w_bias = v4i32{0, 0, 0, 0};   // 4-bit: - 8 * (sum over the slab of the head's digits), the values' C operand
    if constexpr (BITS == 4) {
      w_bias = v4i32{-8 * row16_sum(w_sum0), -8 * row16_sum(w_sum1), kWDigits == 3 ? -8 * row16_sum(w_sum2) : 0, 0};
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const v4i32 pa = *reinterpret_cast<const v4i32*>(pbuf + j * kMfSlab + 16 * g);   // row j, tokens 16 g .. 16 g + 15
    // ---- weighted values, 16 of the head's dimensions per tile: lane = (head g, d = 16 tile + j; 4-bit: tiles come
    // in pairs from 16 packed bytes a token, d = 32 pair + 2 j and + 1)
    const unsigned char* vrow = st + L::kCodes + (16 * g + (j >> 1)) * RB + 8 * (j & 1);
#pragma unroll
    for (int bt = 0; bt < RB / 16; ++bt) {
      const int at = 16 * (bt ^ swz_v_read);
      const v2i32 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) v2i32*)(vrow + at));                // tokens 16 g .. 16 g + 7
      const v2i32 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) v2i32*)(vrow + 8 * RB + at));       // 16 g + 8 .. 16 g + 15
      const v4i32 vb = v4i32{lo[0], lo[1], hi[0], hi[1]};
      if constexpr (BITS == 8) {
        const v4i32 acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(pa, vb, w_bias, 0, 0, 0);
        float sum = fmaf(static_cast<float>(acc[1]), 256.0f, static_cast<float>(acc[0]));
        if constexpr (kWDigits == 3) sum = fmaf(static_cast<float>(acc[2]), 65536.0f, sum);
        o_acc[bt] = fmaf(o_acc[bt], alpha, sum * w_down);
      } else {
        const v4i32 even = vb & static_cast<int>(kNibbles);
        const v4i32 odd = (vb >> 4) & static_cast<int>(kNibbles);
        const v4i32 acc_e = __builtin_amdgcn_mfma_i32_16x16x64_i8(pa, even, w_bias, 0, 0, 0);
        const v4i32 acc_o = __builtin_amdgcn_mfma_i32_16x16x64_i8(pa, odd, w_bias, 0, 0, 0);
        float sum_e = fmaf(static_cast<float>(acc_e[1]), 256.0f, static_cast<float>(acc_e[0]));
        float sum_o = fmaf(static_cast<float>(acc_o[1]), 256.0f, static_cast<float>(acc_o[0]));
        if constexpr (kWDigits == 3) {
          sum_e = fmaf(static_cast<float>(acc_e[2]), 65536.0f, sum_e);
          sum_o = fmaf(static_cast<float>(acc_o[2]), 65536.0f, sum_o);
        }
        o_acc[2 * bt] = fmaf(o_acc[2 * bt], alpha, sum_e * w_down);
        o_acc[2 * bt + 1] = fmaf(o_acc[2 * bt + 1], alpha, sum_o * w_down);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // (the stage and the weights are free again)
    if (t0 + 2 * t_step < pos) request(t0 + 2 * t_step, stage);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // (a wave with no slab below pos: its first request lands before it leaves)

  // ---- the waves meet: (max, sum, output) per wave and head, then the new token, then the split's record --------
  {
    const float l_row = row16_sum(l_part);
    float* rec = s_rec + (wv * HEADS + g) * L::kRec;
    if (j == 0) {
      rec[0] = m_run;
      rec[1] = l_row;
    }
#pragma unroll
    for (int dt = 0; dt < kDTiles; ++dt) {
      const int d = BITS == 8 ? 16 * dt + j : 32 * (dt >> 1) + 2 * j + (dt & 1);
      rec[2 + d] = o_acc[dt];
    }
  }
  if (wv == kSplitWaves - 1) {
    // the new token is a record of its own: its scores here, its value is s_new[1]
    float dot = 0.0f;
#pragma unroll
    for (int i = 0; i < D / 16; ++i) dot = fmaf(s_q[g][(D / 16) * j + i], s_new[0][(D / 16) * j + i], dot);
    dot = row16_sum(dot);
    if (j == 0) s_new_score[g] = last_split ? dot : -INFINITY;
  }
  __syncthreads();
  for (int item = threadIdx.x; item < HEADS * D; item += kSplitThreads) {
    const int h = item / D, d = item - h * D;
    const float new_score = s_new_score[h];
    float mm = new_score;
#pragma unroll
    for (int w2 = 0; w2 < kSplitWaves; ++w2) mm = fmaxf(mm, s_rec[(w2 * HEADS + h) * L::kRec]);
    float ll = 0.0f, oo = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < kSplitWaves; ++w2) {
      const float* rec = s_rec + (w2 * HEADS + h) * L::kRec;
      const float a = rec[0] == -INFINITY ? 0.0f : exp2f(rec[0] - mm);
      ll += rec[1] * a;
      oo += rec[2 + d] * a;
    }
    if (new_score != -INFINITY) {
      const float b = exp2f(new_score - mm);
      ll += b;
      oo = fmaf(b, s_new[1][d], oo);
    }
    float* out_rec = partials + (static_cast<int64_t>(qh0 + h) * n_splits + split) * GREC;
    if (d == 0) {
      out_rec[0] = mm;
      out_rec[1] = ll;
    }
    out_rec[kAttnRecordHeader + d] = oo;
  }
}

// out[h, d0 .. d0+7] from the records of head h: one thread per eight elements.
template <typename T>
__global__ __launch_bounds__(256) void kv_attend_merge_kernel(const float* __restrict__ partials, T* __restrict__ out,
                                                              const int total, const int head_dim,
                                                              const int n_splits) {
  const int i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= total) return;
  const int h = i / head_dim, d0 = i - h * head_dim;
  float f[8];
  merge_partials8(partials + static_cast<int64_t>(h) * n_splits * (head_dim + kAttnRecordHeader), n_splits, head_dim,
                  d0, f);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[i + e] = from_float<T>(f[e]);
}

// ---- argmax of one row (the greedy sampler of the decode loop) ------------------------------------------
// First index of the maximum, like torch.argmax on a row without ties broken otherwise.
template <typename T>
__global__ __launch_bounds__(1024) void argmax_row_kernel(const T* __restrict__ x, const int n, int64_t* __restrict__ out,
                                                          int64_t* __restrict__ token, int64_t* __restrict__ step64,
                                                          int32_t* __restrict__ step32) {
  __shared__ float s_val[16];
  __shared__ int s_idx[16];
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  constexpr int V = Pack<T>::N;
  const bool aligned = (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
  const int n_vec = aligned ? n / V : 0;
  // 16-byte packets, eight in flight per thread (a row of logits is a few round trips, not a
  // bandwidth problem); a thread sees its indices in increasing order, so a strict '>' keeps the
  // first maximum
  constexpr int kFlight = 8;
  for (int p0 = threadIdx.x; p0 < n_vec; p0 += kFlight * blockDim.x) {
    u32x4 raw[kFlight];
#pragma unroll
    for (int u = 0; u < kFlight; ++u) {
      const int p = p0 + u * blockDim.x;
      raw[u] = p < n_vec ? load16(x + static_cast<int64_t>(p) * V) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < kFlight; ++u) {
      const int p = p0 + u * blockDim.x;
      if (p >= n_vec) break;
      float f[V];
      Pack<T>::unpack(raw[u], f);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        if (f[e] > best) { best = f[e]; best_i = p * V + e; }
      }
    }
  }
  for (int i = n_vec * V + threadIdx.x; i < n; i += blockDim.x) {
    const float v = to_float(x[i]);
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, kWave);
    const int oi = __shfl_xor(best_i, off, kWave);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  if (lane == 0) { s_val[wv] = best; s_idx[wv] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < static_cast<int>(blockDim.x) / kWave; ++w) {
      if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) { best = s_val[w]; best_i = s_idx[w]; }
    }
    const int64_t winner = best_i == 0x7fffffff ? 0 : best_i;
    out[0] = winner;
    // the bookkeeping of a greedy decode loop, when asked for: next input token, position counters
    if (token != nullptr) token[0] = winner;
    if (step64 != nullptr) step64[0] += 1;
    if (step32 != nullptr) step32[0] += 1;
  }
}

// The same over kArgmaxBlocks workgroups, each taking a contiguous slice of the row; the workgroup that
// finishes last (a ticket from one atomic counter; nobody waits) picks the winner among the slices' first
// maxima, does the loop's bookkeeping and, when asked, copies the winner's row of the embedding table to
// `hidden_out`: the next decode step then starts at its first GEMV instead of at an embedding launch.
// part_val / part_idx / counter: kArgmaxBlocks floats, as many ints and one arrival counter that is zero before
// the first call and set back to zero by every call.
constexpr int kArgmaxBlocks = 32;
template <typename T>
__global__ __launch_bounds__(256) void argmax_split_kernel(const T* __restrict__ x, const int n, int64_t* __restrict__ out,
                                                           int64_t* __restrict__ token, int64_t* __restrict__ step64,
                                                           int32_t* __restrict__ step32, const T* __restrict__ embed,
                                                           T* __restrict__ hidden_out, const int hidden,
                                                           float* part_val, int* part_idx, unsigned* counter) {
  __shared__ float s_val[4];
  __shared__ int s_idx[4];
  __shared__ int s_winner;   // -1: this workgroup is not the last one
  constexpr int V = Pack<T>::N;
  // slices of whole 16-byte packets (the row's base is 16-byte aligned: checked by the caller)
  const int per = ((n + kArgmaxBlocks - 1) / kArgmaxBlocks + V - 1) / V * V;
  const int begin = min(static_cast<int>(blockIdx.x) * per, n), end = min(begin + per, n);
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  const int n_vec = (end - begin) / V;
  constexpr int kFlight = 2;
  for (int p0 = threadIdx.x; p0 < n_vec; p0 += kFlight * blockDim.x) {
    u32x4 raw[kFlight];
#pragma unroll
    for (int u = 0; u < kFlight; ++u) {
      const int p = p0 + u * blockDim.x;
      raw[u] = p < n_vec ? load16(x + begin + static_cast<int64_t>(p) * V) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < kFlight; ++u) {
      const int p = p0 + u * blockDim.x;
      if (p >= n_vec) break;
      float f[V];
      Pack<T>::unpack(raw[u], f);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        if (f[e] > best) { best = f[e]; best_i = begin + p * V + e; }
      }
    }
  }
  for (int i = begin + n_vec * V + threadIdx.x; i < end; i += blockDim.x) {
    const float v = to_float(x[i]);
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
  }
  auto take = [&](float ov, int oi) {
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  };
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) take(__shfl_xor(best, off, kWave), __shfl_xor(best_i, off, kWave));
  const int lane = threadIdx.x & (kWave - 1), wv = threadIdx.x / kWave;
  if (lane == 0) { s_val[wv] = best; s_idx[wv] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < static_cast<int>(blockDim.x) / kWave; ++w) take(s_val[w], s_idx[w]);
    __hip_atomic_store(part_val + blockIdx.x, best, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(part_idx + blockIdx.x, best_i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();   // the slice's result is visible to the other XCDs before the ticket is
    const unsigned ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    s_winner = ticket == gridDim.x - 1 ? 0 : -1;
  }
  __syncthreads();
  if (s_winner < 0) return;
  // the last workgroup: every slice's result is in memory
  if (wv == 0) {
    best = -INFINITY, best_i = 0x7fffffff;
    if (lane < static_cast<int>(gridDim.x)) {
      best = __hip_atomic_load(part_val + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      best_i = __hip_atomic_load(part_idx + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) take(__shfl_xor(best, off, kWave), __shfl_xor(best_i, off, kWave));
    if (lane == 0) {
      const int64_t winner = best_i == 0x7fffffff ? 0 : best_i;
      out[0] = winner;
      if (token != nullptr) token[0] = winner;
      if (step64 != nullptr) step64[0] += 1;
      if (step32 != nullptr) step32[0] += 1;
      __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next call
      s_winner = static_cast<int>(winner);
    }
  }
  __syncthreads();
  if (embed != nullptr) {
    const T* row = embed + static_cast<int64_t>(s_winner) * hidden;
    for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) store16(hidden_out + i, load16(row + i));
  }
}

int splits_for(int t_max) {
  int s = (t_max + 63) / 64;
  if (s > 64) s = 64;
  return s < 1 ? 1 : s;
}

template <typename T, int BITS, int D>
int launch_attn_rep(int rep, dim3 grid, hipStream_t stream, const T* q, const uint8_t* kc,
                    const uint8_t* vc, const float* ks, const float* vs, T* out, float* part, int* count,
                    const int32_t* len_dev, float scale_log2, int t_max, int chunk) {
#define LLMQ_ATTN(R)                                                                            \
  case R:                                                                                       \
    hipLaunchKernelGGL((kv_decode_attn_kernel<T, BITS, D, R>), grid, dim3(kAttnThreads), 0, stream, q, kc, \
                       vc, ks, vs, out, part, count, len_dev, scale_log2, t_max, chunk);        \
    break;
  switch (rep) {
    LLMQ_ATTN(1) LLMQ_ATTN(2) LLMQ_ATTN(4) LLMQ_ATTN(8)
    default:
      return llmq_host::fail_invalid("q_heads / kv_heads must be 1, 2, 4 or 8, got %d", rep);
  }
#undef LLMQ_ATTN
  return llmq_host::check_launch("kv_decode_attn_kernel");
}

}  // namespace

extern "C" size_t llmq_kv_decode_workspace_floats(int q_heads, int head_dim, int t_max) {
  // partial records, then one int32 counter per head (sized by q_heads >= kv_heads)
  return static_cast<size_t>(q_heads) * splits_for(t_max) * (head_dim + 2) + q_heads;
}

extern "C" int llmq_kv_append(const void* k_new, const void* v_new, int64_t head_stride,
                              int64_t token_stride, void* k_codes, void* v_codes, float* k_scale,
                              float* v_scale, void* dq_k_or_null, void* dq_v_or_null,
                              const int32_t* pos_dev, int n_new, int kv_heads, int head_dim, int t_max,
                              int bits, int dtype, llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (head_dim < 2 || head_dim > 128 || (head_dim & 1))
    return llmq_host::fail_invalid("head_dim must be even and in [2, 128], got %d", head_dim);
  if (n_new < 0 || kv_heads < 0 || t_max < 0) return llmq_host::fail_invalid("negative size");
  if (n_new == 0 || kv_heads == 0) return 0;
  if (!k_new || !v_new || !k_codes || !v_codes || !k_scale || !v_scale || !pos_dev)
    return llmq_host::fail_invalid("null tensor pointer");
  const int64_t waves = 2LL * kv_heads * n_new;
  const dim3 grid(static_cast<unsigned>((waves + 3) / 4)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LLMQ_APPEND(T, B)                                                                       \
  hipLaunchKernelGGL((kv_append_kernel<T, B>), grid, block, 0, s, static_cast<const T*>(k_new), \
                     static_cast<const T*>(v_new), head_stride, token_stride,                   \
                     static_cast<uint8_t*>(k_codes), static_cast<uint8_t*>(v_codes), k_scale, v_scale, \
                     static_cast<T*>(dq_k_or_null), static_cast<T*>(dq_v_or_null), pos_dev, n_new, \
                     kv_heads, head_dim, t_max)
  switch (dtype) {
    case LLMQ_F32: if (bits == 8) LLMQ_APPEND(float, 8); else LLMQ_APPEND(float, 4); break;
    case LLMQ_F16: if (bits == 8) LLMQ_APPEND(f16_t, 8); else LLMQ_APPEND(f16_t, 4); break;
    case LLMQ_BF16: if (bits == 8) LLMQ_APPEND(bf16_t, 8); else LLMQ_APPEND(bf16_t, 4); break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_APPEND
  return llmq_host::check_launch("kv_append_kernel");
}

extern "C" int llmq_rope_kv_append(const void* q, const void* k, const void* v, int64_t q_row_stride,
                                   int64_t k_row_stride, int64_t v_row_stride, const void* cos_rows,
                                   const void* sin_rows, void* q_out, void* k_codes, void* v_codes, float* k_scale,
                                   float* v_scale, void* dq_k_or_null, void* dq_v_or_null, const int32_t* pos_dev,
                                   int tokens, int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                                   int dtype, llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (tokens < 0 || q_heads < 0 || kv_heads < 0 || t_max < 0) return llmq_host::fail_invalid("negative size");
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  if (tokens == 0 || q_heads + kv_heads == 0) return 0;
  if (!cos_rows || !sin_rows || !pos_dev || (q_heads && (!q || !q_out)) ||
      (kv_heads && (!k || !v || !k_codes || !v_codes || !k_scale || !v_scale)))
    return llmq_host::fail_invalid("null tensor pointer");
  if ((dq_k_or_null == nullptr) != (dq_v_or_null == nullptr))
    return llmq_host::fail_invalid("dq_k and dq_v go together");
  const int64_t waves = static_cast<int64_t>(tokens) * (q_heads + 2 * kv_heads);
  const dim3 grid(static_cast<unsigned>((waves + 3) / 4)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LLMQ_ROPE_APPEND(T, B, D)                                                                          \
  hipLaunchKernelGGL((rope_kv_append_kernel<T, B, D>), grid, block, 0, s, static_cast<const T*>(q),         \
                     static_cast<const T*>(k), static_cast<const T*>(v), q_row_stride, k_row_stride,        \
                     v_row_stride, static_cast<const T*>(cos_rows), static_cast<const T*>(sin_rows),        \
                     static_cast<T*>(q_out), static_cast<uint8_t*>(k_codes), static_cast<uint8_t*>(v_codes), \
                     k_scale, v_scale, static_cast<T*>(dq_k_or_null), static_cast<T*>(dq_v_or_null), pos_dev, \
                     tokens, q_heads, kv_heads, t_max)
#define LLMQ_ROPE_APPEND_T(T)                                             \
  do {                                                                    \
    if (bits == 8 && head_dim == 64) LLMQ_ROPE_APPEND(T, 8, 64);          \
    else if (bits == 8) LLMQ_ROPE_APPEND(T, 8, 128);                      \
    else if (head_dim == 64) LLMQ_ROPE_APPEND(T, 4, 64);                  \
    else LLMQ_ROPE_APPEND(T, 4, 128);                                     \
  } while (0)
  switch (dtype) {
    case LLMQ_F32: LLMQ_ROPE_APPEND_T(float); break;
    case LLMQ_F16: LLMQ_ROPE_APPEND_T(f16_t); break;
    default: LLMQ_ROPE_APPEND_T(bf16_t); break;
  }
#undef LLMQ_ROPE_APPEND_T
#undef LLMQ_ROPE_APPEND
  return llmq_host::check_launch("rope_kv_append_kernel");
}

extern "C" int llmq_kv_dequant(const void* codes, const float* scale, void* out, int kv_heads,
                               int head_dim, int t_max, int n_tokens, int bits, int dtype,
                               llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (n_tokens < 0 || n_tokens > t_max) return llmq_host::fail_invalid("n_tokens %d outside [0, %d]", n_tokens, t_max);
  const int64_t total = static_cast<int64_t>(kv_heads) * n_tokens * head_dim;
  if (total == 0) return 0;
  if (!codes || !scale || !out) return llmq_host::fail_invalid("null tensor pointer");
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LLMQ_DQ(T, B)                                                                           \
  hipLaunchKernelGGL((kv_dequant_kernel<T, B>), grid, block, 0, s, static_cast<const uint8_t*>(codes), \
                     scale, static_cast<T*>(out), kv_heads, head_dim, t_max, n_tokens)
  switch (dtype) {
    case LLMQ_F32: if (bits == 8) LLMQ_DQ(float, 8); else LLMQ_DQ(float, 4); break;
    case LLMQ_F16: if (bits == 8) LLMQ_DQ(f16_t, 8); else LLMQ_DQ(f16_t, 4); break;
    case LLMQ_BF16: if (bits == 8) LLMQ_DQ(bf16_t, 8); else LLMQ_DQ(bf16_t, 4); break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_DQ
  return llmq_host::check_launch("kv_dequant_kernel");
}

extern "C" int llmq_kv_decode_attention(const void* q, const void* k_codes, const void* v_codes,
                                        const float* k_scale, const float* v_scale, void* out,
                                        float* workspace, const int32_t* len_dev, float sm_scale,
                                        int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                                        int dtype, llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads) return llmq_host::fail_invalid("q_heads %d must be a positive multiple of kv_heads %d", q_heads, kv_heads);
  if (t_max <= 0) return llmq_host::fail_invalid("t_max must be positive, got %d", t_max);
  if (!q || !k_codes || !v_codes || !k_scale || !v_scale || !out || !workspace || !len_dev)
    return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes)) & 15u)
    return llmq_host::fail_invalid("cache code pointers must be 16-byte aligned");
  const int rep = q_heads / kv_heads;
  const int splits = splits_for(t_max);
  const int chunk = (t_max + splits - 1) / splits;
  float* part = workspace;
  int* count = reinterpret_cast<int*>(workspace + static_cast<size_t>(q_heads) * splits * (head_dim + 2));
  const dim3 grid(splits, kv_heads);
  const float scale_log2 = sm_scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint8_t* kc = static_cast<const uint8_t*>(k_codes);
  const uint8_t* vc = static_cast<const uint8_t*>(v_codes);
#define LLMQ_GO(T, B, D)                                                                        \
  return launch_attn_rep<T, B, D>(rep, grid, s, static_cast<const T*>(q), kc, vc, k_scale, v_scale, \
                                  static_cast<T*>(out), part, count, len_dev, scale_log2, t_max, chunk)
#define LLMQ_BD(T)                                                                              \
  if (bits == 8) { if (head_dim == 64) LLMQ_GO(T, 8, 64); else LLMQ_GO(T, 8, 128); }            \
  else { if (head_dim == 64) LLMQ_GO(T, 4, 64); else LLMQ_GO(T, 4, 128); }
  switch (dtype) {
    case LLMQ_F32: LLMQ_BD(float)
    case LLMQ_F16: LLMQ_BD(f16_t)
    case LLMQ_BF16: LLMQ_BD(bf16_t)
  }
#undef LLMQ_BD
#undef LLMQ_GO
  return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
}

// ---- the same attention for callers that cannot allocate ----------------------------------------------
// The partial records and arrival counters live in a file-scope device array instead of a caller's
// workspace. Every GPU the library runs on holds its own copy of the array (at its own address, found once
// per device with hipGetSymbolAddress) until the process ends. Layout: kStaticCounters int32 arrival
// counters first, at a fixed place whatever the geometry of a call, then the partial records.
constexpr int kStaticMaxQHeads = 128;
constexpr int kStaticCounters = 256;  // >= kStaticMaxQHeads, and a whole number of 256-byte lines
constexpr size_t kStaticPartFloats = static_cast<size_t>(kStaticMaxQHeads) * 64 * (128 + 2);
static __device__ __align__(256) float g_attn_scratch[kStaticCounters + kStaticPartFloats];

namespace {
__global__ void clear_counters_kernel(int* __restrict__ count) { count[threadIdx.x] = 0; }

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

// The array's address on the current device; looked up on the first call per device. Returns nullptr
// with the error text set when the runtime refuses.
float* static_scratch() {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess || device < 0 || device >= kMaxDevices) {
    llmq_host::set_error("static scratch: hipGetDevice gave device %d (%s)", device, hipGetErrorString(err));
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_attn_scratch));
    if (err != hipSuccess || ptr == nullptr) {
      llmq_host::set_error("static scratch: hipGetSymbolAddress failed on device %d (%s)", device,
                           hipGetErrorString(err));
      return nullptr;
    }
    g_scratch_ptr[device] = static_cast<float*>(ptr);
  }
  return g_scratch_ptr[device];
}
}  // namespace

extern "C" int llmq_kv_decode_attention_static(const void* q, const void* k_codes, const void* v_codes,
                                               const float* k_scale, const float* v_scale, void* out,
                                               const int32_t* len_dev, float sm_scale, int q_heads,
                                               int kv_heads, int head_dim, int t_max, int bits, int dtype,
                                               llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads) return llmq_host::fail_invalid("q_heads %d must be a positive multiple of kv_heads %d", q_heads, kv_heads);
  if (q_heads > kStaticMaxQHeads)
    return llmq_host::fail_invalid("the static scratch holds up to %d query heads, got %d (use llmq_kv_decode_attention "
                                   "with a workspace of your own)", kStaticMaxQHeads, q_heads);
  if (t_max <= 0) return llmq_host::fail_invalid("t_max must be positive, got %d", t_max);
  if (!q || !k_codes || !v_codes || !k_scale || !v_scale || !out || !len_dev)
    return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes)) & 15u)
    return llmq_host::fail_invalid("cache code pointers must be 16-byte aligned");
  if (dtype != LLMQ_F32 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  const int rep = q_heads / kv_heads;
  if (rep != 1 && rep != 2 && rep != 4 && rep != 8)
    return llmq_host::fail_invalid("q_heads / kv_heads must be 1, 2, 4 or 8, got %d", rep);
  const int splits = splits_for(t_max);
  if (static_cast<size_t>(q_heads) * splits * (head_dim + 2) > kStaticPartFloats)
    return llmq_host::fail_invalid("partial records exceed the static scratch");
  float* scratch = static_scratch();
  if (scratch == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
  int* count = reinterpret_cast<int*>(scratch);
  float* part = scratch + kStaticCounters;
  const int chunk = (t_max + splits - 1) / splits;
  const dim3 grid(splits, kv_heads);
  const float scale_log2 = sm_scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // the counters must start at zero whatever the last call on this GPU left behind (a fill kernel, not
  // a memset: a caller may be capturing a graph)
  hipLaunchKernelGGL(clear_counters_kernel, dim3(1), dim3(kStaticCounters), 0, s, count);
  if (int rc = llmq_host::check_launch("clear_counters_kernel")) return rc;
  const uint8_t* kc = static_cast<const uint8_t*>(k_codes);
  const uint8_t* vc = static_cast<const uint8_t*>(v_codes);
#define LLMQ_GO(T, B, D)                                                                        \
  return launch_attn_rep<T, B, D>(rep, grid, s, static_cast<const T*>(q), kc, vc, k_scale, v_scale, \
                                  static_cast<T*>(out), part, count, len_dev, scale_log2, t_max, chunk)
#define LLMQ_BD(T)                                                                              \
  if (bits == 8) { if (head_dim == 64) LLMQ_GO(T, 8, 64); else LLMQ_GO(T, 8, 128); }            \
  else { if (head_dim == 64) LLMQ_GO(T, 4, 64); else LLMQ_GO(T, 4, 128); }
  switch (dtype) {
    case LLMQ_F32: LLMQ_BD(float)
    case LLMQ_F16: LLMQ_BD(f16_t)
    default: LLMQ_BD(bf16_t)
  }
#undef LLMQ_BD
#undef LLMQ_GO
}

extern "C" int llmq_kv_rope_append_attend(const void* qkv, const void* cos_table, const void* sin_table,
                                          void* k_codes, void* v_codes, float* k_scale, float* v_scale,
                                          void* out, const int32_t* pos_dev, float sm_scale, int q_heads,
                                          int kv_heads, int head_dim, int t_max, int bits, int dtype,
                                          llmq_stream_t stream) {
  if (bits != 8 && bits != 4) return llmq_host::fail_invalid("KV cache bits must be 8 or 4, got %d", bits);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads)
    return llmq_host::fail_invalid("q_heads %d must be a positive multiple of kv_heads %d", q_heads, kv_heads);
  if (t_max <= 0) return llmq_host::fail_invalid("t_max must be positive, got %d", t_max);
  if (!qkv || !cos_table || !sin_table || !k_codes || !v_codes || !k_scale || !v_scale || !out || !pos_dev)
    return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes)) & 15u)
    return llmq_host::fail_invalid("cache code pointers must be 16-byte aligned");
  const float scale_log2 = sm_scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(q_heads), block(kFusedThreads);
#define LLMQ_FUSED(T, B, D)                                                                      \
  hipLaunchKernelGGL((kv_rope_append_attend_kernel<T, B, D>), grid, block, 0, s, static_cast<const T*>(qkv), \
                     static_cast<const T*>(cos_table), static_cast<const T*>(sin_table),          \
                     static_cast<uint8_t*>(k_codes), static_cast<uint8_t*>(v_codes), k_scale, v_scale, \
                     static_cast<T*>(out), pos_dev, scale_log2, q_heads, kv_heads, t_max)
#define LLMQ_FUSED_BD(T)                                                                         \
  if (bits == 8) { if (head_dim == 64) { LLMQ_FUSED(T, 8, 64); } else { LLMQ_FUSED(T, 8, 128); } } \
  else { if (head_dim == 64) { LLMQ_FUSED(T, 4, 64); } else { LLMQ_FUSED(T, 4, 128); } }
  switch (dtype) {
    case LLMQ_F32: LLMQ_FUSED_BD(float) break;
    case LLMQ_F16: LLMQ_FUSED_BD(f16_t) break;
    case LLMQ_BF16: LLMQ_FUSED_BD(bf16_t) break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_FUSED_BD
#undef LLMQ_FUSED
  return llmq_host::check_launch("kv_rope_append_attend_kernel");
}

extern "C" int llmq_argmax_advance(const void* x, int n, int64_t* out_index, int64_t* token_or_null,
                                   int64_t* step64_or_null, int32_t* step32_or_null, int dtype,
                                   llmq_stream_t stream) {
  if (n <= 0) return llmq_host::fail_invalid("argmax of an empty row");
  if (!x || !out_index) return llmq_host::fail_invalid("null tensor pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LLMQ_ARGMAX(T)                                                                                     \
  hipLaunchKernelGGL((argmax_row_kernel<T>), dim3(1), dim3(1024), 0, s, static_cast<const T*>(x), n, out_index, \
                     token_or_null, step64_or_null, step32_or_null)
  switch (dtype) {
    case LLMQ_F32: LLMQ_ARGMAX(float); break;
    case LLMQ_F16: LLMQ_ARGMAX(f16_t); break;
    case LLMQ_BF16: LLMQ_ARGMAX(bf16_t); break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_ARGMAX
  return llmq_host::check_launch("argmax_row_kernel");
}

extern "C" size_t llmq_argmax_workspace_bytes(void) { return kArgmaxBlocks * 8 + 256; }

extern "C" int llmq_argmax_advance_embed(const void* x, int n, int64_t* out_index, int64_t* token_or_null,
                                         int64_t* step64_or_null, int32_t* step32_or_null,
                                         const void* embed_or_null, void* hidden_out_or_null, int hidden_dim,
                                         void* workspace, int dtype, llmq_stream_t stream) {
  if (n <= 0) return llmq_host::fail_invalid("argmax of an empty row");
  if (!x || !out_index || !workspace) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(workspace)) & 15u)
    return llmq_host::fail_invalid("the row and the workspace must be 16-byte aligned");
  const int packet = dtype == LLMQ_F32 ? 4 : 8;
  if (embed_or_null != nullptr) {
    if (!hidden_out_or_null || hidden_dim <= 0 || hidden_dim % packet != 0)
      return llmq_host::fail_invalid("the embedding hand-off needs an output row and a width that is a multiple of %d, got %d",
                                     packet, hidden_dim);
    if ((reinterpret_cast<uintptr_t>(embed_or_null) | reinterpret_cast<uintptr_t>(hidden_out_or_null)) & 15u)
      return llmq_host::fail_invalid("embedding table and output row must be 16-byte aligned");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* part_val = static_cast<float*>(workspace);
  int* part_idx = reinterpret_cast<int*>(part_val + kArgmaxBlocks);
  unsigned* counter = reinterpret_cast<unsigned*>(part_idx + kArgmaxBlocks);
#define LLMQ_ARGMAX(T)                                                                                              \
  hipLaunchKernelGGL((argmax_split_kernel<T>), dim3(kArgmaxBlocks), dim3(256), 0, s, static_cast<const T*>(x), n,   \
                     out_index, token_or_null, step64_or_null, step32_or_null, static_cast<const T*>(embed_or_null), \
                     static_cast<T*>(hidden_out_or_null), hidden_dim, part_val, part_idx, counter)
  switch (dtype) {
    case LLMQ_F32: LLMQ_ARGMAX(float); break;
    case LLMQ_F16: LLMQ_ARGMAX(f16_t); break;
    case LLMQ_BF16: LLMQ_ARGMAX(bf16_t); break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_ARGMAX
  return llmq_host::check_launch("argmax_split_kernel");
}

extern "C" int llmq_argmax_row(const void* x, int n, int64_t* out_index, int dtype, llmq_stream_t stream) {
  return llmq_argmax_advance(x, n, out_index, nullptr, nullptr, nullptr, dtype, stream);
}

extern "C" size_t llmq_kv_attend_partials_floats(int q_heads, int head_dim, int n_splits) {
  return static_cast<size_t>(q_heads) * n_splits * (head_dim + kAttnRecordHeader);
}

extern "C" int llmq_kv_rope_append_attend_split(const void* qkv, const void* cos_table, const void* sin_table,
                                                void* k_codes, void* v_codes, float* k_scale, float* v_scale,
                                                float* partials, const int32_t* pos_dev, float sm_scale,
                                                int q_heads, int kv_heads, int head_dim, int t_max, int bits,
                                                int n_splits, int dtype, llmq_stream_t stream) {
  if (bits != 8 && bits != 4 && bits != 16)
    return llmq_host::fail_invalid("KV cache bits must be 8 or 4 (or 16: an unquantized cache of the model's dtype), got %d", bits);
  if (bits == 16 && dtype != LLMQ_F16 && dtype != LLMQ_BF16)
    return llmq_host::fail_invalid("an unquantized cache (bits 16) holds float16 or bfloat16 values, got dtype code %d", dtype);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads)
    return llmq_host::fail_invalid("q_heads %d must be a positive multiple of kv_heads %d", q_heads, kv_heads);
  if (t_max <= 0) return llmq_host::fail_invalid("t_max must be positive, got %d", t_max);
  if (n_splits < 1 || n_splits > 256) return llmq_host::fail_invalid("n_splits must be in [1, 256], got %d", n_splits);
  if (!qkv || !cos_table || !sin_table || !k_codes || !v_codes || !k_scale || !v_scale || !partials || !pos_dev)
    return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(k_codes) | reinterpret_cast<uintptr_t>(v_codes) |
       reinterpret_cast<uintptr_t>(partials)) & 15u)
    return llmq_host::fail_invalid("cache code and record pointers must be 16-byte aligned");
  const float scale_log2 = sm_scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Four query heads of a kv head per workgroup once the caller asks for 32 splits or more (or for 8 on a cache of
  // 2048 rows or more, which then takes the matrix-core form below): measured on the vector ALU at 32 splits, ctx
  // 8 K / 16 K / 32 K: 9.7 / 13.6 / 20.9 us per layer against 13.0 / 19.7 / 32.0 us for one head per workgroup at
  // its best split count; below that the one-head form, which puts more workgroups on the chip, is as fast or faster.
  const int rep_heads = q_heads / kv_heads;
  // (heads of 128: the vector-ALU form has twice the arithmetic per cache row, and the matrix-core form is ahead at every
  // cache length: the Llama-3-8B architecture's step at 600 cached tokens, 1968 us a token against 2038)
  const int mf_min_cache = head_dim == 128 ? 0 : kMfMinCache;
  // (the unquantized cache keeps the one-head form: it is the baseline's step, not a path to tune)
  const bool grouped = bits != 16 && rep_heads % 4 == 0 && (n_splits >= 32 || (n_splits >= 8 && t_max >= mf_min_cache));
  const dim3 grid(grouped ? q_heads / 4 : q_heads, n_splits), block(kSplitThreads);
  if (grouped && t_max >= mf_min_cache) {
    // long caches: the matrix-core form (see the kernel's comment for what it changes in the arithmetic)
#define LLMQ_SPLIT_MFMA(T, B, D)                                                                                  \
  do {                                                                                                            \
    auto kernel = kv_rope_append_attend_split_mfma_kernel<T, B, D>;                                               \
    constexpr int kMfLdsBytes = MfLds<B, D>::kBytes;                                                              \
    static bool raised = false; /* per instantiation; worst case two threads both set it */                       \
    if (!raised) {                                                                                                \
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                           \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kMfLdsBytes);        \
      if (err != hipSuccess) {                                                                                    \
        llmq_host::set_error("raising the LDS limit failed: %s", hipGetErrorString(err));                         \
        return static_cast<int>(err);                                                                             \
      }                                                                                                           \
      raised = true;                                                                                              \
    }                                                                                                             \
    hipLaunchKernelGGL(kernel, grid, block, kMfLdsBytes, s, static_cast<const T*>(qkv),                           \
                       static_cast<const T*>(cos_table), static_cast<const T*>(sin_table),                        \
                       static_cast<uint8_t*>(k_codes), static_cast<uint8_t*>(v_codes), k_scale, v_scale, partials, \
                       pos_dev, scale_log2, q_heads, kv_heads, t_max);                                            \
  } while (0)
#define LLMQ_SPLIT_MFMA_D(T)                                                        \
  if (bits == 8) { if (head_dim == 64) LLMQ_SPLIT_MFMA(T, 8, 64); else LLMQ_SPLIT_MFMA(T, 8, 128); } \
  else { if (head_dim == 64) LLMQ_SPLIT_MFMA(T, 4, 64); else LLMQ_SPLIT_MFMA(T, 4, 128); }           \
  break;
    switch (dtype) {
      case LLMQ_F32: LLMQ_SPLIT_MFMA_D(float)
      case LLMQ_F16: LLMQ_SPLIT_MFMA_D(f16_t)
      case LLMQ_BF16: LLMQ_SPLIT_MFMA_D(bf16_t)
      default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
    }
#undef LLMQ_SPLIT_MFMA_D
#undef LLMQ_SPLIT_MFMA
    return llmq_host::check_launch("kv_rope_append_attend_split_mfma_kernel");
  }
#define LLMQ_SPLIT(T, B, D)                                                                            \
  do {                                                                                                 \
    if (grouped) {                                                                                     \
      hipLaunchKernelGGL((kv_rope_append_attend_split_kernel<T, B, D, 4>), grid, block, 0, s,          \
                         static_cast<const T*>(qkv), static_cast<const T*>(cos_table),                 \
                         static_cast<const T*>(sin_table), static_cast<uint8_t*>(k_codes),             \
                         static_cast<uint8_t*>(v_codes), k_scale, v_scale, partials, pos_dev,          \
                         scale_log2, q_heads, kv_heads, t_max);                                        \
    } else {                                                                                           \
      hipLaunchKernelGGL((kv_rope_append_attend_split_kernel<T, B, D, 1>), grid, block, 0, s,          \
                         static_cast<const T*>(qkv), static_cast<const T*>(cos_table),                 \
                         static_cast<const T*>(sin_table), static_cast<uint8_t*>(k_codes),             \
                         static_cast<uint8_t*>(v_codes), k_scale, v_scale, partials, pos_dev,          \
                         scale_log2, q_heads, kv_heads, t_max);                                        \
    }                                                                                                  \
  } while (0)
#define LLMQ_SPLIT_BD(T)                                                                               \
  if (bits == 8) { if (head_dim == 64) LLMQ_SPLIT(T, 8, 64); else LLMQ_SPLIT(T, 8, 128); }             \
  else { if (head_dim == 64) LLMQ_SPLIT(T, 4, 64); else LLMQ_SPLIT(T, 4, 128); }                       \
  break;
#define LLMQ_SPLIT_16(T)                                                                               \
  do {                                                                                                 \
    if (head_dim == 64) {                                                                              \
      hipLaunchKernelGGL((kv_rope_append_attend_split_kernel<T, 16, 64, 1>), grid, block, 0, s,        \
                         static_cast<const T*>(qkv), static_cast<const T*>(cos_table),                 \
                         static_cast<const T*>(sin_table), static_cast<uint8_t*>(k_codes),             \
                         static_cast<uint8_t*>(v_codes), k_scale, v_scale, partials, pos_dev,          \
                         scale_log2, q_heads, kv_heads, t_max);                                        \
    } else {                                                                                           \
      hipLaunchKernelGGL((kv_rope_append_attend_split_kernel<T, 16, 128, 1>), grid, block, 0, s,       \
                         static_cast<const T*>(qkv), static_cast<const T*>(cos_table),                 \
                         static_cast<const T*>(sin_table), static_cast<uint8_t*>(k_codes),             \
                         static_cast<uint8_t*>(v_codes), k_scale, v_scale, partials, pos_dev,          \
                         scale_log2, q_heads, kv_heads, t_max);                                        \
    }                                                                                                  \
  } while (0)
  if (bits == 16) {
    if (dtype == LLMQ_F16) LLMQ_SPLIT_16(f16_t); else LLMQ_SPLIT_16(bf16_t);
    return llmq_host::check_launch("kv_rope_append_attend_split_kernel");
  }
#undef LLMQ_SPLIT_16
  switch (dtype) {
    case LLMQ_F32: LLMQ_SPLIT_BD(float)
    case LLMQ_F16: LLMQ_SPLIT_BD(f16_t)
    case LLMQ_BF16: LLMQ_SPLIT_BD(bf16_t)
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
#undef LLMQ_SPLIT_BD
#undef LLMQ_SPLIT
  return llmq_host::check_launch("kv_rope_append_attend_split_kernel");
}

extern "C" int llmq_kv_attend_merge(const float* partials, void* out, int q_heads, int head_dim, int n_splits,
                                    int dtype, llmq_stream_t stream) {
  if (q_heads < 0 || head_dim <= 0 || head_dim % 8 || n_splits < 1)
    return llmq_host::fail_invalid("bad sizes q_heads=%d head_dim=%d (a multiple of 8) n_splits=%d", q_heads, head_dim,
                                   n_splits);
  const int total = q_heads * head_dim;
  if (total == 0) return 0;
  if (!partials || !out) return llmq_host::fail_invalid("null tensor pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((total / 8 + 255) / 256), block(256);
  switch (dtype) {
    case LLMQ_F32:
      hipLaunchKernelGGL((kv_attend_merge_kernel<float>), grid, block, 0, s, partials, static_cast<float*>(out), total, head_dim, n_splits);
      break;
    case LLMQ_F16:
      hipLaunchKernelGGL((kv_attend_merge_kernel<f16_t>), grid, block, 0, s, partials, static_cast<f16_t*>(out), total, head_dim, n_splits);
      break;
    case LLMQ_BF16:
      hipLaunchKernelGGL((kv_attend_merge_kernel<bf16_t>), grid, block, 0, s, partials, static_cast<bf16_t*>(out), total, head_dim, n_splits);
      break;
    default: return llmq_host::fail_invalid("unsupported dtype code %d", dtype);
  }
  return llmq_host::check_launch("kv_attend_merge_kernel");
}
