// Causal grouped-query attention of a prompt on the matrix core, gfx950:
//
//   out[i, h, :] = softmax_j<=i( scale * q[i, h, :] . k[hk, j, :] ) @ v[hk, :, :],   hk = h / (q_heads / kv_heads)
//
// what the reference's prompt pass gets from transformers' attention (scaled_dot_product_attention with
// is_causal and enable_gqa) on the rotated queries and on the K / V its FakeQuantCache hands back
// (llmquant/quantizers/fake.py:39-55): k and v here are those dequantized values, [kv_heads, tokens, head_dim].
// Scores and the weighted sum are accumulated in fp32, the probabilities rounded to the 16-bit type before they
// meet V (as the flash kernels do), one division at the end.
//
// Shape. A workgroup of four waves owns 32 queries of one head, and the key blocks (32 keys) up to the diagonal
// are dealt to its waves in turn: a wave walks blocks w, w + 4, ... on its own, with no barrier inside the walk,
// and the four partial results (maximum, sum, weighted sum) are merged through LDS at the end, in wave order,
// so that the sum is the same on every run and a query's result does not depend on how long the prompt is.
// That puts 8 waves on every CU for the 512-token prompt of a 32-head model, where one wave per 32 queries
// would leave half the SIMDs without work and the last block of queries walking 16 key blocks alone.
//
// Both products are computed transposed so that a lane owns one query: S^T = K Q^T (A = 32 keys x 16 d,
// B = 16 d x 32 queries: both operands are 16-byte row reads, Q kept in registers for the whole walk) leaves lane
// (query, half) with 16 of the block's 32 scores, so the running maximum and sum of a query are in-lane
// reductions plus one exchange between the two halves; O^T = V^T P^T (A = head_dim x keys, B = keys x queries)
// takes the probabilities straight out of those registers as its B operand (the k index of the MFMA is just a
// naming of the keys, the same on both operands) and V^T from the wave's own LDS tile: the block's rows of V go
// there as they lie in memory (global_load_lds_dwordx4, no register in between, the 16-byte pieces of odd keys
// XOR-swizzled by four so that the reads below spread over the banks), and ds_read_b64_tr_b16 hands lane
// (d, half) four keys of its column per read. Among the 16 lanes of a group, that instruction gives lane l, as
// its element j, element l % 4 of what lane 4 j + l / 4 points at: with lane 4 j + i pointing at key j,
// columns 4 i .. 4 i + 3, lane l gets column l of keys 0..3. The next block's K and V are requested as soon as
// this block's K has been consumed, into the tile's other buffer.
#include "llmq_device.h"

namespace {

using namespace llmq;

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));

constexpr int kQueriesPerGroup = 32, kWavesPerGroup = 4, kKeysPerBlock = 32;

template <typename T> __device__ __forceinline__ v16f mfma16(u32x4 a, u32x4 b, v16f c);
template <> __device__ __forceinline__ v16f mfma16<bf16_t>(u32x4 a, u32x4 b, v16f c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
}
template <> __device__ __forceinline__ v16f mfma16<f16_t>(u32x4 a, u32x4 b, v16f c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float lo, float hi) {
  return static_cast<uint32_t>(bf16_bits_rne(lo)) | (static_cast<uint32_t>(bf16_bits_rne(hi)) << 16);
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float lo, float hi) {
  const _Float16 a = static_cast<_Float16>(lo), b = static_cast<_Float16>(hi);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, a)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, b)) << 16);
}

// Key of a 32-key block that register r of an S^T tile holds in lane half lh (the MFMA's result layout: row
// 8 (r / 4) + 4 lh + r % 4).
__device__ __forceinline__ int key_of(int lh, int r) { return 8 * (r >> 2) + 4 * lh + (r & 3); }

template <int D> struct Lds {
  static constexpr int kTile = 2 * kKeysPerBlock * D * 2;          // bytes of one wave's V tile, two buffers
  static constexpr int kRow = D + 4;                               // floats of a row of a partial result
  static constexpr int kPartial = kQueriesPerGroup * kRow * 4;     // bytes of one wave's partial result
  static constexpr int kBody = kWavesPerGroup * (kPartial > kTile ? kPartial : kTile);
  static constexpr int kBytes = kBody + 2 * kWavesPerGroup * kQueriesPerGroup * 4;   // + maxima and sums
};

template <typename T, int D>
__global__ __launch_bounds__(kWavesPerGroup * kWave, 2) void prefill_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ out, const int tokens,
    const int q_heads, const int kv_heads, const float scale_log2e) {
  constexpr int kDSteps = D / 16;    // k-steps of S^T = K Q^T
  constexpr int kDTiles = D / 32;    // row tiles of O^T
  __shared__ __attribute__((aligned(16))) unsigned char s_mem[Lds<D>::kBytes];

  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wv = __builtin_amdgcn_readfirstlane(tid / kWave);   // (in a scalar register: the walk's block index, and every branch on it, is the wave's)
  const int lm = lane & 31, lh = lane >> 5;
  // the long walks (late query blocks) first
  const int qb = static_cast<int>(gridDim.x) - 1 - static_cast<int>(blockIdx.x);
  const int h = blockIdx.y, hk = h / (q_heads / kv_heads);
  const int q0 = qb * kQueriesPerGroup;   // (< tokens: see the grid)
  const int my_query = q0 + lm;
  const T* kh = k + static_cast<int64_t>(hk) * tokens * D;
  const T* vh = v + static_cast<int64_t>(hk) * tokens * D;

  // Q^T operand: lane (query, half) holds d 16 t + 8 lh .. + 7 of its query
  u32x4 qreg[kDSteps];
  {
    const T* row = q + (static_cast<int64_t>(min(my_query, tokens - 1)) * q_heads + h) * D + 8 * lh;
#pragma unroll
    for (int t = 0; t < kDSteps; ++t) qreg[t] = load16(row + 16 * t);
  }
  const int n_blocks = min(q0 + kQueriesPerGroup - 1, tokens - 1) / kKeysPerBlock + 1;   // up to the diagonal

  // K of a block straight into the A operand's registers; V into the LDS tile: transfer i of a wave covers
  // bytes 1024 i + 16 lane of the tile, which is piece (slot ^ 4 (key & 1)) of key (1024 i + 16 lane) / (2 D)
  constexpr int kTileBytes = kKeysPerBlock * D * 2, kVInstr = kTileBytes / 1024, kRowBytes = 2 * D;
  unsigned char* tile = s_mem + wv * Lds<D>::kTile;
  uint32_t v_off[kVInstr];   // byte offsets into a block of V (before the clamp of the key to the prompt's end)
  int v_key[kVInstr];
#pragma unroll
  for (int i = 0; i < kVInstr; ++i) {
    const int at = 1024 * i + 16 * lane, key = at / kRowBytes, slot = (at % kRowBytes) / 16;
    v_key[i] = key;
    v_off[i] = static_cast<uint32_t>((slot ^ ((key & 1) << 2)) * 16);
  }
  u32x4 kreg[kDSteps];
  auto request = [&](int b, int buf) {
    const int j0 = b * kKeysPerBlock;
    const T* row = kh + static_cast<int64_t>(min(j0 + lm, tokens - 1)) * D + 8 * lh;
#pragma unroll
    for (int t = 0; t < kDSteps; ++t) kreg[t] = load16(row + 16 * t);
#pragma unroll
    for (int i = 0; i < kVInstr; ++i) {
      const unsigned char* src = reinterpret_cast<const unsigned char*>(vh) +
                                 static_cast<int64_t>(min(j0 + v_key[i], tokens - 1)) * kRowBytes + v_off[i];
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const u32x4*>(src),
                                       reinterpret_cast<u32x4*>(tile + buf * kTileBytes + 1024 * i), 16, 0, 0);
    }
  };
  // where this lane points for the transposing reads: key 4 lh + j of a group of eight, columns
  // 32 t + 16 (g & 1) + 4 i .. + 3, with g = lane / 16, j = lane % 16 / 4, i = lane % 4
  uint32_t tr_at[kDTiles];
  {
    const int g = lane >> 4, j = (lane >> 2) & 3, i = lane & 3;
#pragma unroll
    for (int t = 0; t < kDTiles; ++t) {
      const int piece = 4 * t + 2 * (g & 1) + (i >> 1);
      tr_at[t] = static_cast<uint32_t>((4 * lh + j) * kRowBytes + (piece ^ ((j & 1) << 2)) * 16 + (i & 1) * 8);
    }
  }

  v16f o[kDTiles];
#pragma unroll
  for (int t = 0; t < kDTiles; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;   // of this lane's query, in units of log2

  if (wv < n_blocks) request(wv, 0);
  int buf = 0;
  for (int b = wv; b < n_blocks; b += kWavesPerGroup, buf ^= 1) {
    const int j0 = b * kKeysPerBlock;
    // this block's K and V have arrived (nothing else of this wave is in flight)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    v16f s;
#pragma unroll
    for (int r = 0; r < 16; ++r) s[r] = 0.0f;
#pragma unroll
    for (int t = 0; t < kDSteps; ++t) s = mfma16<T>(kreg[t], qreg[t], s);
    // (the other buffer: its last readers were the previous block's MFMAs, whose operands have long arrived)
    if (b + kWavesPerGroup < n_blocks) request(b + kWavesPerGroup, buf ^ 1);

    // keys beyond the query or the prompt out (only the blocks on the diagonal and at the prompt's end have any)
    if (j0 + kKeysPerBlock - 1 > min(q0, tokens - 1)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = j0 + key_of(lh, r);
        if (key > my_query || key >= tokens) s[r] = -INFINITY;
      }
    }
    // the block's maximum in units of log2 (scale_log2e > 0: the largest score gives it), then
    // p = 2^(s scale_log2e - m), one multiply-add per score
    float m_blk = s[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) m_blk = fmaxf(m_blk, s[r]);
    m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, kWave)) * scale_log2e;
    // finite: the block's first key is at or below every query of the group (rows past the prompt's end repeat
    // its last query and are not stored)
    const float m_new = fmaxf(m_run, m_blk);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float l_blk = 0.0f;
    uint32_t p[8];
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      const float p0 = __builtin_amdgcn_exp2f(fmaf(s[r], scale_log2e, -m_new));
      const float p1 = __builtin_amdgcn_exp2f(fmaf(s[r + 1], scale_log2e, -m_new));
      l_blk += p0 + p1;
      p[r >> 1] = pack2<T>(p0, p1);
    }
    l_blk += __shfl_xor(l_blk, 32, kWave);
    l_run = l_run * alpha + l_blk;
    m_run = m_new;
    // (a multiplication by 1 changes nothing: skipped when no query of the wave has a new maximum, which is
    // most blocks once the walk is a few blocks old)
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < kDTiles; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
    }

    // O^T += V^T P^T: k-step st covers the keys that registers 8 st .. 8 st + 7 hold (key_of): two transposing
    // reads, keys 16 st + 4 lh + 0..3 and 16 st + 8 + 4 lh + 0..3
    const unsigned char* vt = tile + buf * kTileBytes;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const u32x4 pb = {p[4 * st], p[4 * st + 1], p[4 * st + 2], p[4 * st + 3]};
#pragma unroll
      for (int t = 0; t < kDTiles; ++t) {
        const unsigned char* at = vt + tr_at[t] + 16 * st * kRowBytes;
        const uint2 a_lo = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4s*)(at)));
        const uint2 a_hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) v4s*)(at + 8 * kRowBytes)));
        o[t] = mfma16<T>(u32x4{a_lo.x, a_lo.y, a_hi.x, a_hi.y}, pb, o[t]);
      }
    }
  }

  // ---- merge the four walks: m = max m_w, l = sum l_w 2^(m_w - m), O = sum O_w 2^(m_w - m), in wave order ------
  float* s_max = reinterpret_cast<float*>(s_mem + Lds<D>::kBody);
  float* s_sum = s_max + kWavesPerGroup * kQueriesPerGroup;
  if (lh == 0) s_max[wv * kQueriesPerGroup + lm] = m_run;
  __syncthreads();   // also: every wave is done with its V tiles, which the partial results overwrite
  float m_all = s_max[lm];
#pragma unroll
  for (int w = 1; w < kWavesPerGroup; ++w) m_all = fmaxf(m_all, s_max[w * kQueriesPerGroup + lm]);
  const float mine = m_run == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_all);   // (wave 0 always has a block)
  if (lh == 0) s_sum[wv * kQueriesPerGroup + lm] = l_run * mine;
  float* part = reinterpret_cast<float*>(s_mem + wv * Lds<D>::kPartial);   // [32 queries][D + 4]
#pragma unroll
  for (int t = 0; t < kDTiles; ++t)
#pragma unroll
    for (int r = 0; r < 16; r += 4) {
      // registers r .. r + 3 are d = 32 t + 8 (r / 4) + 4 lh + 0..3
      const v4f piece = {o[t][r] * mine, o[t][r + 1] * mine, o[t][r + 2] * mine, o[t][r + 3] * mine};
      *reinterpret_cast<v4f*>(part + lm * Lds<D>::kRow + 32 * t + key_of(lh, r)) = piece;
    }
  __syncthreads();
  constexpr int kChunks = D / 8;   // 16-byte pieces of an output row
  for (int c = tid; c < kQueriesPerGroup * kChunks; c += kWavesPerGroup * kWave) {
    const int row = c / kChunks, piece = c % kChunks;
    if (q0 + row >= tokens) continue;
    float total = 0.0f;
    v4f lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = lo;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) {
      const float* src = reinterpret_cast<const float*>(s_mem + w * Lds<D>::kPartial) + row * Lds<D>::kRow + piece * 8;
      lo += *reinterpret_cast<const v4f*>(src);
      hi += *reinterpret_cast<const v4f*>(src + 4);
      total += s_sum[w * kQueriesPerGroup + row];
    }
    const float inv = 1.0f / total;
    const u32x4 packed = {pack2<T>(lo[0] * inv, lo[1] * inv), pack2<T>(lo[2] * inv, lo[3] * inv),
                          pack2<T>(hi[0] * inv, hi[1] * inv), pack2<T>(hi[2] * inv, hi[3] * inv)};
    store16(out + (static_cast<int64_t>(q0 + row) * q_heads + h) * D + piece * 8, packed);
  }
}

}  // namespace

extern "C" int llmq_prefill_attention(const void* q, const void* k, const void* v, void* out, int tokens, int q_heads,
                                      int kv_heads, int head_dim, float scale, int dtype, llmq_stream_t stream) {
  if (tokens < 0 || q_heads <= 0 || kv_heads <= 0) return llmq_host::fail_invalid("bad shape: tokens=%d q_heads=%d kv_heads=%d", tokens, q_heads, kv_heads);
  if (q_heads % kv_heads != 0) return llmq_host::fail_invalid("q_heads %d is not a multiple of kv_heads %d", q_heads, kv_heads);
  if (q_heads > 65535) return llmq_host::fail_invalid("at most 65535 query heads (one grid row each), got %d", q_heads);
  if (head_dim != 64 && head_dim != 128) return llmq_host::fail_invalid("head_dim must be 64 or 128, got %d", head_dim);
  if (!(scale > 0.0f) || scale > 3.0e38f) return llmq_host::fail_invalid("scale must be positive and finite, got %g", static_cast<double>(scale));
  if (dtype != LLMQ_F16 && dtype != LLMQ_BF16) return llmq_host::fail_invalid("q, k, v must be float16 or bfloat16, got dtype code %d", dtype);
  if (tokens == 0) return 0;
  if (!q || !k || !v || !out) return llmq_host::fail_invalid("null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v) | reinterpret_cast<uintptr_t>(out)) & 15u)
    return llmq_host::fail_invalid("q, k, v and out must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((tokens + kQueriesPerGroup - 1) / kQueriesPerGroup, q_heads), block(kWavesPerGroup * kWave);
  const float scale_log2e = scale * 1.4426950408889634f;
#define LLMQ_ATTN(T, D)                                                                                          \
  hipLaunchKernelGGL((prefill_attention_kernel<T, D>), grid, block, 0, s, static_cast<const T*>(q),              \
                     static_cast<const T*>(k), static_cast<const T*>(v), static_cast<T*>(out), tokens, q_heads,   \
                     kv_heads, scale_log2e)
  if (dtype == LLMQ_BF16) {
    if (head_dim == 64) LLMQ_ATTN(bf16_t, 64); else LLMQ_ATTN(bf16_t, 128);
  } else {
    if (head_dim == 64) LLMQ_ATTN(f16_t, 64); else LLMQ_ATTN(f16_t, 128);
  }
#undef LLMQ_ATTN
  return llmq_host::check_launch("prefill_attention_kernel");
}
