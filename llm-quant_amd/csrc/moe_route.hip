// Routing plan of a Mixture-of-Experts layer in one launch, and the weighted sum of the experts'
// outputs per token in another.
//
// KernelQuantExperts._plan (llmquant/quantizers/kernel.py:176-214) builds the plan of the batched
// GEMV from about ten PyTorch kernels (stable argsort, scatter_add, cumsum, arange arithmetic):
// ~45 us per layer under graph replay, three times the two GEMVs it prepares. The batched path only
// runs for a handful of tokens, i.e. a few dozen (token, slot) rows, so one workgroup does all of it:
//   order      stable sort of the rows by expert (a counting sort: thread e walks the rows in
//              order and places those of expert e, so equal keys keep their order)
//   blocks     every expert gets per_expert = max(1, ceil(rows / limit)) entries
//              (expert, first[e] + b * limit, clamp(count[e] - b * limit, 0, limit)),
//              first = exclusive prefix sum of the per-expert counts
// The results are the integers the PyTorch form produces.
#include "llmq_device.h"

namespace {

constexpr int kRouteThreads = 1024;
constexpr int kRouteMaxExperts = 1024;   // one thread per expert
constexpr int kRouteMaxRows = 8192;      // expert ids staged in LDS as 16-bit values

__global__ __launch_bounds__(kRouteThreads) void route_plan_kernel(
    const int64_t* __restrict__ expert_of_row, const int n_rows, const int n_experts, const int limit,
    const int per_expert, int64_t* __restrict__ order, int32_t* __restrict__ block_expert,
    int32_t* __restrict__ block_row0, int32_t* __restrict__ block_rows) {
  __shared__ uint16_t s_id[kRouteMaxRows];
  __shared__ int s_count[kRouteMaxExperts];
  __shared__ int s_scan[2][kRouteMaxExperts];
  const int tid = threadIdx.x;

  if (tid < n_experts) s_count[tid] = 0;
  __syncthreads();
  for (int i = tid; i < n_rows; i += kRouteThreads) {
    // an id outside the layer's experts is counted with the nearest valid one
    const int64_t raw = expert_of_row[i];
    const int e = raw < 0 ? 0 : (raw >= n_experts ? n_experts - 1 : static_cast<int>(raw));
    s_id[i] = static_cast<uint16_t>(e);
    atomicAdd(&s_count[e], 1);
  }
  __syncthreads();

  // inclusive prefix sum over the experts (doubling steps), then exclusive = inclusive - count
  int src = 0;
  if (tid < n_experts) s_scan[0][tid] = s_count[tid];
  __syncthreads();
  for (int step = 1; step < n_experts; step <<= 1) {
    if (tid < n_experts) s_scan[src ^ 1][tid] = s_scan[src][tid] + (tid >= step ? s_scan[src][tid - step] : 0);
    __syncthreads();
    src ^= 1;
  }
  const int count = tid < n_experts ? s_count[tid] : 0;
  const int first = tid < n_experts ? s_scan[src][tid] - count : 0;

  // stable placement: thread e visits the rows in order
  if (tid < n_experts && count > 0) {
    int pos = first;
    for (int i = 0; i < n_rows; ++i) {
      if (s_id[i] == tid) order[pos++] = i;
    }
  }
  // the blocks of expert e
  if (tid < n_experts) {
    for (int b = 0; b < per_expert; ++b) {
      const int step = b * limit;
      const int left = count - step;
      const int slot = tid * per_expert + b;
      block_expert[slot] = tid;
      block_row0[slot] = first + step;
      block_rows[slot] = left < 0 ? 0 : (left > limit ? limit : left);
    }
  }
}

// final[t, c] = the rows routed from token t, each times its routing weight, added up in sorted
// order with every product and sum rounded to T. One thread per (token, column).
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const T* __restrict__ rows_out,
                                                          const int64_t* __restrict__ order,
                                                          const T* __restrict__ weights, T* __restrict__ final_out,
                                                          const int n_rows, const int top_k, const int width) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int t = blockIdx.y;
  if (c >= width) return;
  float acc = 0.0f;
  for (int i = 0; i < n_rows; ++i) {
    const int64_t flat = order[i];  // the same address for the whole workgroup
    // (an entry that is not a row index of this problem names no token here: skipped)
    if (flat < 0 || flat / top_k != t) continue;
    const float prod = llmq::round_through<T>(llmq::to_float(rows_out[static_cast<int64_t>(i) * width + c]) *
                                              llmq::to_float(weights[flat]));
    acc = llmq::round_through<T>(acc + prod);
  }
  final_out[static_cast<int64_t>(t) * width + c] = llmq::from_float<T>(acc);
}

}  // namespace

extern "C" int llmq_moe_combine(const void* rows_out, const int64_t* order, const void* weights, void* final_out,
                                int n_rows, int top_k, int n_tokens, int width, int dtype, llmq_stream_t stream) {
  if (n_rows < 0 || top_k <= 0 || n_tokens < 0 || width < 0)
    return llmq_host::fail_invalid("bad dimension rows=%d top_k=%d tokens=%d width=%d", n_rows, top_k, n_tokens, width);
  if (n_tokens == 0 || width == 0) return 0;
  if (n_tokens > 65535) return llmq_host::fail_invalid("at most 65535 tokens per launch, got %d", n_tokens);
  if (!final_out || !weights || (n_rows > 0 && (!rows_out || !order))) return llmq_host::fail_invalid("null tensor pointer");
  const dim3 grid((width + 255) / 256, n_tokens), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LLMQ_COMBINE(T)                                                                                       \
  hipLaunchKernelGGL(moe_combine_kernel<T>, grid, block, 0, s, static_cast<const T*>(rows_out), order,        \
                     static_cast<const T*>(weights), static_cast<T*>(final_out), n_rows, top_k, width)
  switch (dtype) {
    case LLMQ_F32: LLMQ_COMBINE(float); break;
    case LLMQ_F16: LLMQ_COMBINE(llmq::f16_t); break;
    case LLMQ_BF16: LLMQ_COMBINE(llmq::bf16_t); break;
    default: return llmq_host::fail_invalid("dtype code %d is not float32, float16 or bfloat16", dtype);
  }
#undef LLMQ_COMBINE
  return llmq_host::check_launch("moe_combine_kernel");
}

extern "C" int llmq_route_plan_blocks_per_expert(int n_rows, int limit) {
  if (limit <= 0) return 0;
  const int blocks = (n_rows + limit - 1) / limit;
  return blocks < 1 ? 1 : blocks;
}

extern "C" int llmq_route_plan_supported(int n_rows, int n_experts) {
  return n_rows >= 0 && n_rows <= kRouteMaxRows && n_experts >= 1 && n_experts <= kRouteMaxExperts ? 1 : 0;
}

extern "C" int llmq_route_plan(const int64_t* expert_of_row, int n_rows, int n_experts, int limit, int64_t* order,
                               int32_t* block_expert, int32_t* block_row0, int32_t* block_rows,
                               llmq_stream_t stream) {
  if (limit <= 0) return llmq_host::fail_invalid("the run length limit must be positive, got %d", limit);
  if (!llmq_route_plan_supported(n_rows, n_experts))
    return llmq_host::fail_invalid("the routing-plan kernel takes up to %d rows and %d experts, got %d and %d",
                                   kRouteMaxRows, kRouteMaxExperts, n_rows, n_experts);
  if (!block_expert || !block_row0 || !block_rows || (n_rows > 0 && (!expert_of_row || !order)))
    return llmq_host::fail_invalid("null tensor pointer");
  hipLaunchKernelGGL(route_plan_kernel, dim3(1), dim3(kRouteThreads), 0, static_cast<hipStream_t>(stream),
                     expert_of_row, n_rows, n_experts, limit, llmq_route_plan_blocks_per_expert(n_rows, limit), order,
                     block_expert, block_row0, block_rows);
  return llmq_host::check_launch("route_plan_kernel");
}
