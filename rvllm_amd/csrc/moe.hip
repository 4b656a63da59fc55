// Routing for a mixture of experts whose experts are chosen by the token's id: a table [vocab, top] names each
// id's experts.  Nothing here waits for the host: the sorted order is made on the device, with room for the worst
// case, so a step's launches do not depend on the tokens and can be replayed from a graph.
//
//   moe_route     sorts the step's (token, choice) pairs by expert.  Each expert's rows start at a multiple of
//                 `tile` rows (the grouped product takes a tile of rows against one expert's matrix):
//                   slot_of[t * top + k]   the sorted row of token t's k-th choice
//                   row_token[r]           the token of sorted row r, -1 for the filling rows
//                   tile_group[r / tile]   the expert of a tile of rows, -1 for tiles past the last expert's
//                 `capacity` rows (a multiple of tile) hold every case: tokens * top + experts * (tile - 1) at most.
//   moe_combine   out[t] = weight * sum_k y[slot_of[t * top + k]] (+ shared[t]), the sum in 32-bit, choices in order
//
// The place of a row inside its expert's rows depends on the order in which the threads arrive; each row's result
// does not, since the products work row by row.
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_THREADS 1024

__global__ void __launch_bounds__(MOE_THREADS)
moe_route_kernel(const int* __restrict__ token_ids, int num_tokens, const int* __restrict__ table, int vocab, int top,
                 int experts, int tile, int capacity, int* __restrict__ slot_of, int* __restrict__ row_token,
                 int* __restrict__ tile_group) {
  __shared__ int count[MOE_MAX_EXPERTS];
  __shared__ int first[MOE_MAX_EXPERTS];
  const int tid = threadIdx.x;
  const int slots = num_tokens * top;
  for (int e = tid; e < experts; e += MOE_THREADS) count[e] = 0;
  for (int r = tid; r < capacity; r += MOE_THREADS) row_token[r] = -1;
  for (int i = tid; i < capacity / tile; i += MOE_THREADS) tile_group[i] = -1;
  __syncthreads();
  for (int s = tid; s < slots; s += MOE_THREADS) {
    const int id = token_ids[s / top];
    const int e = (id >= 0 && id < vocab) ? table[(size_t)id * top + s % top] : -1;
    if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = at;
      const int tiles = (count[e] + tile - 1) / tile;
      for (int i = 0; i < tiles; ++i) tile_group[at / tile + i] = e;
      at += tiles * tile;
      count[e] = 0;  // counts again below, as the rows take their places
    }
  }
  __syncthreads();
  for (int s = tid; s < slots; s += MOE_THREADS) {
    const int id = token_ids[s / top];
    const int e = (id >= 0 && id < vocab) ? table[(size_t)id * top + s % top] : -1;
    int row = -1;
    if (e >= 0 && e < experts) {
      row = first[e] + atomicAdd(&count[e], 1);
      row_token[row] = s / top;
    }
    slot_of[s] = row;  // -1: the table names no expert of this layer; the choice adds nothing
  }
}

extern "C" int rv_moe_route(hipStream_t stream, const int* token_ids, int num_tokens, const int* table, int vocab,
                            int top, int experts, int tile, int capacity, int* slot_of, int* row_token,
                            int* tile_group) {
  RV_CHECK(num_tokens >= 0 && vocab > 0 && top > 0, "moe_route: bad sizes tokens=%d vocab=%d top=%d", num_tokens, vocab, top);
  RV_CHECK(experts > 0 && experts <= MOE_MAX_EXPERTS, "moe_route: %d experts, at most %d are supported", experts,
           MOE_MAX_EXPERTS);
  RV_CHECK(tile > 0 && capacity % tile == 0 && (long long)capacity >= (long long)num_tokens * top + (long long)experts * (tile - 1),
           "moe_route: %d rows do not hold every case of %d choices among %d experts in tiles of %d", capacity,
           num_tokens * top, experts, tile);
  if (num_tokens == 0) return 0;
  moe_route_kernel<<<dim3(1), dim3(MOE_THREADS), 0, stream>>>(token_ids, num_tokens, table, vocab, top, experts, tile,
                                                             capacity, slot_of, row_token, tile_group);
  RV_LAUNCH_CHECK("moe_route");
  return 0;
}

template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int* __restrict__ slot_of, int top, float weight,
                                   const void* __restrict__ shared, int shared_slices, long long shared_stride,
                                   T* __restrict__ out, int width) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const size_t at = (size_t)t * width + i;
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
      const int row = slot_of[(size_t)t * top + k];
      if (row >= 0) acc += rv_to_float(y[(size_t)row * width + i]);
    }
    acc *= weight;
    if (shared != nullptr) {
      if (shared_slices == 0) {
        acc += rv_to_float(((const T*)shared)[at]);
      } else {  // the K slices of the shared expert's last product, added in their order, then rounded as stored
        float sum = 0.f;
        const float* p = (const float*)shared + at;
        int s = 0;
        for (; s + 4 <= shared_slices; s += 4) {  // four reads on their way together, added in the slices' order
          const float q0 = p[(size_t)s * shared_stride], q1 = p[(size_t)(s + 1) * shared_stride];
          const float q2 = p[(size_t)(s + 2) * shared_stride], q3 = p[(size_t)(s + 3) * shared_stride];
          sum += q0, sum += q1, sum += q2, sum += q3;
        }
        for (; s < shared_slices; ++s) sum += p[(size_t)s * shared_stride];
        acc += rv_round_to<T>(sum);
      }
    }
    out[at] = rv_from_float<T>(acc);
  }
}

// shared: null, values of type `dtype` [tokens, width] (shared_slices 0), or 32-bit partial sums
// [shared_slices][tokens][width], shared_stride elements apart.
extern "C" int rv_moe_combine(hipStream_t stream, const void* y, const int* slot_of, int top, float weight,
                              const void* shared, int shared_slices, long long shared_stride, void* out, int dtype,
                              int num_tokens, int width) {
  RV_CHECK(num_tokens >= 0 && width > 0 && top > 0, "moe_combine: bad sizes tokens=%d width=%d top=%d", num_tokens, width, top);
  RV_CHECK(shared_slices >= 0 && (shared_slices == 0 || shared_stride >= (long long)num_tokens * width),
           "moe_combine: bad partial sums");
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens), block(width >= 1024 ? 1024 : (width > 256 ? 512 : 256));  // few rows: a row's reads side by side
  if (dtype == RV_F32)
    moe_combine_kernel<float><<<grid, block, 0, stream>>>((const float*)y, slot_of, top, weight, shared, shared_slices,
                                                          shared_stride, (float*)out, width);
  else if (dtype == RV_BF16)
    moe_combine_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)y, slot_of, top, weight, shared,
                                                           shared_slices, shared_stride, (bf16_t*)out, width);
  else
    return rv_fail("moe_combine: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("moe_combine");
  return 0;
}

// ---------------------------------------------------------------------------
// Routing by the activations: a router's 32-bit logits [tokens, experts] give every token the `top` experts with
// the largest logits (the largest first; of equal ones the lower index), each with the weight sigmoid(logit) (mode
// 0).  A wave a token: every lane holds the logits e * 64 + lane, the largest is found by a sum-free exchange
// (value, then index) and struck out, `top` times.  The result, chosen [tokens, top], is a table for moe_route
// with the token's row as its id.
// ---------------------------------------------------------------------------
#define MOE_TOPK_PER (MOE_MAX_EXPERTS / RV_WAVE)

__global__ void __launch_bounds__(256)
moe_topk_kernel(const float* __restrict__ logits, int num_tokens, int experts, int top, int* __restrict__ chosen,
                float* __restrict__ weights) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int t = blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  if (t >= num_tokens) return;  // the whole wave
  const float* row = logits + (size_t)t * experts;
  float v[MOE_TOPK_PER];
#pragma unroll
  for (int e = 0; e < MOE_TOPK_PER; ++e) {
    const int i = e * RV_WAVE + lane;
    const float x = i < experts ? row[i] : -INFINITY;
    v[e] = x == x ? x : -INFINITY;  // a NaN is never chosen
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int e = 0; e < MOE_TOPK_PER; ++e) {
      const int i = e * RV_WAVE + lane;
      if (i < experts && (v[e] > best || (v[e] == best && i < at))) best = v[e], at = i;
    }
#pragma unroll
    for (int off = RV_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, RV_WAVE);
      const int oa = __shfl_xor(at, off, RV_WAVE);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    if (at >= experts) at = k;  // nothing left to choose from (every logit NaN or struck out): any expert, weight 0
    if (lane == 0) {
      chosen[(size_t)t * top + k] = at;
      weights[(size_t)t * top + k] = best > -INFINITY ? 1.0f / (1.0f + expf(-best)) : 0.f;
    }
#pragma unroll
    for (int e = 0; e < MOE_TOPK_PER; ++e)
      if (e * RV_WAVE + lane == at) v[e] = -INFINITY;
  }
}

extern "C" int rv_moe_topk(hipStream_t stream, const float* logits, int num_tokens, int experts, int top, int* chosen,
                           float* weights) {
  RV_CHECK(logits && chosen && weights && num_tokens >= 0, "moe_topk: bad arguments");
  RV_CHECK(experts > 0 && experts <= MOE_MAX_EXPERTS && top > 0 && top <= experts,
           "moe_topk: %d of %d experts (at most %d)", top, experts, MOE_MAX_EXPERTS);
  if (num_tokens == 0) return 0;
  moe_topk_kernel<<<dim3(rv_div_up(num_tokens, 4)), dim3(256), 0, stream>>>(logits, num_tokens, experts, top, chosen,
                                                                            weights);
  RV_LAUNCH_CHECK("moe_topk");
  return 0;
}

// xs[slot_of[p]] = weights[p] * x[p / top], rounded to T: the rows of the experts' first product where a choice's
// weight multiplies the expert's input.  A block a (token, choice) pair; a pair without a row is skipped; rows of
// xs that no pair names are left as they are.
template <typename T>
__global__ void moe_scale_rows_kernel(const T* __restrict__ x, const int* __restrict__ slot_of,
                                      const float* __restrict__ weights, int top, T* __restrict__ xs, int width) {
  const int p = blockIdx.x;
  const int row = slot_of[p];
  if (row < 0) return;
  const float w = weights[p];
  const T* src = x + (size_t)(p / top) * width;
  T* dst = xs + (size_t)row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = rv_from_float<T>(w * rv_to_float(src[i]));
}

extern "C" int rv_moe_scale_rows(hipStream_t stream, const void* x, const int* slot_of, const float* weights, int top,
                                 void* xs, int dtype, int num_tokens, int width) {
  RV_CHECK(x && slot_of && weights && xs && num_tokens >= 0 && top > 0 && width > 0, "moe_scale_rows: bad arguments");
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens * top), block(256);
  if (dtype == RV_F32)
    moe_scale_rows_kernel<float><<<grid, block, 0, stream>>>((const float*)x, slot_of, weights, top, (float*)xs, width);
  else if (dtype == RV_BF16)
    moe_scale_rows_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, slot_of, weights, top, (bf16_t*)xs, width);
  else
    return rv_fail("moe_scale_rows: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("moe_scale_rows");
  return 0;
}
