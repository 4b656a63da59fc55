// Layer norm with weight and bias, and the residual sum of a model that keeps several copies ("streams") of its
// residual stream and mixes them with learned weights (hyper-connections):
//
//   layernorm        y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b         x float or T, y of type T
//   streams_update   for the S streams x_1 .. x_S of a token ([S, tokens, width], float, in place) and a sublayer's
//                    result y (type T, or unreduced 32-bit partial sums, or wa * y + wb * y2 of two of these):
//                      x_t <- sum_s mix[s, t] x_s + mult * out[t] * (ls .* y)          all streams from the old ones
//                    then, optionally, the next sublayer's input and its norm in one go:
//                      u = sum_s in[s] x_s;   next = layernorm(u)                      (type T)
//                    and, optionally, total = sum_s x_s (float [tokens, width]).
//                    Without y the streams are only read (the first sublayer of a step); with `seed` they are first
//                    set to S copies of `seed` (float [tokens, width]: the embedding's output).
//
// All arithmetic is 32-bit.  A block takes a row; the order of a row's additions depends on the width alone.
#include "common.h"

#define SN_THREADS 256
#define SN_MAX_STREAMS 8

template <typename T>
__device__ __forceinline__ float sn_branch(const void* p, int slices, long long stride, size_t at) {
  if (slices == 0) return rv_to_float(((const T*)p)[at]);
  const float* q = (const float*)p + at;
  float v = 0.f;
  int s = 0;
  for (; s + 4 <= slices; s += 4) {  // four reads on their way at a time; the sums in the slices' order as ever
    const float a = q[(size_t)s * stride], b = q[(size_t)(s + 1) * stride], c = q[(size_t)(s + 2) * stride],
                d = q[(size_t)(s + 3) * stride];
    v += a;
    v += b;
    v += c;
    v += d;
  }
  for (; s < slices; ++s) v += q[(size_t)s * stride];
  return v;
}

// mean and 1 / sqrt(variance + eps) of the row whose values the threads hold in u[E] (element e * SN_THREADS + tid);
// E == 0: the values are read again from `again` (float, the row's start).
template <int E>
__device__ __forceinline__ void sn_moments(const float* u, const float* again, int width, float eps, float* scratch,
                                           float& mean, float& inv) {
  float sum = 0.f;
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) sum += (e * SN_THREADS + (int)threadIdx.x < width) ? u[e] : 0.f;
  } else {
    for (int i = threadIdx.x; i < width; i += SN_THREADS) sum += again[i];
  }
  mean = rv_block_sum(sum, scratch) / (float)width;
  float dev = 0.f;
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float d = (e * SN_THREADS + (int)threadIdx.x < width) ? u[e] - mean : 0.f;
      dev = fmaf(d, d, dev);
    }
  } else {
    for (int i = threadIdx.x; i < width; i += SN_THREADS) {
      const float d = again[i] - mean;
      dev = fmaf(d, d, dev);
    }
  }
  inv = 1.0f / sqrtf(rv_block_sum(dev, scratch) / (float)width + eps);
}

template <typename TI, typename TO, int E>
__global__ void __launch_bounds__(SN_THREADS)
layernorm_kernel(const TI* __restrict__ x, const int* __restrict__ row_index, const void* __restrict__ w,
                 const void* __restrict__ b, int wb_f32, TO* __restrict__ y, int width, float eps) {
  __shared__ float scratch[16];
  const int in_row = row_index ? row_index[blockIdx.x] : (int)blockIdx.x;
  const TI* xr = x + (size_t)in_row * width;
  TO* yr = y + (size_t)blockIdx.x * width;
  constexpr int N = E > 0 ? E : 1;
  float u[N];
  float mean, inv;
  if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      u[e] = i < width ? rv_to_float(xr[i]) : 0.f;
    }
    sn_moments<E>(u, nullptr, width, eps, scratch, mean, inv);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      if (i < width) yr[i] = rv_from_float<TO>((u[e] - mean) * inv * rv_load_w(w, wb_f32, i) + rv_load_w(b, wb_f32, i));
    }
  } else {
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += SN_THREADS) sum += rv_to_float(xr[i]);
    mean = rv_block_sum(sum, scratch) / (float)width;
    float dev = 0.f;
    for (int i = threadIdx.x; i < width; i += SN_THREADS) {
      const float d = rv_to_float(xr[i]) - mean;
      dev = fmaf(d, d, dev);
    }
    inv = 1.0f / sqrtf(rv_block_sum(dev, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += SN_THREADS)
      yr[i] = rv_from_float<TO>((rv_to_float(xr[i]) - mean) * inv * rv_load_w(w, wb_f32, i) + rv_load_w(b, wb_f32, i));
  }
}

// w and b are both float (wb_f32) or both bf16.
extern "C" int rv_layernorm(hipStream_t stream, const void* x, int x_dtype, const int* row_index, const void* w,
                            const void* b, int wb_f32, void* y, int y_dtype, int rows, int width, float eps) {
  RV_CHECK(rows >= 0 && width > 0 && x && w && b && y, "layernorm: bad arguments rows=%d width=%d", rows, width);
  if (rows == 0) return 0;
  dim3 grid(rows), block(SN_THREADS);
#define RV_LN(TI, TO, E) \
  layernorm_kernel<TI, TO, E><<<grid, block, 0, stream>>>((const TI*)x, row_index, w, b, wb_f32, (TO*)y, width, eps)
#define RV_LN_T(TI, TO)                              \
  do {                                               \
    const int e_ = rv_div_up(width, SN_THREADS);     \
    if (e_ <= 1) RV_LN(TI, TO, 1);                   \
    else if (e_ <= 4) RV_LN(TI, TO, 4);              \
    else if (e_ <= 16) RV_LN(TI, TO, 16);            \
    else RV_LN(TI, TO, 0);                           \
  } while (0)
  if (x_dtype == RV_F32 && y_dtype == RV_F32) RV_LN_T(float, float);
  else if (x_dtype == RV_F32 && y_dtype == RV_BF16) RV_LN_T(float, bf16_t);
  else if (x_dtype == RV_BF16 && y_dtype == RV_BF16) RV_LN_T(bf16_t, bf16_t);
  else return rv_fail("layernorm: unsupported dtypes %d -> %d", x_dtype, y_dtype);
#undef RV_LN_T
#undef RV_LN
  RV_LAUNCH_CHECK("layernorm");
  return 0;
}

struct StreamsParams {
  float* streams;            // [S, tokens, width]
  long long stream_stride;   // tokens * width
  const float* seed;         // [tokens, width] or null
  const void* branch;        // T or partial sums; null: the streams are only read
  int slices;
  long long slice_stride;
  const void* branch2;       // null, or the second of two weighted branches
  int slices2;
  long long slice_stride2;
  float wa, wb;
  const float* layer_scale;  // [width] or null
  const float* mix;          // [S, S], from -> to
  const float* out_w;        // [S]
  float mult;
  const float* in_w;         // [S] of the next sublayer, or null
  const void* norm_w;        // the next norm's weight and bias
  const void* norm_b;
  int norm_f32;
  void* next;                // T [tokens, width], with in_w
  float* total;              // [tokens, width] or null
  int S, width;
  float eps;
};

// ST: the number of streams where it is one of the usual few (their sums are then written out in registers), 0: any
// number up to SN_MAX_STREAMS.  A stream's sum over the old streams is added in their order either way.
template <typename T, int E, int ST>
__global__ void __launch_bounds__(SN_THREADS) streams_update_kernel(StreamsParams P) {
  __shared__ float scratch[16];
  __shared__ float s_mix[SN_MAX_STREAMS * SN_MAX_STREAMS], s_out[SN_MAX_STREAMS], s_in[SN_MAX_STREAMS];
  constexpr int SMAX = ST > 0 ? ST : SN_MAX_STREAMS;
  const int S = ST > 0 ? ST : P.S, width = P.width;
  const size_t row0 = (size_t)blockIdx.x * width;
  if (threadIdx.x < S * S) s_mix[threadIdx.x] = P.branch ? P.mix[threadIdx.x] : 0.f;
  if (threadIdx.x < S) {
    s_out[threadIdx.x] = P.branch ? P.mult * P.out_w[threadIdx.x] : 0.f;
    s_in[threadIdx.x] = P.in_w ? P.in_w[threadIdx.x] : 0.f;
  }
  __syncthreads();
  constexpr int N = E > 0 ? E : 1;
  float u[N];
  // one element of the row: its streams moved on and written, the next sublayer's input returned
  auto element = [&](int i) -> float {
    float old[SMAX], fresh[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s)
      if (s < S) old[s] = P.seed ? P.seed[row0 + i] : P.streams[(size_t)s * P.stream_stride + row0 + i];
    if (P.branch) {
      float y = sn_branch<T>(P.branch, P.slices, P.slice_stride, row0 + i);
      if (P.branch2) y = P.wa * y + P.wb * sn_branch<T>(P.branch2, P.slices2, P.slice_stride2, row0 + i);
      if (P.layer_scale) y *= P.layer_scale[i];
#pragma unroll
      for (int t = 0; t < SMAX; ++t) {
        if (t < S) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < SMAX; ++s)
            if (s < S) acc = fmaf(s_mix[s * S + t], old[s], acc);
          fresh[t] = fmaf(s_out[t], y, acc);
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SMAX; ++s)
        if (s < S) fresh[s] = old[s];
    }
    float in_sum = 0.f, all = 0.f;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
      if (s < S) {
        if (P.branch || P.seed) P.streams[(size_t)s * P.stream_stride + row0 + i] = fresh[s];
        in_sum = fmaf(s_in[s], fresh[s], in_sum);
        all += fresh[s];
      }
    }
    if (P.total) P.total[row0 + i] = all;
    return in_sum;
  };
  if constexpr (E > 0 && ST > 0) {
    // a few streams and a row that the registers hold: everything a thread's elements need is asked for first (the
    // old streams, the branch with all its slices), then worked on, so that the reads of one element do not wait
    // behind the writes of the one before
    float olds[E][SMAX], ys[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      ys[e] = 0.f;
#pragma unroll
      for (int s = 0; s < SMAX; ++s) olds[e][s] = 0.f;
      if (i < width) {
#pragma unroll
        for (int s = 0; s < SMAX; ++s)
          olds[e][s] = P.seed ? P.seed[row0 + i] : P.streams[(size_t)s * P.stream_stride + row0 + i];
        if (P.branch) {
          float y = sn_branch<T>(P.branch, P.slices, P.slice_stride, row0 + i);
          if (P.branch2) y = P.wa * y + P.wb * sn_branch<T>(P.branch2, P.slices2, P.slice_stride2, row0 + i);
          if (P.layer_scale) y *= P.layer_scale[i];
          ys[e] = y;
        }
      }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      u[e] = 0.f;
      if (i < width) {
        float fresh[SMAX];
#pragma unroll
        for (int t = 0; t < SMAX; ++t) {
          if (P.branch) {
            float acc = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < SMAX; ++s2) acc = fmaf(s_mix[s2 * S + t], olds[e][s2], acc);
            fresh[t] = fmaf(s_out[t], ys[e], acc);
          } else {
            fresh[t] = olds[e][t];
          }
        }
        float in_sum = 0.f, all = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < SMAX; ++s2) {
          if (P.branch || P.seed) P.streams[(size_t)s2 * P.stream_stride + row0 + i] = fresh[s2];
          in_sum = fmaf(s_in[s2], fresh[s2], in_sum);
          all += fresh[s2];
        }
        if (P.total) P.total[row0 + i] = all;
        u[e] = in_sum;
      }
    }
  } else if constexpr (E > 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      u[e] = i < width ? element(i) : 0.f;
    }
  } else {
    for (int i = threadIdx.x; i < width; i += SN_THREADS) element(i);
  }
  if (P.in_w == nullptr) return;
  T* next = (T*)P.next + row0;
  float mean, inv;
  if constexpr (E > 0) {
    sn_moments<E>(u, nullptr, width, P.eps, scratch, mean, inv);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int i = e * SN_THREADS + threadIdx.x;
      if (i < width)
        next[i] = rv_from_float<T>((u[e] - mean) * inv * rv_load_w(P.norm_w, P.norm_f32, i) + rv_load_w(P.norm_b, P.norm_f32, i));
    }
  } else {
    // a row wider than the registers hold: the input is worked out again from the streams (a thread reads back
    // what it wrote itself), once for each of the three passes
    auto again = [&](int i) -> float {
      float in_sum = 0.f;
      for (int s = 0; s < S; ++s) in_sum = fmaf(s_in[s], P.streams[(size_t)s * P.stream_stride + row0 + i], in_sum);
      return in_sum;
    };
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += SN_THREADS) sum += again(i);
    mean = rv_block_sum(sum, scratch) / (float)width;
    float dev = 0.f;
    for (int i = threadIdx.x; i < width; i += SN_THREADS) {
      const float d = again(i) - mean;
      dev = fmaf(d, d, dev);
    }
    inv = 1.0f / sqrtf(rv_block_sum(dev, scratch) / (float)width + P.eps);
    for (int i = threadIdx.x; i < width; i += SN_THREADS)
      next[i] = rv_from_float<T>((again(i) - mean) * inv * rv_load_w(P.norm_w, P.norm_f32, i) + rv_load_w(P.norm_b, P.norm_f32, i));
  }
}

extern "C" int rv_streams_update(hipStream_t stream, float* streams, long long stream_stride, const float* seed,
                                 const void* branch, int slices, long long slice_stride, const void* branch2,
                                 int slices2, long long slice_stride2, float wa, float wb, const float* layer_scale,
                                 const float* mix, const float* out_w, float mult, const float* in_w,
                                 const void* norm_w, const void* norm_b, int norm_f32, void* next, float* total,
                                 int dtype, int num_streams, int rows, int width, float eps) {
  RV_CHECK(streams && rows >= 0 && width > 0 && num_streams >= 1 && num_streams <= SN_MAX_STREAMS,
           "streams_update: bad arguments rows=%d width=%d streams=%d", rows, width, num_streams);
  RV_CHECK(stream_stride >= (long long)rows * width, "streams_update: the streams overlap");
  RV_CHECK(branch == nullptr || (mix && out_w), "streams_update: a branch needs the weights that mix and add it");
  RV_CHECK(branch != nullptr || branch2 == nullptr, "streams_update: a second branch without a first");
  RV_CHECK((in_w == nullptr) == (next == nullptr) && (in_w == nullptr || (norm_w && norm_b)),
           "streams_update: the next sublayer's input needs its weights, its norm and a place");
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= (long long)rows * width) && slices2 >= 0 &&
               (slices2 == 0 || slice_stride2 >= (long long)rows * width),
           "streams_update: bad partial sums");
  if (rows == 0) return 0;
  StreamsParams P;
  P.streams = streams, P.stream_stride = stream_stride, P.seed = seed, P.branch = branch, P.slices = slices;
  P.slice_stride = slice_stride, P.branch2 = branch2, P.slices2 = slices2, P.slice_stride2 = slice_stride2;
  P.wa = wa, P.wb = wb, P.layer_scale = layer_scale, P.mix = mix, P.out_w = out_w, P.mult = mult, P.in_w = in_w;
  P.norm_w = norm_w, P.norm_b = norm_b, P.norm_f32 = norm_f32, P.next = next, P.total = total, P.S = num_streams;
  P.width = width, P.eps = eps;
  dim3 grid(rows), block(SN_THREADS);
#define RV_SU_S(T, E)                                                                            \
  do {                                                                                           \
    if (num_streams == 1) streams_update_kernel<T, E, 1><<<grid, block, 0, stream>>>(P);         \
    else if (num_streams == 2) streams_update_kernel<T, E, 2><<<grid, block, 0, stream>>>(P);    \
    else if (num_streams == 4) streams_update_kernel<T, E, 4><<<grid, block, 0, stream>>>(P);    \
    else streams_update_kernel<T, E, 0><<<grid, block, 0, stream>>>(P);                          \
  } while (0)
#define RV_SU_T(T)                                   \
  do {                                               \
    const int e_ = rv_div_up(width, SN_THREADS);     \
    if (e_ <= 1) RV_SU_S(T, 1);                      \
    else if (e_ <= 4) RV_SU_S(T, 4);                 \
    else if (e_ <= 8) RV_SU_S(T, 8);                 \
    else if (e_ <= 16) RV_SU_S(T, 16);               \
    else RV_SU_S(T, 0);                              \
  } while (0)
  if (dtype == RV_F32) RV_SU_T(float);
  else if (dtype == RV_BF16) RV_SU_T(bf16_t);
  else return rv_fail("streams_update: unsupported dtype %d", dtype);
#undef RV_SU_T
#undef RV_SU_S
  RV_LAUNCH_CHECK("streams_update");
  return 0;
}
