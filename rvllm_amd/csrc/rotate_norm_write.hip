// Queries and keys of an attention layer whose rotation covers the first `rot` dimensions of a head and pairs
// dimension i with i + rot / 2, and whose per-head RMS norm may come after the rotation and may have no weight;
// the values may be the keys as they were projected (no value projection).  One wave a head of a token.
//
//   rotation  (u, v) = (x[i], x[i + rot/2]) -> (u cos a - v sin a, v cos a + u sin a), a = position * f_i, i < rot/2;
//             dimensions from `rot` on pass unchanged.  cos and sin come from the step's 32-bit table.
//   norm      x / sqrt(mean(x^2) + eps) * (offset + w[d]) over the head's first `norm_dim` dimensions (all of them,
//             unless the head is stored wider than it is, with zeros behind: then the mean is over the head's own
//             size and the zeros stay zeros); w null: no weight;
//             norm_mode 0: none, 1: before the rotation, 2: after it
//   write     queries to q_out [tokens, nq * hd]; keys (rotated, normed) and values into the paged cache of
//             kv_layout.h at the token's position; a negative page skips the write.  v_col < 0: the value is the
//             key as it came in, before rotation and norm.
//   bias      null, or one 32-bit number for every column of a row of `in`: the projections' biases, added as the
//             row is read (to queries, keys and values alike; the sum is rounded to the activations' type, as a
//             projection with its bias would have been stored)
// All arithmetic is 32-bit; rows of `in` are ld apart and hold the queries from q_col and the keys from k_col on.
#include "common.h"
#include "kv_layout.h"

#define RNW_MAX_HD 512
#define RNW_E (RNW_MAX_HD / RV_WAVE)

template <typename T>
__global__ void __launch_bounds__(256)
rotate_norm_write_kernel(const T* __restrict__ in, long long ld, int q_col, int k_col, int v_col,
                         const float* __restrict__ bias, T* __restrict__ q_out, const void* __restrict__ q_w, const void* __restrict__ k_w, int w_f32,
                         float eps, float offset, int norm_mode, const float* __restrict__ cos_t,
                         const float* __restrict__ sin_t, int rot, const int* __restrict__ positions,
                         const int* __restrict__ token_req, const int* __restrict__ table, int table_width,
                         T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int num_pages, int num_tokens,
                         int nq, int nkv, int hd, int write_kv, int norm_dim) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  const int per_token = nq + nkv;
  if (unit >= (long long)num_tokens * per_token) return;
  const int t = (int)(unit / per_token);
  const int head = (int)(unit - (long long)t * per_token);
  const bool is_q = head < nq;
  if (!is_q && !write_kv) return;
  const int kvh = head - nq;
  const int col0 = is_q ? q_col + head * hd : k_col + kvh * hd;
  const T* src = in + (long long)t * ld + col0;
  const float* b = bias ? bias + col0 : nullptr;
  const void* w = is_q ? q_w : k_w;
  const int half = rot / 2;
  float raw[RNW_E], val[RNW_E];
  float ss_raw = 0.f;
#pragma unroll
  for (int e = 0; e < RNW_E; ++e) {
    const int d = e * RV_WAVE + lane;
    raw[e] = d < hd ? (b ? rv_round_to<T>(rv_to_float(src[d]) + b[d]) : rv_to_float(src[d])) : 0.f;
    ss_raw = fmaf(raw[e], raw[e], ss_raw);
  }
  float inv_before = 1.0f;
  if (norm_mode == 1) inv_before = 1.0f / sqrtf(rv_wave_sum(ss_raw) / (float)norm_dim + eps);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < RNW_E; ++e) {
    const int d = e * RV_WAVE + lane;
    float x = raw[e];
    if (norm_mode == 1 && d < norm_dim) x *= inv_before * (w ? offset + rv_load_w(w, w_f32, d) : 1.0f);
    if (d < rot) {
      const int partner = d < half ? d + half : d - half;
      float y = b ? rv_round_to<T>(rv_to_float(src[partner]) + b[partner]) : rv_to_float(src[partner]);
      if (norm_mode == 1) y *= inv_before * (w ? offset + rv_load_w(w, w_f32, partner) : 1.0f);
      const int i = d < half ? d : d - half;
      const float c = cos_t[(long long)t * half + i], s = sin_t[(long long)t * half + i];
      x = d < half ? x * c - y * s : x * c + y * s;
    }
    val[e] = x;
    ss = fmaf(x, x, ss);
  }
  if (norm_mode == 2) {
    const float inv = 1.0f / sqrtf(rv_wave_sum(ss) / (float)norm_dim + eps);
#pragma unroll
    for (int e = 0; e < RNW_E; ++e) {
      const int d = e * RV_WAVE + lane;
      if (d < norm_dim) val[e] *= inv * (w ? offset + rv_load_w(w, w_f32, d) : 1.0f);
    }
  }
  if (is_q) {
    T* dst = q_out + ((long long)t * nq + head) * hd;
#pragma unroll
    for (int e = 0; e < RNW_E; ++e) {
      const int d = e * RV_WAVE + lane;
      if (d < hd) dst[d] = rv_from_float<T>(val[e]);
    }
    return;
  }
  const int pos = positions[t];
  const int page = table[(long long)token_req[t] * table_width + pos / page_size];
  if (page < 0 || page >= num_pages) return;
  const int slot = pos % page_size;
  const T* vsrc = v_col >= 0 ? in + (long long)t * ld + v_col + kvh * hd : nullptr;
  const float* vb = (bias && v_col >= 0) ? bias + v_col + kvh * hd : nullptr;
#pragma unroll
  for (int e = 0; e < RNW_E; ++e) {
    const int d = e * RV_WAVE + lane;
    if (d < hd) {
      k_pages[rv_k_index(page, kvh, slot, d, nkv, page_size, hd)] = rv_from_float<T>(val[e]);
      v_pages[rv_v_index(page, kvh, slot, d, nkv, page_size, hd)] =
          vsrc ? (vb ? rv_from_float<T>(rv_to_float(vsrc[d]) + vb[d]) : vsrc[d]) : rv_from_float<T>(raw[e]);
    }
  }
}

extern "C" int rv_rotate_norm_write(hipStream_t stream, const void* in, long long ld, int q_col, int k_col, int v_col,
                                    const float* bias, void* q_out, const void* q_w, const void* k_w, int w_f32, float eps, float offset,
                                    int norm_mode, const float* cos_t, const float* sin_t, int rot,
                                    const int* positions, const int* token_req, const int* table, int table_width,
                                    void* k_pages, void* v_pages, int page_size, int num_pages, int dtype,
                                    int num_tokens, int nq, int nkv, int hd, int write_kv, int norm_dim) {
  RV_CHECK(in && q_out && positions && token_req, "rotate_norm_write: null argument");
  RV_CHECK(nq > 0 && nkv > 0 && hd > 0 && hd <= RNW_MAX_HD, "rotate_norm_write: head size %d must be at most %d", hd,
           RNW_MAX_HD);
  RV_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0 && (rot == 0 || (cos_t && sin_t)),
           "rotate_norm_write: %d rotated dimensions of %d need an even count and the step's table", rot, hd);
  RV_CHECK(norm_mode >= 0 && norm_mode <= 2, "rotate_norm_write: norm_mode %d", norm_mode);
  RV_CHECK(norm_dim >= rot && norm_dim >= 1 && norm_dim <= hd,
           "rotate_norm_write: the norm runs over %d of a head's %d dimensions, %d of them rotated", norm_dim, hd, rot);
  RV_CHECK(!write_kv || (table && k_pages && v_pages && page_size > 0 && page_size % RV_V_GROUP == 0),
           "rotate_norm_write: no cache to write to");
  if (num_tokens == 0) return 0;
  const long long units = (long long)num_tokens * (nq + nkv);
  dim3 grid(rv_div_up(units, 4)), block(256);
#define RV_RNW(T)                                                                                                    \
  rotate_norm_write_kernel<T><<<grid, block, 0, stream>>>((const T*)in, ld, q_col, k_col, v_col, bias, (T*)q_out, q_w, k_w, \
                                                          w_f32, eps, offset, norm_mode, cos_t, sin_t, rot, positions, \
                                                          token_req, table, table_width, (T*)k_pages, (T*)v_pages,     \
                                                          page_size, num_pages, num_tokens, nq, nkv, hd, write_kv, norm_dim)
  if (dtype == RV_F32) RV_RNW(float);
  else if (dtype == RV_BF16) RV_RNW(bf16_t);
  else return rv_fail("rotate_norm_write: unsupported dtype %d", dtype);
#undef RV_RNW
  RV_LAUNCH_CHECK("rotate_norm_write");
  return 0;
}
