// Two more mixers that carry a state of fixed size from token to token:
//
//   matrix memory (the mLSTM of xLSTM), a head at a time, with log gates i and f and a running maximum m that
//   keeps the exponentials in range (m starts at 0):
//       m' = max(f + m, i);  keep = e^(f + m - m'),  take = e^(i - m')
//       S' = keep S + take k v^T;   n' = keep n + take k;   o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)
//     memory_gates   walks n and m (a vector and a number a head) and leaves keep, take and the divisor of every
//                    token; the log gates come from capped inputs: i = cap tanh((a + b_i) / cap),
//                    f = logsigmoid(cap tanh((a' + b_f) / cap))
//     memory_matrix  walks S with these and reads it out
//
//   gated linear recurrent unit (the real-gated LRU of Griffin), a channel at a time:
//       r = sigmoid(g_r + b_r),  i = sigmoid(g_i + b_i),  log a = -8 r softplus(lam),  a = e^(log a)
//       S' = a S + sqrt(1 - a^2) i u;   out = S' * gelu_tanh(y)
//
// The states, gates, decays, their exponentials and logarithms are 32-bit whatever the activations' type T.  A
// request's tokens are walked in their order by the lanes that own a part of its state, and nothing is added across
// waves, so what a token's output is does not depend on how the request's tokens were cut into steps or on what
// else the step holds.  The state of a request lies in its slot, `slot_stride` floats apart from the next; a slot
// is all zeros when a request gets it.
#include "common.h"

__device__ __forceinline__ float rg_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float rg_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

template <int CTRL>
__device__ __forceinline__ float rg_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// Sum over LANES (a power of two) neighbouring lanes that share a column; every one of them gets it.
template <int LANES>
__device__ __forceinline__ float rg_group_sum(float v) {
  if constexpr (LANES >= 2) v += rg_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  if constexpr (LANES >= 4) v += rg_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) v += rg_dpp<0x141>(v);   // row_half_mirror
  if constexpr (LANES >= 16) v += rg_dpp<0x140>(v);  // row_mirror
  if constexpr (LANES >= 32) v += __shfl_xor(v, 16, RV_WAVE);
  if constexpr (LANES >= 64) v += __shfl_xor(v, 32, RV_WAVE);
  return v;
}

// ---------------------------------------------------------------------------
// memory_gates.  A wave a (head, request); lane l holds the elements e * 64 + l of n.  The tokens' keys and queries
// come CHUNK at a time into registers, a chunk ahead of the one worked on; a token's log gates are worked out by
// the lane of its place in the chunk and handed round.
//   rows  T [tokens, ld]: q of head h at q_col + h dk, k at k_col + h dk, the gates' inputs at i_col + h, f_col + h
//   n [heads, dk] at n_off and m [heads] at m_off of the request's slot
//   gates float [tokens, heads, 3]: keep, take, the divisor
// ---------------------------------------------------------------------------
template <typename T, int PER, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
memory_gates_kernel(const T* __restrict__ rows, long long ld, int q_col, int k_col, int i_col, int f_col,
                    const float* __restrict__ i_bias, const float* __restrict__ f_bias, float cap, float q_scale,
                    float* __restrict__ state, long long slot_stride, long long n_off, long long m_off,
                    const int* __restrict__ q_start, const int* __restrict__ state_slot, float* __restrict__ gates,
                    int heads, int dk) {
  const int lane = threadIdx.x;
  const int h = blockIdx.x;
  const int req = blockIdx.y;
  float* slot = state + (long long)state_slot[req] * slot_stride;
  float* n_mem = slot + n_off + (long long)h * dk;
  float n[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) n[e] = e * RV_WAVE + lane < dk ? n_mem[e * RV_WAVE + lane] : 0.f;
  float m = slot[m_off + h];
  const float bi = i_bias[h], bf = f_bias[h];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float nk[CHUNK][PER], nq[CHUNK][PER], ngi = 0.f, ngf = 0.f;  // the chunk ahead
  auto fetch = [&](int tb) {
#pragma unroll
    for (int c = 0; c < CHUNK; ++c) {
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        const int d = e * RV_WAVE + lane;
        const bool ok = tb + c < t1 && d < dk;
        const T* row = rows + (long long)(ok ? tb + c : t0) * ld + (long long)h * dk + (ok ? d : 0);
        nk[c][e] = ok ? rv_to_float(row[k_col]) : 0.f;
        nq[c][e] = ok ? rv_to_float(row[q_col]) * q_scale : 0.f;
      }
    }
    const bool ok = lane < CHUNK && tb + lane < t1;
    const T* row = rows + (long long)(ok ? tb + lane : t0) * ld + h;
    ngi = rv_to_float(row[i_col]);
    ngf = rv_to_float(row[f_col]);
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    float k[CHUNK][PER], q[CHUNK][PER];
#pragma unroll
    for (int c = 0; c < CHUNK; ++c)
#pragma unroll
      for (int e = 0; e < PER; ++e) k[c][e] = nk[c][e], q[c][e] = nq[c][e];
    const float log_in = cap * tanhf((ngi + bi) / cap);
    const float capped = cap * tanhf((ngf + bf) / cap);
    const float log_forget = -rg_softplus(-capped);
    if (tb + CHUNK < t1) fetch(tb + CHUNK);
    const int count = min(CHUNK, t1 - tb);
#pragma unroll
    for (int c = 0; c < CHUNK; ++c) {
      if (c < count) {
        const float li = __shfl(log_in, c, RV_WAVE), lf = __shfl(log_forget, c, RV_WAVE);
        const float m_new = fmaxf(lf + m, li);
        const float keep = expf(lf + m - m_new), take = expf(li - m_new);
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < PER; ++e) {
          n[e] = fmaf(take, k[c][e], keep * n[e]);
          dot = fmaf(n[e], q[c][e], dot);
        }
        dot = rv_wave_sum(dot);
        m = m_new;
        if (lane == 0) {
          float* g = gates + ((long long)(tb + c) * heads + h) * 3;
          g[0] = keep, g[1] = take, g[2] = fmaxf(fabsf(dot), expf(-m_new)) + 1e-6f;
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < PER; ++e)
    if (e * RV_WAVE + lane < dk) n_mem[e * RV_WAVE + lane] = n[e];
  if (lane == 0) slot[m_off + h] = m;
}

#define RG_GATES_PER_MAX 16

extern "C" int rv_memory_gates(hipStream_t stream, const void* rows, int dtype, long long ld, int q_col, int k_col,
                               int i_col, int f_col, const float* i_bias, const float* f_bias, float cap,
                               float q_scale, float* state, long long slot_stride, long long n_off, long long m_off,
                               const int* q_start, const int* state_slot, float* gates, int num_requests, int heads,
                               int dk) {
  RV_CHECK(rows && i_bias && f_bias && state && q_start && state_slot && gates, "memory_gates: null argument");
  RV_CHECK(heads > 0 && dk > 0 && num_requests >= 0 && cap > 0.f, "memory_gates: bad sizes heads=%d dk=%d", heads, dk);
  const int per = rv_div_up(dk, RV_WAVE);
  RV_CHECK(per <= RG_GATES_PER_MAX, "memory_gates: a key size of %d is more than %d", dk, RG_GATES_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(heads, num_requests), block(RV_WAVE);
#define RV_MG(T, PER, CHUNK)                                                                                          \
  memory_gates_kernel<T, PER, CHUNK><<<grid, block, 0, stream>>>((const T*)rows, ld, q_col, k_col, i_col, f_col, i_bias, \
                                                                 f_bias, cap, q_scale, state, slot_stride, n_off, m_off, \
                                                                 q_start, state_slot, gates, heads, dk)
#define RV_MG_T(T)                              \
  do {                                          \
    if (per <= 1) RV_MG(T, 1, 16);              \
    else if (per <= 2) RV_MG(T, 2, 16);         \
    else if (per <= 4) RV_MG(T, 4, 8);          \
    else if (per <= 8) RV_MG(T, 8, 4);          \
    else RV_MG(T, 16, 2);                       \
  } while (0)
  if (dtype == RV_F32) RV_MG_T(float);
  else if (dtype == RV_BF16) RV_MG_T(bf16_t);
  else return rv_fail("memory_gates: unsupported dtype %d", dtype);
#undef RV_MG_T
#undef RV_MG
  RV_LAUNCH_CHECK("memory_gates");
  return 0;
}

// ---------------------------------------------------------------------------
// memory_matrix.  A column j of a head's S (its dk numbers) never meets another column, so LANES neighbouring lanes
// own one: lane `sub` of them holds rows sub * PER .. + PER.  A wave holds 64 / LANES columns of one head of one
// request and walks the request's tokens of this step in order, CHUNK at a time through registers and LDS.
//   rows  T [tokens, ld]: q of head h at q_col + h dk, k at k_col + h dk, v at v_col + h dv
//   gates float [tokens, heads, 3]: keep, take, the divisor (memory_gates)
//   S     float [heads, dv, dk] at s_off of the request's slot (a column's dk numbers side by side)
//   out   float [tokens, heads dv]
// What a token's sums are does not depend on CHUNK: the same multiply-adds in the same order.
// ---------------------------------------------------------------------------
template <typename T, int PER, int LANES, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
memory_matrix_kernel(const T* __restrict__ rows, long long ld, int q_col, int k_col, int v_col, float q_scale,
                     const float* __restrict__ gates, float* __restrict__ state, long long slot_stride,
                     long long s_off, const int* __restrict__ q_start, const int* __restrict__ state_slot,
                     float* __restrict__ out, int heads, int dk, int dv) {
  constexpr int COLS = RV_WAVE / LANES;
  constexpr int DKP = PER * LANES;
  constexpr int NK = (CHUNK * DKP + RV_WAVE - 1) / RV_WAVE;
  constexpr int NV = (CHUNK * COLS + RV_WAVE - 1) / RV_WAVE;
  __shared__ __attribute__((aligned(16))) float sk[CHUNK][DKP];
  __shared__ __attribute__((aligned(16))) float sq[CHUNK][DKP];
  __shared__ float sv[CHUNK][COLS];
  __shared__ float sg[CHUNK][3];
  const int lane = threadIdx.x;
  const int sub = lane % LANES;
  const int cl = lane / LANES;
  const int j = blockIdx.x * COLS + cl;
  const int h = blockIdx.y;
  const int req = blockIdx.z;
  const bool col = j < dv;
  const int jj = col ? j : dv - 1;  // a lane past the last column works on a copy and writes nothing
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + ((long long)h * dv + jj) * dk + sub * PER;
  const bool vec = (dk % 4 == 0) && (((uintptr_t)S_mem & 15) == 0);
  float S[PER];
#pragma unroll
  for (int e = 0; e < PER; e += 4) {
    if (vec && sub * PER + e < dk) {
      const float4 v4 = *(const float4*)(S_mem + e);
      S[e] = v4.x, S[e + 1] = v4.y, S[e + 2] = v4.z, S[e + 3] = v4.w;
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) S[e + u] = sub * PER + e + u < dk ? S_mem[e + u] : 0.f;
    }
  }
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float rk[NK], rq[NK], rv[NV], rg = 0.f;
  auto fetch = [&](int tb) {
#pragma unroll
    for (int r = 0; r < NK; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / DKP, i = idx % DKP;
      const bool ok = tok < CHUNK && tb + tok < t1 && i < dk;
      const T* row = rows + (long long)(ok ? tb + tok : t0) * ld + (long long)h * dk + (ok ? i : 0);
      rk[r] = ok ? rv_to_float(row[k_col]) : 0.f;
      rq[r] = ok ? rv_to_float(row[q_col]) * q_scale : 0.f;
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / COLS, c = idx % COLS;
      const int jc = blockIdx.x * COLS + c;
      const bool ok = tok < CHUNK && tb + tok < t1 && jc < dv;
      rv[r] = ok ? rv_to_float(rows[(long long)(tb + tok) * ld + v_col + (long long)h * dv + jc]) : 0.f;
    }
    const int tok = lane / 3;
    if (lane < CHUNK * 3 && tb + tok < t1) rg = gates[((long long)(tb + tok) * heads + h) * 3 + lane % 3];
  };
  auto stage = [&]() {
#pragma unroll
    for (int r = 0; r < NK; ++r) {
      const int idx = r * RV_WAVE + lane;
      if (idx < CHUNK * DKP) (&sk[0][0])[idx] = rk[r], (&sq[0][0])[idx] = rq[r];
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int idx = r * RV_WAVE + lane;
      if (idx < CHUNK * COLS) (&sv[0][0])[idx] = rv[r];
    }
    if (lane < CHUNK * 3) (&sg[0][0])[lane] = rg;
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    __syncthreads();  // the chunk before has been read
    stage();
    __syncthreads();
    if (tb + CHUNK < t1) fetch(tb + CHUNK);
    const int n = min(CHUNK, t1 - tb);
    for (int t = 0; t < n; ++t) {
      float kk[PER], qq[PER];
#pragma unroll
      for (int e = 0; e < PER; e += 4) {
        const float4 k4 = *(const float4*)&sk[t][sub * PER + e];
        const float4 q4 = *(const float4*)&sq[t][sub * PER + e];
        kk[e] = k4.x, kk[e + 1] = k4.y, kk[e + 2] = k4.z, kk[e + 3] = k4.w;
        qq[e] = q4.x, qq[e + 1] = q4.y, qq[e + 2] = q4.z, qq[e + 3] = q4.w;
      }
      const float keep = sg[t][0];
      const float tv = sg[t][1] * sv[t][cl];
      float o = 0.f;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        S[e] = fmaf(tv, kk[e], keep * S[e]);
        o = fmaf(S[e], qq[e], o);
      }
      o = rg_group_sum<LANES>(o);
      if (col && sub == 0) out[(long long)(tb + t) * heads * dv + (long long)h * dv + j] = o / sg[t][2];
    }
  }
  if (col) {
#pragma unroll
    for (int e = 0; e < PER; e += 4) {
      if (vec && sub * PER + e < dk) {
        *(float4*)(S_mem + e) = make_float4(S[e], S[e + 1], S[e + 2], S[e + 3]);
      } else {
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (sub * PER + e + u < dk) S_mem[e + u] = S[e + u];
      }
    }
  }
}

#define RG_MATRIX_PER 8
#define RG_MATRIX_PER_MAX 16

// Lanes that share a column of S for this key size: a function of dk alone, so that a token's sums are added in
// one order always.
static int rg_matrix_lanes(int dk) {
  int lanes = 1;
  while (lanes < 16 && rv_div_up(dk, lanes) > RG_MATRIX_PER) lanes *= 2;
  while (lanes < RV_WAVE && rv_div_up(dk, lanes) > RG_MATRIX_PER_MAX) lanes *= 2;
  return lanes;
}

// `longest`: the most tokens a request brings in this step (the size of the chunks is chosen by it).
extern "C" int rv_memory_matrix(hipStream_t stream, const void* rows, int dtype, long long ld, int q_col, int k_col,
                                int v_col, float q_scale, const float* gates, float* state, long long slot_stride,
                                long long s_off, const int* q_start, const int* state_slot, float* out,
                                int num_requests, int heads, int dk, int dv, int longest) {
  RV_CHECK(rows && gates && state && q_start && state_slot && out, "memory_matrix: null argument");
  RV_CHECK(heads > 0 && dk > 0 && dv > 0 && num_requests >= 0, "memory_matrix: bad sizes heads=%d dk=%d dv=%d", heads,
           dk, dv);
  const int lanes = rg_matrix_lanes(dk);
  const int per = rv_div_up(dk, lanes);
  RV_CHECK(per <= RG_MATRIX_PER_MAX, "memory_matrix: a key size of %d is more than %d", dk, RG_MATRIX_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(dv, RV_WAVE / lanes), heads, num_requests), block(RV_WAVE);
  const bool few = longest <= 2;  // decoded tokens: small chunks, little LDS, more waves a CU
#define RV_MM(T, PER, LANES, CHUNK)                                                                               \
  memory_matrix_kernel<T, PER, LANES, CHUNK><<<grid, block, 0, stream>>>((const T*)rows, ld, q_col, k_col, v_col, \
                                                                         q_scale, gates, state, slot_stride, s_off, \
                                                                         q_start, state_slot, out, heads, dk, dv)
#define RV_MM_L(T, PER, LANES, CHUNK)          \
  do {                                         \
    if (few) RV_MM(T, PER, LANES, 2);          \
    else RV_MM(T, PER, LANES, CHUNK);          \
  } while (0)
#define RV_MM_T(T)                                           \
  do {                                                       \
    if (lanes == 1 && per <= 4) RV_MM_L(T, 4, 1, 16);        \
    else if (lanes == 1) RV_MM_L(T, 8, 1, 16);               \
    else if (lanes == 2) RV_MM_L(T, 8, 2, 16);               \
    else if (lanes == 4) RV_MM_L(T, 8, 4, 16);               \
    else if (lanes == 8) RV_MM_L(T, 8, 8, 16);               \
    else if (lanes == 16 && per <= 8) RV_MM_L(T, 8, 16, 16); \
    else if (lanes == 16) RV_MM_L(T, 16, 16, 8);             \
    else if (lanes == 32) RV_MM_L(T, 16, 32, 4);             \
    else RV_MM_L(T, 16, 64, 2);                              \
  } while (0)
  if (dtype == RV_F32) RV_MM_T(float);
  else if (dtype == RV_BF16) RV_MM_T(bf16_t);
  else return rv_fail("memory_matrix: unsupported dtype %d", dtype);
#undef RV_MM_T
#undef RV_MM_L
#undef RV_MM
  RV_LAUNCH_CHECK("memory_matrix");
  return 0;
}

// ---------------------------------------------------------------------------
// gated_linear_scan.  A lane a channel of a request; the tokens' operands come CHUNK at a time into registers, a
// chunk ahead of the one worked on.  1 - a^2 is taken as -expm1(2 log a), which keeps its digits where a is near 1.
//   u      T [tokens, ld_u]      the convolved input
//   gates  float [tokens, ld_g]  channel c = b * block + j: g_r at b * 2 block + j, g_i at b * 2 block + block + j
//                                (what a product by blocks against each block's two matrices, one after the other,
//                                leaves)
//   y      T [tokens, ld_y]      the other branch before its activation
//   S      float [channels] at s_off of the request's slot
//   out    T [tokens, channels] = S' * gelu_tanh(y), the activation rounded to T first
// ---------------------------------------------------------------------------
template <typename T, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
gated_linear_scan_kernel(const T* __restrict__ u, long long ld_u, const float* __restrict__ gates, long long ld_g,
                         int block_size, const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                         const float* __restrict__ lam, const T* __restrict__ y, long long ld_y,
                         float* __restrict__ state, long long slot_stride, long long s_off,
                         const int* __restrict__ q_start, const int* __restrict__ state_slot, T* __restrict__ out,
                         int channels) {
  const int ch = blockIdx.x * RV_WAVE + threadIdx.x;
  const int req = blockIdx.y;
  const bool live = ch < channels;
  const int c = live ? ch : channels - 1;
  const int b = c / block_size, jn = c - b * block_size;
  const long long g_r = (long long)b * 2 * block_size + jn, g_i = g_r + block_size;
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + c;
  float S = *S_mem;
  const float rate = -8.0f * rg_softplus(lam[c]);
  const float br = r_bias[c], bi = i_bias[c];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float nu[CHUNK], nr[CHUNK], ni[CHUNK], ny[CHUNK];
  auto fetch = [&](int tb) {
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) {
      const long long t = tb + k < t1 ? tb + k : t0;
      nu[k] = rv_to_float(u[t * ld_u + c]);
      nr[k] = gates[t * ld_g + g_r];
      ni[k] = gates[t * ld_g + g_i];
      ny[k] = rv_to_float(y[t * ld_y + c]);
    }
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    float a[CHUNK], x[CHUNK], gy[CHUNK];
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) {  // nothing here waits for S: the tokens' decays and inputs side by side
      const float log_a = rate * rg_sigmoid(nr[k] + br);
      a[k] = expf(log_a);
      x[k] = sqrtf(-expm1f(2.0f * log_a)) * rg_sigmoid(ni[k] + bi) * nu[k];
      gy[k] = rv_round_to<T>(rv_gated<float, 0>(ny[k], 1.0f));
    }
    if (tb + CHUNK < t1) fetch(tb + CHUNK);
    const int count = min(CHUNK, t1 - tb);
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) {
      if (k < count) {
        S = fmaf(a[k], S, x[k]);
        if (live) out[(long long)(tb + k) * channels + ch] = rv_from_float<T>(S * gy[k]);
      }
    }
  }
  if (live) *S_mem = S;
}

extern "C" int rv_gated_linear_scan(hipStream_t stream, const void* u, long long ld_u, const float* gates,
                                    long long ld_g, int block_size, const float* r_bias, const float* i_bias,
                                    const float* lam, const void* y, long long ld_y, float* state,
                                    long long slot_stride, long long s_off, const int* q_start, const int* state_slot,
                                    void* out, int dtype, int num_requests, int channels, int longest) {
  RV_CHECK(u && gates && r_bias && i_bias && lam && y && state && q_start && state_slot && out,
           "gated_linear_scan: null argument");
  RV_CHECK(channels > 0 && block_size > 0 && channels % block_size == 0 && num_requests >= 0 && ld_u >= channels &&
               ld_y >= channels && ld_g >= 2LL * channels,
           "gated_linear_scan: bad sizes channels=%d block=%d", channels, block_size);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(channels, RV_WAVE), num_requests), block(RV_WAVE);
  const bool few = longest <= 2;
#define RV_GS(T, CHUNK)                                                                                            \
  gated_linear_scan_kernel<T, CHUNK><<<grid, block, 0, stream>>>((const T*)u, ld_u, gates, ld_g, block_size, r_bias, \
                                                                 i_bias, lam, (const T*)y, ld_y, state, slot_stride, \
                                                                 s_off, q_start, state_slot, (T*)out, channels)
  if (dtype == RV_F32) { if (few) RV_GS(float, 1); else RV_GS(float, 8); }
  else if (dtype == RV_BF16) { if (few) RV_GS(bf16_t, 1); else RV_GS(bf16_t, 8); }
  else return rv_fail("gated_linear_scan: unsupported dtype %d", dtype);
#undef RV_GS
  RV_LAUNCH_CHECK("gated_linear_scan");
  return 0;
}
