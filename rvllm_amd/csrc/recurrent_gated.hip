// Two more mixers that carry a state of fixed size from token to token:
//
//   matrix memory (the mLSTM of xLSTM), a head at a time, with log gates i and f and a running maximum m that
//   keeps the exponentials in range (m starts at 0):
//       m' = max(f + m, i);  keep = e^(f + m - m'),  take = e^(i - m')
//       S' = keep S + take k v^T;   n' = keep n + take k;   o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6)
//     memory_gates   walks m (a number a head) and leaves keep, take and e^(-m') of every token; the log gates
//                    come from capped inputs: i = cap tanh((a + b_i) / cap), f = logsigmoid(cap tanh((a' + b_f) / cap))
//     memory_matrix  walks S with these and reads it out; n is walked as one more column of S (a value of 1), whose
//                    read-out is n' . q; the division is left to the kernel that norms the heads
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
// memory_gates.  The running maximum is one number a head, walked token by token; everything else about a token's
// gates is worked out side by side.  A wave a (head, request), 64 tokens at a time: lane l works out the log gates
// of token l of the chunk, the maximum's walk (an add and a max a token) is done by all lanes alike with the
// tokens' log gates handed round, and lane l then takes the exponentials of its token.
//   rows   T [tokens, ld]: the gates' inputs of head h at i_col + h and f_col + h
//   m [heads] at m_off of the request's slot
//   gates  float [tokens, heads, 3]: keep = e^(f + m - m'), take = e^(i - m'), floor = e^(-m')
// ---------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(RV_WAVE)
memory_gates_kernel(const T* __restrict__ rows, long long ld, int i_col, int f_col, const float* __restrict__ i_bias,
                    const float* __restrict__ f_bias, float cap, float* __restrict__ state, long long slot_stride,
                    long long m_off, const int* __restrict__ q_start, const int* __restrict__ state_slot,
                    float* __restrict__ gates, int heads) {
  const int lane = threadIdx.x;
  const int h = blockIdx.x;
  const int req = blockIdx.y;
  float* m_mem = state + (long long)state_slot[req] * slot_stride + m_off + h;
  float m = *m_mem;
  const float bi = i_bias[h], bf = f_bias[h];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  for (int tb = t0; tb < t1; tb += RV_WAVE) {
    const int count = min(RV_WAVE, t1 - tb);
    const bool mine = lane < count;
    const T* row = rows + (long long)(mine ? tb + lane : t0) * ld + h;
    const float log_in = cap * tanhf((rv_to_float(row[i_col]) + bi) / cap);
    const float capped = cap * tanhf((rv_to_float(row[f_col]) + bf) / cap);
    const float log_forget = -rg_softplus(-capped);
    float m_before = 0.f, m_after = 0.f;
    for (int c = 0; c < count; ++c) {
      // token c's log gates from lane c: c is the same in every lane, so a read of that lane's register
      const float li = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, log_in), c));
      const float lf = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, log_forget), c));
      const float m_new = fmaxf(lf + m, li);
      if (lane == c) m_before = m, m_after = m_new;
      m = m_new;
    }
    if (mine) {
      float* g = gates + ((long long)(tb + lane) * heads + h) * 3;
      g[0] = expf(log_forget + m_before - m_after);
      g[1] = expf(log_in - m_after);
      g[2] = expf(-m_after);
    }
  }
  if (lane == 0) *m_mem = m;
}

extern "C" int rv_memory_gates(hipStream_t stream, const void* rows, int dtype, long long ld, int i_col, int f_col,
                               const float* i_bias, const float* f_bias, float cap, float* state,
                               long long slot_stride, long long m_off, const int* q_start, const int* state_slot,
                               float* gates, int num_requests, int heads) {
  RV_CHECK(rows && i_bias && f_bias && state && q_start && state_slot && gates, "memory_gates: null argument");
  RV_CHECK(heads > 0 && num_requests >= 0 && cap > 0.f, "memory_gates: bad sizes heads=%d", heads);
  if (num_requests == 0) return 0;
  dim3 grid(heads, num_requests), block(RV_WAVE);
  if (dtype == RV_F32)
    memory_gates_kernel<float><<<grid, block, 0, stream>>>((const float*)rows, ld, i_col, f_col, i_bias, f_bias, cap,
                                                           state, slot_stride, m_off, q_start, state_slot, gates, heads);
  else if (dtype == RV_BF16)
    memory_gates_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)rows, ld, i_col, f_col, i_bias, f_bias, cap,
                                                            state, slot_stride, m_off, q_start, state_slot, gates, heads);
  else
    return rv_fail("memory_gates: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("memory_gates");
  return 0;
}

// ---------------------------------------------------------------------------
// memory_matrix.  A column j of a head's S (its dk numbers) never meets another column, so LANES neighbouring lanes
// own one: lane `sub` of them holds rows sub * PER .. + PER.  A wave holds 64 / LANES columns of one head of one
// request and walks the request's tokens of this step in order, CHUNK at a time through registers and LDS.
// Column dv is n: its value is 1 for every token, it lives at n_off, and its read-out goes to `dots`.
//   rows  T [tokens, ld]: q of head h at q_col + h dk, k at k_col + h dk, v at v_col + h dv
//   gates float [tokens, heads, 3]: keep, take, e^(-m') (memory_gates)
//   S     float [heads, dv, dk] at s_off of the request's slot (a column's dk numbers side by side)
//   n     float [heads, dk] at n_off
//   out   float [tokens, heads dv] = S'^T q, not yet divided;  dots float [tokens, heads] = n' . q
// What a token's sums are does not depend on CHUNK: the same multiply-adds in the same order.
// ---------------------------------------------------------------------------
template <typename T, int PER, int LANES, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
memory_matrix_kernel(const T* __restrict__ rows, long long ld, int q_col, int k_col, int v_col, float q_scale,
                     const float* __restrict__ gates, float* __restrict__ state, long long slot_stride,
                     long long s_off, long long n_off, const int* __restrict__ q_start,
                     const int* __restrict__ state_slot, float* __restrict__ out, float* __restrict__ dots, int heads,
                     int dk, int dv) {
  constexpr int COLS = RV_WAVE / LANES;
  constexpr int DKP = PER * LANES;
  constexpr int NK = (CHUNK * DKP + RV_WAVE - 1) / RV_WAVE;
  constexpr int NV = (CHUNK * COLS + RV_WAVE - 1) / RV_WAVE;
  __shared__ __attribute__((aligned(16))) float sk[CHUNK][DKP];
  __shared__ __attribute__((aligned(16))) float sq[CHUNK][DKP];
  __shared__ float sv[CHUNK][COLS];
  __shared__ float sg[CHUNK][2];
  const int lane = threadIdx.x;
  const int sub = lane % LANES;
  const int cl = lane / LANES;
  const int j = blockIdx.x * COLS + cl;
  const int h = blockIdx.y;
  const int req = blockIdx.z;
  const bool col = j <= dv;
  const bool is_n = j == dv;
  const int jj = j < dv ? j : dv - 1;  // a lane past the last column works on a copy and writes nothing
  float* slot = state + (long long)state_slot[req] * slot_stride;
  float* S_mem = (is_n ? slot + n_off + (long long)h * dk : slot + s_off + ((long long)h * dv + jj) * dk) + sub * PER;
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
  float* dst = is_n ? dots + h : out + (long long)h * dv + jj;  // where a token's read-out goes, rows dst_stride apart
  const long long dst_stride = is_n ? heads : (long long)heads * dv;
  const int t0 = q_start[req], t1 = q_start[req + 1];
  // A chunk's operands as they lie in memory, read without a condition from addresses that exist (a token past the
  // request's end reads the first one's, a dimension past dk the first), so that no read waits for the one before;
  // they become numbers, with zeros where nothing is, when they go into LDS.
  T rk[NK], rq[NK], rv[NV];
  float rg = 0.f;
  auto fetch = [&](int tb) {
#pragma unroll
    for (int r = 0; r < NK; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / DKP, i = idx % DKP;
      const bool ok = tok < CHUNK && tb + tok < t1 && i < dk;
      const T* row = rows + (long long)(ok ? tb + tok : t0) * ld + (long long)h * dk + (ok ? i : 0);
      rk[r] = row[k_col];
      rq[r] = row[q_col];
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / COLS, c = idx % COLS;
      const int jc = blockIdx.x * COLS + c;
      const bool ok = tok < CHUNK && tb + tok < t1 && jc < dv;
      rv[r] = rows[(long long)(ok ? tb + tok : t0) * ld + v_col + (long long)h * dv + (ok ? jc : 0)];
    }
    const int tok = lane / 2;
    const bool ok = lane < CHUNK * 2 && tb + tok < t1;
    rg = gates[((long long)(ok ? tb + tok : t0) * heads + h) * 3 + lane % 2];
  };
  auto stage = [&](int tb) {  // what fetch(tb) brought
#pragma unroll
    for (int r = 0; r < NK; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / DKP, i = idx % DKP;
      const bool ok = tok < CHUNK && tb + tok < t1 && i < dk;
      if (idx < CHUNK * DKP) {
        (&sk[0][0])[idx] = ok ? rv_to_float(rk[r]) : 0.f;
        (&sq[0][0])[idx] = ok ? rv_to_float(rq[r]) * q_scale : 0.f;
      }
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / COLS, c = idx % COLS;
      const int jc = blockIdx.x * COLS + c;
      const bool ok = tok < CHUNK && tb + tok < t1 && jc < dv;
      if (idx < CHUNK * COLS) (&sv[0][0])[idx] = ok ? rv_to_float(rv[r]) : (jc == dv ? 1.0f : 0.f);
    }
    if (lane < CHUNK * 2) (&sg[0][0])[lane] = rg;
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    __syncthreads();  // the chunk before has been read
    stage(tb);
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
      if (col && sub == 0) dst[(long long)(tb + t) * dst_stride] = o;
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
                                long long s_off, long long n_off, const int* q_start, const int* state_slot,
                                float* out, float* dots, int num_requests, int heads, int dk, int dv, int longest) {
  RV_CHECK(rows && gates && state && q_start && state_slot && out && dots, "memory_matrix: null argument");
  RV_CHECK(heads > 0 && dk > 0 && dv > 0 && num_requests >= 0, "memory_matrix: bad sizes heads=%d dk=%d dv=%d", heads,
           dk, dv);
  const int lanes = rg_matrix_lanes(dk);
  const int per = rv_div_up(dk, lanes);
  RV_CHECK(per <= RG_MATRIX_PER_MAX, "memory_matrix: a key size of %d is more than %d", dk, RG_MATRIX_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(dv + 1, RV_WAVE / lanes), heads, num_requests), block(RV_WAVE);  // the values' columns and n
  const bool few = longest <= 2;  // decoded tokens: small chunks, little LDS, more waves a CU
#define RV_MM(T, PER, LANES, CHUNK)                                                                               \
  memory_matrix_kernel<T, PER, LANES, CHUNK><<<grid, block, 0, stream>>>((const T*)rows, ld, q_col, k_col, v_col, \
                                                                         q_scale, gates, state, slot_stride, s_off, \
                                                                         n_off, q_start, state_slot, out, dots, heads, \
                                                                         dk, dv)
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
// gated_linear_scan.  A lane a channel of a request.  1 - a^2 is taken as -expm1(2 log a), which keeps its digits
// where a is near 1.  What a token brings to the walk (its decay a, its input x = sqrt(1 - a^2) i u and the other
// branch's activation) does not wait for S, only S' = a S + x does:
//   few tokens a request (decoding): one kernel, a token's terms worked out where it is walked;
//   many (prompts): the terms of all tokens and channels side by side by one launch (gated_linear_terms), then the
//   walk alone, CHUNK tokens' terms in registers a chunk ahead: three reads, a multiply-add and a product a token.
// Both ways a token's terms come from the same function and its S from the same chain of multiply-adds.
//   u      T [tokens, ld_u]      the convolved input
//   gates  float [tokens, ld_g]  channel c = b * block + j: g_r at b * 2 block + j, g_i at b * 2 block + block + j
//                                (what a product by blocks against each block's two matrices, one after the other,
//                                leaves)
//   y      T [tokens, ld_y]      the other branch before its activation
//   S      float [channels] at s_off of the request's slot
//   out    T [tokens, channels] = S' * gelu_tanh(y), the activation rounded to T first
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void rg_unit_terms(float u, float g_r, float g_i, float y, float rate, float br, float bi,
                                              float& a, float& x, float& gy) {
  const float log_a = rate * rg_sigmoid(g_r + br);
  a = expf(log_a);
  x = sqrtf(-expm1f(2.0f * log_a)) * rg_sigmoid(g_i + bi) * u;
  gy = rv_round_to<T>(rv_gated<float, 0>(y, 1.0f));
}

template <typename T>
__global__ void __launch_bounds__(RV_WAVE)
gated_linear_scan_kernel(const T* __restrict__ u, long long ld_u, const float* __restrict__ gates, long long ld_g,
                         int block_size, const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                         const float* __restrict__ lam, const T* __restrict__ y, long long ld_y,
                         float* __restrict__ state, long long slot_stride, long long s_off,
                         const int* __restrict__ q_start, const int* __restrict__ state_slot, T* __restrict__ out,
                         int channels) {
  const int ch = blockIdx.x * RV_WAVE + threadIdx.x;
  const int req = blockIdx.y;
  if (ch >= channels) return;
  const int b = ch / block_size, jn = ch - b * block_size;
  const long long g_r = (long long)b * 2 * block_size + jn, g_i = g_r + block_size;
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + ch;
  float S = *S_mem;
  const float rate = -8.0f * rg_softplus(lam[ch]);
  const float br = r_bias[ch], bi = i_bias[ch];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  for (long long t = t0; t < t1; ++t) {
    float a, x, gy;
    rg_unit_terms<T>(rv_to_float(u[t * ld_u + ch]), gates[t * ld_g + g_r], gates[t * ld_g + g_i],
                     rv_to_float(y[t * ld_y + ch]), rate, br, bi, a, x, gy);
    S = fmaf(a, S, x);
    out[t * channels + ch] = rv_from_float<T>(S * gy);
  }
  *S_mem = S;
}

// terms: float [2, tokens, channels] (a, then x); act: T [tokens, channels]
template <typename T>
__global__ void __launch_bounds__(256)
gated_linear_terms_kernel(const T* __restrict__ u, long long ld_u, const float* __restrict__ gates, long long ld_g,
                          int block_size, const float* __restrict__ r_bias, const float* __restrict__ i_bias,
                          const float* __restrict__ lam, const T* __restrict__ y, long long ld_y,
                          float* __restrict__ terms, T* __restrict__ act, int num_tokens, int channels) {
  const int ch = blockIdx.x * 256 + threadIdx.x;
  const long long t = blockIdx.y;
  if (ch >= channels) return;
  const int b = ch / block_size, jn = ch - b * block_size;
  const long long g_r = (long long)b * 2 * block_size + jn, g_i = g_r + block_size;
  const float rate = -8.0f * rg_softplus(lam[ch]);
  float a, x, gy;
  rg_unit_terms<T>(rv_to_float(u[t * ld_u + ch]), gates[t * ld_g + g_r], gates[t * ld_g + g_i],
                   rv_to_float(y[t * ld_y + ch]), rate, r_bias[ch], i_bias[ch], a, x, gy);
  terms[t * channels + ch] = a;
  terms[((long long)num_tokens + t) * channels + ch] = x;
  act[t * channels + ch] = rv_from_float<T>(gy);
}

template <typename T, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
gated_linear_walk_kernel(const float* __restrict__ terms, const T* __restrict__ act, float* __restrict__ state,
                         long long slot_stride, long long s_off, const int* __restrict__ q_start,
                         const int* __restrict__ state_slot, T* __restrict__ out, int num_tokens, int channels) {
  const int ch = blockIdx.x * RV_WAVE + threadIdx.x;
  const int req = blockIdx.y;
  if (ch >= channels) return;
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + ch;
  float S = *S_mem;
  const float* ta = terms + ch;
  const float* tx = terms + (long long)num_tokens * channels + ch;
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float na[CHUNK], nx[CHUNK], ng[CHUNK];
  auto fetch = [&](int tb) {
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) {
      const long long t = tb + k < t1 ? tb + k : t0;
      na[k] = ta[t * channels];
      nx[k] = tx[t * channels];
      ng[k] = rv_to_float(act[t * channels + ch]);
    }
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    float a[CHUNK], x[CHUNK], gy[CHUNK];
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) a[k] = na[k], x[k] = nx[k], gy[k] = ng[k];
    if (tb + CHUNK < t1) fetch(tb + CHUNK);
    const int count = min(CHUNK, t1 - tb);
#pragma unroll
    for (int k = 0; k < CHUNK; ++k) {
      if (k < count) {
        S = fmaf(a[k], S, x[k]);
        out[(long long)(tb + k) * channels + ch] = rv_from_float<T>(S * gy[k]);
      }
    }
  }
  *S_mem = S;
}

// `terms` (float [2, tokens, channels]) and `act` (of `dtype`, [tokens, channels]) are scratch for the two-launch
// form; null: the one-launch form.
extern "C" int rv_gated_linear_scan(hipStream_t stream, const void* u, long long ld_u, const float* gates,
                                    long long ld_g, int block_size, const float* r_bias, const float* i_bias,
                                    const float* lam, const void* y, long long ld_y, float* state,
                                    long long slot_stride, long long s_off, const int* q_start, const int* state_slot,
                                    void* out, int dtype, int num_requests, int num_tokens, int channels, float* terms,
                                    void* act) {
  RV_CHECK(u && gates && r_bias && i_bias && lam && y && state && q_start && state_slot && out,
           "gated_linear_scan: null argument");
  RV_CHECK(channels > 0 && block_size > 0 && channels % block_size == 0 && num_requests >= 0 && num_tokens >= 0 &&
               ld_u >= channels && ld_y >= channels && ld_g >= 2LL * channels,
           "gated_linear_scan: bad sizes channels=%d block=%d", channels, block_size);
  RV_CHECK((terms == nullptr) == (act == nullptr), "gated_linear_scan: the scratch is both or neither");
  RV_CHECK(dtype == RV_F32 || dtype == RV_BF16, "gated_linear_scan: unsupported dtype %d", dtype);
  if (num_requests == 0 || num_tokens == 0) return 0;
  dim3 grid(rv_div_up(channels, RV_WAVE), num_requests), block(RV_WAVE);
#define RV_GS(T)                                                                                                     \
  do {                                                                                                               \
    if (terms == nullptr) {                                                                                          \
      gated_linear_scan_kernel<T><<<grid, block, 0, stream>>>((const T*)u, ld_u, gates, ld_g, block_size, r_bias,    \
                                                              i_bias, lam, (const T*)y, ld_y, state, slot_stride,    \
                                                              s_off, q_start, state_slot, (T*)out, channels);        \
    } else {                                                                                                         \
      RV_CHECK(num_tokens < 65536, "gated_linear_scan: %d tokens are too many for one launch", num_tokens);          \
      gated_linear_terms_kernel<T><<<dim3(rv_div_up(channels, 256), num_tokens), dim3(256), 0, stream>>>(            \
          (const T*)u, ld_u, gates, ld_g, block_size, r_bias, i_bias, lam, (const T*)y, ld_y, terms, (T*)act,        \
          num_tokens, channels);                                                                                     \
      gated_linear_walk_kernel<T, 16><<<grid, block, 0, stream>>>(terms, (const T*)act, state, slot_stride, s_off,   \
                                                                  q_start, state_slot, (T*)out, num_tokens,          \
                                                                  channels);                                         \
    }                                                                                                                \
  } while (0)
  if (dtype == RV_F32) RV_GS(float);
  else RV_GS(bf16_t);
#undef RV_GS
  RV_LAUNCH_CHECK("gated_linear_scan");
  return 0;
}
