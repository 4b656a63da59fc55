// Mixers that carry a state of fixed size from token to token instead of keys and values:
//
//   causal_conv        a short convolution over time for every channel, its activation, and optionally the
//                      scaling of groups of channels to unit length
//   conv_state_update  the last taps - 1 inputs of every channel, kept for the request's next step
//   delta_rule         the gated delta rule, a matrix S [dk, dv] a head:
//                        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   selective_scan     a diagonal state S [channel, n]:
//                        S <- exp(dt A) S + dt x B;  y = S . C + D x;  y <- y silu(z)
//   head_norm_gate     o / rms(o) * w * silu(gate), a head at a time
//   gate_mul           a * sigmoid(gate) or a * silu(gate), element by element
//
// The states, the decays, their exponentials and logarithms, the step sizes and the unit norms are 32-bit whatever
// the activations' type T; the convolution's sum is 32-bit and its activated output is rounded to T once.  A
// request's tokens are walked in their order by the waves that own a part of its state, so what a token's output
// is does not depend on how the request's tokens were cut into steps or on what else the step holds.  The state of
// a request lies in its slot, `slot_stride` floats apart from the next; a slot is all zeros when a request gets it.
#include "common.h"

#define REC_MAX_TAPS 16

__device__ __forceinline__ float rec_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float rec_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float rec_silu(float x) { return x / (1.0f + expf(-x)); }

// Sum over the LANES (a power of two) neighbouring lanes that share a column or channel; every one of them gets it.
// A token's work is one chain of dependent steps, and a wave often has its SIMD to itself, so the exchanges'
// latency counts: within 16 lanes they are DPP moves between registers (pairs, then pairs of pairs, then the two
// halves of 8 and of 16 mirrored, each half already holding its own sum in every lane), not trips through LDS.
template <int CTRL>
__device__ __forceinline__ float rec_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int LANES>
__device__ __forceinline__ float rec_group_sum(float v) {
  if constexpr (LANES >= 2) v += rec_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
  if constexpr (LANES >= 4) v += rec_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
  if constexpr (LANES >= 8) v += rec_dpp<0x141>(v);   // row_half_mirror
  if constexpr (LANES >= 16) v += rec_dpp<0x140>(v);  // row_mirror
  if constexpr (LANES >= 32) v += __shfl_xor(v, 16, RV_WAVE);
  if constexpr (LANES >= 64) v += __shfl_xor(v, 32, RV_WAVE);
  return v;
}

// The exponential of the scan's decay, once a state and token: the accurate one in a 32-bit engine; under bf16
// activations the hardware's (base two, an error of about 1e-6), as the other kernels' activations there.
template <typename T>
__device__ __forceinline__ float rec_decay_exp(float x);
template <>
__device__ __forceinline__ float rec_decay_exp<float>(float x) { return expf(x); }
template <>
__device__ __forceinline__ float rec_decay_exp<bf16_t>(float x) {
  return __builtin_amdgcn_exp2f(1.4426950408889634f * x);
}

// ---------------------------------------------------------------------------
// Short causal convolution.  Channel c of token t at position p:
//   y = act(bias[c] + sum_j w[c][j] * in[p - (taps - 1) + j][c]),   j = 0 .. taps - 1 (the last tap is the token's own)
// Inputs from before the step's first token of the request come from the state (its row s holds the input at
// position first - (taps - 1) + s); a fresh slot's zeros are the zeros before the start of a sequence.
// A wave takes a group of `group` channels of one token; with unit_eps >= 0 the group's outputs are divided by
// sqrt(sum y^2 + unit_eps) and the first `scaled_groups` groups multiplied by `group_scale`.
// `move_state`: every request of the step brings exactly one token (the host knows), so the lane that works on a
// channel is the only one that reads that channel's state rows, and moves them on itself (a row up, the token's
// input last) instead of leaving that to conv_state_update.
// ---------------------------------------------------------------------------
template <typename T, typename TO>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ in, long long ld_in, const float* __restrict__ w, const float* __restrict__ bias,
                   int taps, float* __restrict__ state, long long slot_stride, long long state_off,
                   int state_ld, const int* __restrict__ positions, const int* __restrict__ token_req,
                   const int* __restrict__ q_start, const int* __restrict__ chunk_start,
                   const int* __restrict__ state_slot, TO* __restrict__ out, long long ld_out, int channels, int group,
                   int groups, int num_tokens, float unit_eps, int scaled_groups, float group_scale, int move_state,
                   int act) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  if (unit >= (long long)num_tokens * groups) return;  // the whole wave
  const int t = (int)(unit / groups);
  const int grp = (int)(unit - (long long)t * groups);
  const int req = token_req[t];
  const int first_pos = chunk_start[req];
  const int first_tok = q_start[req];
  const int rel = positions[t] - first_pos;  // place of the token in its portion
  float* st = state + (long long)state_slot[req] * slot_stride + state_off;
  float ss = 0.f;
  for (int c0 = 0; c0 < group; c0 += RV_WAVE) {  // (two passes when the group is normed: the sum, then the store)
    const int c = grp * group + c0 + lane;
    if (c0 + lane < group && c < channels) {
      float acc = bias ? bias[c] : 0.f;
      for (int j = 0; j < taps; ++j) {
        const int r = rel - (taps - 1) + j;
        const float x = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c])
                               : st[(long long)(taps - 1 + r) * state_ld + c];
        acc = fmaf(w[(long long)c * taps + j], x, acc);
      }
      const float y = rv_round_to<T>(act == 0 ? rec_silu(acc) : acc);
      if (unit_eps < 0.f) {
        out[(long long)t * ld_out + c] = rv_from_float<TO>(y);
        if (move_state) {  // rel is 0: rows 1 .. taps - 2 move up, the token's input goes last
          for (int s_ = 0; s_ + 2 < taps; ++s_) st[(long long)s_ * state_ld + c] = st[(long long)(s_ + 1) * state_ld + c];
          if (taps > 1) st[(long long)(taps - 2) * state_ld + c] = rv_to_float(in[(long long)first_tok * ld_in + c]);
        }
      }
      ss = fmaf(y, y, ss);
    }
  }
  if (unit_eps < 0.f) return;
  ss = rv_wave_sum(ss);
  const float mult = (grp < scaled_groups ? group_scale : 1.0f) / sqrtf(ss + unit_eps);
  for (int c0 = 0; c0 < group; c0 += RV_WAVE) {
    const int c = grp * group + c0 + lane;
    if (c0 + lane < group && c < channels) {
      float acc = bias ? bias[c] : 0.f;
      for (int j = 0; j < taps; ++j) {
        const int r = rel - (taps - 1) + j;
        const float x = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c])
                               : st[(long long)(taps - 1 + r) * state_ld + c];
        acc = fmaf(w[(long long)c * taps + j], x, acc);
      }
      out[(long long)t * ld_out + c] = rv_from_float<TO>(rv_round_to<T>(act == 0 ? rec_silu(acc) : acc) * mult);
      if (move_state) {
        for (int s_ = 0; s_ + 2 < taps; ++s_) st[(long long)s_ * state_ld + c] = st[(long long)(s_ + 1) * state_ld + c];
        if (taps > 1) st[(long long)(taps - 2) * state_ld + c] = rv_to_float(in[(long long)first_tok * ld_in + c]);
      }
    }
  }
}

// in: [tokens, ld_in] of type `dtype`, the channels from the given address on.  w: float [channels, taps]; bias:
// float [channels] or null.  state: float, row s of a slot's block at state_off + s * state_ld.  out: float
// (out_f32) or `dtype`.  unit_eps < 0: no unit length.  act 0: silu, 1: none.
extern "C" int rv_causal_conv(hipStream_t stream, const void* in, int dtype, long long ld_in, const float* w,
                              const float* bias, int taps, float* state, long long slot_stride,
                              long long state_off, int state_ld, const int* positions, const int* token_req,
                              const int* q_start, const int* chunk_start, const int* state_slot, void* out,
                              int out_f32, long long ld_out, int channels, int group, int num_tokens, float unit_eps,
                              int scaled_groups, float group_scale, int move_state, int act) {
  RV_CHECK(in && w && state && positions && token_req && q_start && chunk_start && state_slot && out,
           "causal_conv: null argument");
  RV_CHECK(taps >= 1 && taps <= REC_MAX_TAPS && channels > 0 && group > 0 && num_tokens >= 0 && state_ld >= channels,
           "causal_conv: bad sizes taps=%d channels=%d group=%d", taps, channels, group);
  RV_CHECK(act == 0 || act == 1, "causal_conv: activation %d (0: silu, 1: none)", act);
  if (num_tokens == 0) return 0;
  const int groups = rv_div_up(channels, group);
  const long long units = (long long)num_tokens * groups;
  dim3 grid(rv_div_up(units, 4)), block(256);
#define RV_CC(T, TO)                                                                                                 \
  causal_conv_kernel<T, TO><<<grid, block, 0, stream>>>((const T*)in, ld_in, w, bias, taps, state, slot_stride,      \
                                                        state_off, state_ld, positions, token_req, q_start,          \
                                                        chunk_start, state_slot, (TO*)out, ld_out, channels, group,  \
                                                        groups, num_tokens, unit_eps, scaled_groups, group_scale,     \
                                                        move_state, act)
  if (dtype == RV_F32) RV_CC(float, float);
  else if (dtype == RV_BF16 && out_f32) RV_CC(bf16_t, float);
  else if (dtype == RV_BF16) RV_CC(bf16_t, bf16_t);
  else return rv_fail("causal_conv: unsupported dtype %d", dtype);
#undef RV_CC
  RV_LAUNCH_CHECK("causal_conv");
  return 0;
}

// After the step: row s of the state becomes the input at position end - (taps - 1) + s, taken from the step's
// tokens or, where the portion is shorter than taps - 1, from the rows the state held.  A thread owns a channel of
// a request and reads all it needs before it writes.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ in, long long ld_in, int taps, float* __restrict__ state,
                                         long long slot_stride, long long state_off, int state_ld,
                                         const int* __restrict__ q_start, const int* __restrict__ state_slot,
                                         int channels) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int req = blockIdx.y;
  if (c >= channels) return;
  const int first_tok = q_start[req];
  const int n = q_start[req + 1] - first_tok;
  float* st = state + (long long)state_slot[req] * slot_stride + state_off;
  float keep[REC_MAX_TAPS];
#pragma unroll
  for (int s = 0; s < REC_MAX_TAPS - 1; ++s) {
    if (s < taps - 1) {
      const int r = n - (taps - 1) + s;
      keep[s] = r >= 0 ? rv_to_float(in[(long long)(first_tok + r) * ld_in + c]) : st[(long long)(s + n) * state_ld + c];
    }
  }
#pragma unroll
  for (int s = 0; s < REC_MAX_TAPS - 1; ++s)
    if (s < taps - 1) st[(long long)s * state_ld + c] = keep[s];
}

extern "C" int rv_conv_state_update(hipStream_t stream, const void* in, int dtype, long long ld_in, int taps,
                                    float* state, long long slot_stride, long long state_off, int state_ld,
                                    const int* q_start, const int* state_slot, int channels, int num_requests) {
  RV_CHECK(in && state && q_start && state_slot, "conv_state_update: null argument");
  RV_CHECK(taps >= 1 && taps <= REC_MAX_TAPS && channels > 0 && state_ld >= channels && num_requests >= 0,
           "conv_state_update: bad sizes");
  if (num_requests == 0 || taps == 1) return 0;
  dim3 grid(rv_div_up(channels, 256), num_requests), block(256);
  if (dtype == RV_F32)
    conv_state_update_kernel<float><<<grid, block, 0, stream>>>((const float*)in, ld_in, taps, state, slot_stride,
                                                                state_off, state_ld, q_start, state_slot, channels);
  else if (dtype == RV_BF16)
    conv_state_update_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)in, ld_in, taps, state, slot_stride,
                                                                 state_off, state_ld, q_start, state_slot, channels);
  else
    return rv_fail("conv_state_update: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("conv_state_update");
  return 0;
}

// ---------------------------------------------------------------------------
// Gated delta rule.  A column j of a head's S (its dk numbers) never meets another column, so LANES neighbouring
// lanes own one: lane `sub` of them holds rows sub * PER .. + PER.  A wave holds 64 / LANES columns of one head of
// one request and walks the request's tokens of this step in order.  Going to memory for every token would cost a
// round trip a token (the walk is a chain), so the tokens' operands come CHUNK at a time: all lanes read the chunk's
// keys, queries, values and gate inputs side by side into registers while the chunk before is worked on, and put
// them into LDS once that is done; decay and beta are worked out there, once a token.
//   qkv  float [tokens, ld]: q of key head g at q_off + g dk, k at k_off + g dk, v of head h at v_off + h dv
//   ab   T [tokens, ld_ab]: the decay's input a at a_col + h, beta's input at b_col + h
//   g = exp(-exp(A_log[h]) softplus(a + dt_bias[h])),  beta = sigmoid(b)
//   S    float [heads, dv, dk] at s_off of the request's slot (a column's dk numbers side by side)
//   out  float [tokens, heads dv]
// What a token's sums are does not depend on CHUNK: the same multiply-adds in the same order.
// ---------------------------------------------------------------------------
template <typename T, int PER, int LANES, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
delta_rule_kernel(const float* __restrict__ qkv, long long ld, int q_off, int k_off, int v_off,
                  const T* __restrict__ ab, long long ld_ab, int a_col, int b_col, const float* __restrict__ A_log,
                  const float* __restrict__ dt_bias, float* __restrict__ state, long long slot_stride,
                  long long s_off, const int* __restrict__ q_start, const int* __restrict__ state_slot,
                  float* __restrict__ out, int heads, int kv_heads, int dk, int dv) {
  constexpr int COLS = RV_WAVE / LANES;
  constexpr int DKP = PER * LANES;                          // the key size, padded
  constexpr int NK = (CHUNK * DKP + RV_WAVE - 1) / RV_WAVE;  // keys (and queries) a lane brings in a chunk
  constexpr int NV = (CHUNK * COLS + RV_WAVE - 1) / RV_WAVE;
  __shared__ __attribute__((aligned(16))) float sk[CHUNK][DKP];
  __shared__ __attribute__((aligned(16))) float sq[CHUNK][DKP];
  __shared__ float sv[CHUNK][COLS];
  __shared__ float sdecay[CHUNK], sbeta[CHUNK];
  const int lane = threadIdx.x;
  const int sub = lane % LANES;
  const int cl = lane / LANES;
  const int j = blockIdx.x * COLS + cl;
  const int h = blockIdx.y;
  const int req = blockIdx.z;
  const int g = h / (heads / kv_heads);
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
  const float rate = -expf(A_log[h]);
  const float bias = dt_bias[h];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float rk[NK], rq[NK], rv[NV], ra = 0.f, rb = 0.f;
  auto fetch = [&](int tb) {  // the chunk from token tb on, into registers
#pragma unroll
    for (int r = 0; r < NK; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / DKP, i = idx % DKP;
      const bool ok = tok < CHUNK && tb + tok < t1 && i < dk;
      const float* row = qkv + (long long)(ok ? tb + tok : t0) * ld + g * dk + (ok ? i : 0);
      rk[r] = ok ? row[k_off] : 0.f;
      rq[r] = ok ? row[q_off] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < NV; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / COLS, c = idx % COLS;
      const int jc = blockIdx.x * COLS + c;
      const bool ok = tok < CHUNK && tb + tok < t1 && jc < dv;
      rv[r] = ok ? qkv[(long long)(tb + tok) * ld + v_off + h * dv + jc] : 0.f;
    }
    if (lane < CHUNK && tb + lane < t1) {
      ra = rv_to_float(ab[(long long)(tb + lane) * ld_ab + a_col + h]);
      rb = rv_to_float(ab[(long long)(tb + lane) * ld_ab + b_col + h]);
    }
  };
  auto stage = [&]() {  // the registers into LDS
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
    if (lane < CHUNK) {
      sdecay[lane] = expf(rate * rec_softplus(ra + bias));
      sbeta[lane] = rec_sigmoid(rb);
    }
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
      const float decay = sdecay[t];
      const float beta = sbeta[t];
      const float vv = sv[t][cl];
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        S[e] *= decay;
        dot = fmaf(S[e], kk[e], dot);
      }
      dot = rec_group_sum<LANES>(dot);
      const float u = beta * (vv - dot);
      float o = 0.f;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        S[e] = fmaf(kk[e], u, S[e]);
        o = fmaf(S[e], qq[e], o);
      }
      o = rec_group_sum<LANES>(o);
      if (col && sub == 0) out[(long long)(tb + t) * heads * dv + h * dv + j] = o;
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

#define REC_DELTA_PER 8       // rows of a column a lane holds, while up to 16 lanes share the column
#define REC_DELTA_PER_MAX 16  // ... and beyond

// How many lanes share a column of S for this key size: the fewest (a power of two) that leave a lane at most
// REC_DELTA_PER rows, up to 16 lanes (a prompt of one request then has a wave for every SIMD at the sizes in use,
// and the sums stay within a DPP row); larger keys take up to REC_DELTA_PER_MAX rows a lane.  A function of dk
// alone, so that a token's sums are added in one order always.
extern "C" int rv_delta_rule_lanes(int dk) {
  int lanes = 1;
  while (lanes < 16 && rv_div_up(dk, lanes) > REC_DELTA_PER) lanes *= 2;
  while (lanes < RV_WAVE && rv_div_up(dk, lanes) > REC_DELTA_PER_MAX) lanes *= 2;
  return lanes;
}

// `longest`: the most tokens a request brings in this step (the size of the chunks is chosen by it).
extern "C" int rv_delta_rule(hipStream_t stream, const float* qkv, long long ld, int q_off, int k_off, int v_off,
                             const void* ab, int dtype, long long ld_ab, int a_col, int b_col, const float* A_log,
                             const float* dt_bias, float* state, long long slot_stride, long long s_off,
                             const int* q_start, const int* state_slot, float* out, int num_requests, int heads,
                             int kv_heads, int dk, int dv, int longest) {
  RV_CHECK(qkv && ab && A_log && dt_bias && state && q_start && state_slot && out, "delta_rule: null argument");
  RV_CHECK(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dk > 0 && dv > 0 && num_requests >= 0,
           "delta_rule: bad sizes heads=%d kv_heads=%d dk=%d dv=%d", heads, kv_heads, dk, dv);
  const int lanes = rv_delta_rule_lanes(dk);
  const int per = rv_div_up(dk, lanes);
  RV_CHECK(per <= REC_DELTA_PER_MAX, "delta_rule: a key size of %d is more than %d", dk, REC_DELTA_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(dv, RV_WAVE / lanes), heads, num_requests), block(RV_WAVE);
  const bool few = longest <= 2;  // decoded tokens: small chunks, little LDS, more waves a CU
#define RV_DR(T, PER, LANES, CHUNK)                                                                             \
  delta_rule_kernel<T, PER, LANES, CHUNK><<<grid, block, 0, stream>>>(                                          \
      qkv, ld, q_off, k_off, v_off, (const T*)ab, ld_ab, a_col, b_col, A_log, dt_bias, state, slot_stride, s_off, \
      q_start, state_slot, out, heads, kv_heads, dk, dv)
  // chunks of up to 16 tokens while a chunk's keys stay within 2048 numbers (32 registers a lane)
#define RV_DR_L(T, PER, LANES, CHUNK)          \
  do {                                         \
    if (few) RV_DR(T, PER, LANES, 2);          \
    else RV_DR(T, PER, LANES, CHUNK);          \
  } while (0)
#define RV_DR_T(T)                                         \
  do {                                                     \
    if (lanes == 1 && per <= 4) RV_DR_L(T, 4, 1, 16);      \
    else if (lanes == 1) RV_DR_L(T, 8, 1, 16);             \
    else if (lanes == 2) RV_DR_L(T, 8, 2, 16);             \
    else if (lanes == 4) RV_DR_L(T, 8, 4, 16);             \
    else if (lanes == 8) RV_DR_L(T, 8, 8, 16);             \
    else if (lanes == 16 && per <= 8) RV_DR_L(T, 8, 16, 16); \
    else if (lanes == 16) RV_DR_L(T, 16, 16, 8);           \
    else if (lanes == 32) RV_DR_L(T, 16, 32, 4);           \
    else RV_DR_L(T, 16, 64, 2);                            \
  } while (0)
  if (dtype == RV_F32) RV_DR_T(float);
  else if (dtype == RV_BF16) RV_DR_T(bf16_t);
  else return rv_fail("delta_rule: unsupported dtype %d", dtype);
#undef RV_DR_T
#undef RV_DR_L
#undef RV_DR
  RV_LAUNCH_CHECK("delta_rule");
  return 0;
}

// ---------------------------------------------------------------------------
// Selective scan.  LANES neighbouring lanes own a channel: lane `sub` holds the states sub * PER .. + PER.  A wave
// holds 64 / LANES channels of one request and walks its tokens of this step in order, CHUNK at a time through
// registers and LDS as the delta rule above; the step sizes and the gates' silu are worked out once a token there.
// A channel's y is the sum of its states' products S C added as a balanced tree over the states in their order
// (inside a lane first, then between the lanes), so that it has the same bits however the states are dealt to
// lanes: a lane a state for prompts (a wave for every SIMD from one request), four states a lane for decoded
// tokens (a channel's states then lie in one 16-byte read, and a wave covers four times the channels).
//   x    T [tokens, ld_x]    the convolved, activated input      z   T [tokens, ld_z]   the gate's input
//   dt   T [tokens, ld_dt]   the step's projection; step = softplus(dt + dt_bias[c])
//   bc   T [tokens, ld_bc]   B at b_col, C at c_col, `n_state` each
//   A = -exp(A_log [channels, n_state]);  D [channels]
//   S    float [channels, n_state] at s_off of the request's slot
//   out  T [tokens, channels] = (S . C + D x) silu(z)
// ---------------------------------------------------------------------------
template <typename T, int PER, int LANES, int CHUNK>
__global__ void __launch_bounds__(RV_WAVE)
selective_scan_kernel(const T* __restrict__ x, long long ld_x, const T* __restrict__ z, long long ld_z,
                      const T* __restrict__ dt, long long ld_dt, const float* __restrict__ dt_bias,
                      const T* __restrict__ bc, long long ld_bc, int b_col, int c_col,
                      const float* __restrict__ A_log, const float* __restrict__ D, float* __restrict__ state,
                      long long slot_stride, long long s_off, const int* __restrict__ q_start,
                      const int* __restrict__ state_slot, T* __restrict__ out, int channels, int n_state) {
  // Products and sums stay the separate operations they are written as (fmaf where one rounding is meant): a
  // channel's tree of sums must have the same bits whether its products lie in one lane or in several.
#pragma clang fp contract(off)
  constexpr int CPW = RV_WAVE / LANES;  // channels a wave
  constexpr int NP = PER * LANES;       // the states, padded
  constexpr int NB = (CHUNK * NP + RV_WAVE - 1) / RV_WAVE;
  constexpr int NX = (CHUNK * CPW + RV_WAVE - 1) / RV_WAVE;
  __shared__ __attribute__((aligned(16))) float sB[CHUNK][NP];
  __shared__ __attribute__((aligned(16))) float sC[CHUNK][NP];
  __shared__ float sx[CHUNK][CPW], sg[CHUNK][CPW], sstep[CHUNK][CPW];
  const int lane = threadIdx.x;
  const int sub = lane % LANES;
  const int cl = lane / LANES;
  const int ch0 = blockIdx.x * CPW;
  const int ch = ch0 + cl;
  const int req = blockIdx.y;
  const bool live = ch < channels;
  const int c = live ? ch : channels - 1;
  float* S_mem = state + (long long)state_slot[req] * slot_stride + s_off + (long long)c * n_state + sub * PER;
  float S[PER], A[PER];
  const bool vec = PER == 4 && n_state % 4 == 0 && (((uintptr_t)S_mem & 15) == 0);
  if (vec && sub * PER < n_state) {
    const float4 v4 = *(const float4*)S_mem;
    S[0] = v4.x, S[1 % PER] = v4.y, S[2 % PER] = v4.z, S[3 % PER] = v4.w;
  } else {
#pragma unroll
    for (int e = 0; e < PER; ++e) S[e] = sub * PER + e < n_state ? S_mem[e] : 0.f;
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const int n = sub * PER + e;
    A[e] = n < n_state ? -expf(A_log[(long long)c * n_state + n]) : 0.f;
  }
  const float skip = D[c];
  const int t0 = q_start[req], t1 = q_start[req + 1];
  float rB[NB], rC[NB], rx[NX], rz[NX], rd[NX];
  auto fetch = [&](int tb) {
#pragma unroll
    for (int r = 0; r < NB; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / NP, n = idx % NP;
      const bool ok = tok < CHUNK && tb + tok < t1 && n < n_state;
      const T* row = bc + (long long)(ok ? tb + tok : t0) * ld_bc + (ok ? n : 0);
      rB[r] = ok ? rv_to_float(row[b_col]) : 0.f;
      rC[r] = ok ? rv_to_float(row[c_col]) : 0.f;
    }
#pragma unroll
    for (int r = 0; r < NX; ++r) {
      const int idx = r * RV_WAVE + lane;
      const int tok = idx / CPW, cc = ch0 + idx % CPW;
      const bool ok = tok < CHUNK && tb + tok < t1 && cc < channels;
      const long long t = ok ? tb + tok : t0;
      const int c_ = ok ? cc : 0;
      rx[r] = ok ? rv_to_float(x[t * ld_x + c_]) : 0.f;
      rz[r] = ok ? rv_to_float(z[t * ld_z + c_]) : 0.f;
      rd[r] = ok ? rv_to_float(dt[t * ld_dt + c_]) + dt_bias[c_] : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int r = 0; r < NB; ++r) {
      const int idx = r * RV_WAVE + lane;
      if (idx < CHUNK * NP) (&sB[0][0])[idx] = rB[r], (&sC[0][0])[idx] = rC[r];
    }
#pragma unroll
    for (int r = 0; r < NX; ++r) {
      const int idx = r * RV_WAVE + lane;
      if (idx < CHUNK * CPW) {
        (&sx[0][0])[idx] = rx[r];
        (&sg[0][0])[idx] = rec_silu(rz[r]);
        (&sstep[0][0])[idx] = rec_softplus(rd[r]);
      }
    }
  };
  if (t0 < t1) fetch(t0);
  for (int tb = t0; tb < t1; tb += CHUNK) {
    __syncthreads();
    stage();
    __syncthreads();
    if (tb + CHUNK < t1) fetch(tb + CHUNK);
    const int n_tok = min(CHUNK, t1 - tb);
    for (int t = 0; t < n_tok; ++t) {
      const float step = sstep[t][cl];
      const float xv = sx[t][cl];
      const float sx_ = step * xv;
      float prod[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        S[e] = fmaf(rec_decay_exp<T>(step * A[e]), S[e], sx_ * sB[t][sub * PER + e]);
        prod[e] = S[e] * sC[t][sub * PER + e];  // a product of its own (no contraction here): see the pragma above
      }
#pragma unroll
      for (int w = 1; w < PER; w *= 2)
#pragma unroll
        for (int e = 0; e + w < PER; e += 2 * w) prod[e] += prod[e + w];
      float y = rec_group_sum<LANES>(prod[0]);
      y = fmaf(skip, xv, y);
      if (live && sub == 0) out[(long long)(tb + t) * channels + ch] = rv_from_float<T>(y * sg[t][cl]);
    }
  }
  if (live) {
    if (vec && sub * PER < n_state) {
      *(float4*)S_mem = make_float4(S[0], S[1 % PER], S[2 % PER], S[3 % PER]);
    } else {
#pragma unroll
      for (int e = 0; e < PER; ++e)
        if (sub * PER + e < n_state) S_mem[e] = S[e];
    }
  }
}

#define REC_SCAN_PER_MAX 4

// Lanes that share a channel.  Prompts (`few` 0): one a state up to 64 (every state costs an exponential a token, and
// a prompt of one request wants a wave for every SIMD), then up to REC_SCAN_PER_MAX states a lane.  Steps of decoded
// tokens (`few` 1): REC_SCAN_PER_MAX states a lane.
extern "C" int rv_selective_scan_lanes(int n_state, int few) {
  int lanes = 1;
  if (few) {
    while (lanes < RV_WAVE && rv_div_up(n_state, lanes) > REC_SCAN_PER_MAX) lanes *= 2;
  } else {
    while (lanes < RV_WAVE && lanes < n_state) lanes *= 2;
  }
  return lanes;
}

extern "C" int rv_selective_scan(hipStream_t stream, const void* x, long long ld_x, const void* z, long long ld_z,
                                 const void* dt, long long ld_dt, const float* dt_bias, const void* bc,
                                 long long ld_bc, int b_col, int c_col, const float* A_log, const float* D,
                                 float* state, long long slot_stride, long long s_off, const int* q_start,
                                 const int* state_slot, void* out, int dtype, int num_requests, int channels,
                                 int n_state, int longest) {
  RV_CHECK(x && z && dt && dt_bias && bc && A_log && D && state && q_start && state_slot && out,
           "selective_scan: null argument");
  RV_CHECK(channels > 0 && n_state > 0 && num_requests >= 0, "selective_scan: bad sizes");
  const bool few = longest <= 2;
  const int lanes = rv_selective_scan_lanes(n_state, few);
  const int per = rv_div_up(n_state, lanes);
  RV_CHECK(per <= REC_SCAN_PER_MAX, "selective_scan: %d states a channel are more than %d", n_state,
           REC_SCAN_PER_MAX * RV_WAVE);
  if (num_requests == 0) return 0;
  dim3 grid(rv_div_up(channels, RV_WAVE / lanes), num_requests), block(RV_WAVE);
#define RV_SS(T, PER, LANES, CHUNK)                                                                                \
  selective_scan_kernel<T, PER, LANES, CHUNK><<<grid, block, 0, stream>>>(                                         \
      (const T*)x, ld_x, (const T*)z, ld_z, (const T*)dt, ld_dt, dt_bias, (const T*)bc, ld_bc, b_col, c_col, A_log, \
      D, state, slot_stride, s_off, q_start, state_slot, (T*)out, channels, n_state)
#define RV_SS_T(T)                                     \
  do {                                                 \
    if (few) {                                         \
      if (lanes == 1) RV_SS(T, 4, 1, 2);               \
      else if (lanes == 2) RV_SS(T, 4, 2, 2);          \
      else if (lanes == 4) RV_SS(T, 4, 4, 2);          \
      else if (lanes == 8) RV_SS(T, 4, 8, 2);          \
      else if (lanes == 16) RV_SS(T, 4, 16, 2);        \
      else if (lanes == 32) RV_SS(T, 4, 32, 2);        \
      else RV_SS(T, 4, 64, 2);                         \
    } else if (lanes == 1) RV_SS(T, 1, 1, 16);         \
    else if (lanes == 2) RV_SS(T, 1, 2, 16);           \
    else if (lanes == 4) RV_SS(T, 1, 4, 16);           \
    else if (lanes == 8) RV_SS(T, 1, 8, 16);           \
    else if (lanes == 16) RV_SS(T, 1, 16, 16);         \
    else if (lanes == 32) RV_SS(T, 1, 32, 16);         \
    else if (per <= 1) RV_SS(T, 1, 64, 16);            \
    else if (per <= 2) RV_SS(T, 2, 64, 8);             \
    else RV_SS(T, 4, 64, 4);                           \
  } while (0)
  if (dtype == RV_F32) RV_SS_T(float);
  else if (dtype == RV_BF16) RV_SS_T(bf16_t);
  else return rv_fail("selective_scan: unsupported dtype %d", dtype);
#undef RV_SS_T
#undef RV_SS
  RV_LAUNCH_CHECK("selective_scan");
  return 0;
}

// ---------------------------------------------------------------------------
// out[t][h][:] = o[t][h][:] / sqrt(mean(o[t][h][:]^2) + eps) * w[:] * act(gate[t][h][:]); a wave a (token, head).
// o: float [tokens, heads dv]; gate: T, rows ld_gate apart; w: float [dv], shared by the heads, or (w_per_head)
// [heads dv], every head its own; act 0: sigmoid, 1: silu; out: T.  With `dots` every head's o is first divided by
// max(|dots[t][h]|, floors[(t heads + h) floor_stride]) + 1e-6: the divisor of a matrix memory's read-out.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate, long long ld_gate,
                      const float* __restrict__ w, T* __restrict__ out, int heads, int dv, float eps, long long units,
                      int w_per_head, int act, const float* __restrict__ dots, const float* __restrict__ floors,
                      int floor_stride) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (blockDim.x / RV_WAVE) + threadIdx.x / RV_WAVE;
  if (unit >= units) return;
  const long long t = unit / heads;
  const int h = (int)(unit - t * heads);
  const float* row = o + unit * dv;
  const float den = dots ? fmaxf(fabsf(dots[unit]), floors[unit * floor_stride]) + 1e-6f : 1.0f;
  float ss = 0.f;
  for (int d = lane; d < dv; d += RV_WAVE) {
    const float x = dots ? row[d] / den : row[d];
    ss = fmaf(x, x, ss);
  }
  ss = rv_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int d = lane; d < dv; d += RV_WAVE) {
    const float gv = rv_to_float(gate[t * ld_gate + (long long)h * dv + d]);
    const float wv = w[w_per_head ? (long long)h * dv + d : d];
    const float x = dots ? row[d] / den : row[d];
    out[unit * dv + d] = rv_from_float<T>(x * inv * wv * (act == 0 ? rec_sigmoid(gv) : rec_silu(gv)));
  }
}

extern "C" int rv_head_norm_gate(hipStream_t stream, const float* o, const void* gate, long long ld_gate,
                                 const float* w, void* out, int dtype, int num_tokens, int heads, int dv, float eps,
                                 int w_per_head, int act, const float* dots, const float* floors, int floor_stride) {
  RV_CHECK(o && gate && w && out && heads > 0 && dv > 0 && num_tokens >= 0 && (act == 0 || act == 1),
           "head_norm_gate: bad arguments");
  RV_CHECK((dots == nullptr) == (floors == nullptr) && (dots == nullptr || floor_stride >= 1),
           "head_norm_gate: a divisor takes the dots and their floors");
  if (num_tokens == 0) return 0;
  const long long units = (long long)num_tokens * heads;
  dim3 grid(rv_div_up(units, 4)), block(256);
  if (dtype == RV_F32)
    head_norm_gate_kernel<float><<<grid, block, 0, stream>>>(o, (const float*)gate, ld_gate, w, (float*)out, heads, dv,
                                                             eps, units, w_per_head, act, dots, floors, floor_stride);
  else if (dtype == RV_BF16)
    head_norm_gate_kernel<bf16_t><<<grid, block, 0, stream>>>(o, (const bf16_t*)gate, ld_gate, w, (bf16_t*)out, heads,
                                                              dv, eps, units, w_per_head, act, dots, floors, floor_stride);
  else
    return rv_fail("head_norm_gate: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// ---------------------------------------------------------------------------
// a[t][c] *= act(gate[t][c]), in place; act 0: sigmoid, 1: silu.  gate's rows are ld_gate apart.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void gate_mul_kernel(T* __restrict__ a, const T* __restrict__ gate, long long ld_gate, int width,
                                long long total, int act) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / width;
  const float gv = rv_to_float(gate[t * ld_gate + (idx - t * width)]);
  const float m = act == 0 ? rec_sigmoid(gv) : rec_silu(gv);
  a[idx] = rv_from_float<T>(rv_to_float(a[idx]) * m);
}

extern "C" int rv_gate_mul(hipStream_t stream, void* a, const void* gate, long long ld_gate, int dtype, int rows,
                           int width, int act) {
  RV_CHECK(a && gate && rows >= 0 && width > 0 && ld_gate >= width && (act == 0 || act == 1), "gate_mul: bad arguments");
  if (rows == 0) return 0;
  const long long total = (long long)rows * width;
  dim3 grid(rv_div_up(total, 256)), block(256);
  if (dtype == RV_F32)
    gate_mul_kernel<float><<<grid, block, 0, stream>>>((float*)a, (const float*)gate, ld_gate, width, total, act);
  else if (dtype == RV_BF16)
    gate_mul_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)a, (const bf16_t*)gate, ld_gate, width, total, act);
  else
    return rv_fail("gate_mul: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("gate_mul");
  return 0;
}
