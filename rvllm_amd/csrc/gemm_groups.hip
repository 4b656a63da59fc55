// Many small products in one launch, C_g = A_g * W_g^T, with 32-bit multiply-adds: the products of a group of
// attention heads (one matrix a head, the heads' inputs and outputs side by side in a row) and of a set of experts
// (one matrix an expert, rows sorted by expert).
//
//   heads    group g = blockIdx.z;  A_g = a + g * a_group_stride (its columns inside a row of lda),
//            W_g = w + g * w_group_stride, C_g = c + g * c_group_stride
//   experts  tile_group[blockIdx.y] names the group of a tile of 64 rows (-1: the tile holds no rows and the block
//            does nothing); a_group_stride and c_group_stride are 0; with `row_index` row r of A is row
//            row_index[r] of a (-1: a row of zeros), so the sorted rows need not be copied together first
//
// With `gate`, C = (A W^T) * sigmoid(gate), gate laid out like C (ldg).  Every output is one chain of fused
// multiply-adds over k in order, as in gemm_plain: it does not depend on where its row lies or on the other rows.
#include "common.h"

#define GG_BM 64
#define GG_BN 64
#define GG_BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_groups_plain_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TC* __restrict__ c,
                         const int* __restrict__ row_index, const int* __restrict__ tile_group, int M, int N, int K,
                         long long lda, long long ldw, long long ldc, long long a_group_stride,
                         long long w_group_stride, long long c_group_stride, const TC* __restrict__ gate,
                         long long ldg) {
  __shared__ float a_s[GG_BK][GG_BM + 4];
  __shared__ float w_s[GG_BK][GG_BN + 4];
  const int group = tile_group ? tile_group[blockIdx.y] : (int)blockIdx.z;
  if (group < 0) return;  // the whole block alike
  a += (size_t)group * a_group_stride;
  w += (size_t)group * w_group_stride;
  c += (size_t)group * c_group_stride;
  if (gate) gate += (size_t)group * c_group_stride;
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GG_BM, n0 = blockIdx.x * GG_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const int lr = tid / 4, lk = (tid % 4) * 4;
  const int am = m0 + lr;
  long long a_row = -1;
  if (am < M) a_row = row_index ? row_index[am] : am;
  const int wn = n0 + lr;
  for (int k0 = 0; k0 < K; k0 += GG_BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      a_s[lk + e][lr] = (a_row >= 0 && k < K) ? rv_to_float(a[(size_t)a_row * lda + k]) : 0.f;
      w_s[lk + e][lr] = (wn < N && k < K) ? rv_to_float(w[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w_s[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (gate) v *= 1.0f / (1.0f + expf(-rv_to_float(gate[(size_t)m * ldg + n])));
      c[(size_t)m * ldc + n] = rv_from_float<TC>(v);
    }
  }
}

// groups > 0: the heads' form (tile_group and row_index null).  groups == 0: the experts' form; tile_group holds
// ceil(M / 64) entries, row_index (or null) M.
extern "C" int rv_gemm_groups_plain(hipStream_t stream, const void* a, int a_dtype, const void* w, int w_dtype, void* c,
                                    int c_dtype, const int* row_index, const int* tile_group, int groups, int M, int N,
                                    int K, long long lda, long long ldw, long long ldc, long long a_group_stride,
                                    long long w_group_stride, long long c_group_stride, const void* gate,
                                    long long ldg) {
  RV_CHECK(M >= 0 && N > 0 && K > 0 && groups >= 0, "gemm_groups: bad sizes M=%d N=%d K=%d groups=%d", M, N, K, groups);
  RV_CHECK((groups > 0) == (tile_group == nullptr), "gemm_groups: either a number of groups or the groups of the row tiles");
  RV_CHECK(ldw >= K && ldc >= N && lda >= K, "gemm_groups: leading dimensions too small");
  RV_CHECK(gate == nullptr || ldg >= N, "gemm_groups: the gate's rows are too short");
  if (M == 0) return 0;
  dim3 grid(rv_div_up(N, GG_BN), rv_div_up(M, GG_BM), groups > 0 ? groups : 1), block(256);
  RV_CHECK(grid.y < 65536 && grid.z < 65536, "gemm_groups: too many row tiles or groups for one launch");
#define RV_GG(TA, TW, TC)                                                                                          \
  gemm_groups_plain_kernel<TA, TW, TC><<<grid, block, 0, stream>>>(                                                \
      (const TA*)a, (const TW*)w, (TC*)c, row_index, tile_group, M, N, K, lda, ldw, ldc, a_group_stride,           \
      w_group_stride, c_group_stride, (const TC*)gate, ldg)
  if (a_dtype == RV_F32 && w_dtype == RV_F32 && c_dtype == RV_F32) RV_GG(float, float, float);
  else if (a_dtype == RV_BF16 && w_dtype == RV_BF16 && c_dtype == RV_BF16) RV_GG(bf16_t, bf16_t, bf16_t);
  else if (a_dtype == RV_BF16 && w_dtype == RV_BF16 && c_dtype == RV_F32 && gate == nullptr)
    RV_GG(bf16_t, bf16_t, float);  // 32-bit sums handed on unrounded
  else return rv_fail("gemm_groups: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
#undef RV_GG
  RV_LAUNCH_CHECK("gemm_groups_plain");
  return 0;
}

// ---------------------------------------------------------------------------
// The same products in bf16 on the matrix cores (MFMA 16x16x32), for both forms.  The product is taken
// transposed, C^T = W A^T, as in the few-row product: 16 rows of W are the A operand and 16 rows of a (tokens) the
// B operand, both read straight from memory in the order the instruction sums them (8 consecutive k a lane, 16
// bytes), so a lane ends up with 4 consecutive outputs of one token.  A wave takes 16 tokens against 1 or 4 tiles of
// 16 rows of W (the tokens' values are read once for all of them); the four waves of a block take neighbouring
// rows of W.  Tiles of rows are 16 here (tile_group has an entry for every 16 rows).  Sums are 32-bit.
//
// Epilogues: a gate (C * sigmoid(gate)); or, GLU, the clamped gated activation of an expert applied where the sums
// are held: W holds N gate rows and then N up rows, the wave multiplies both against the same tokens and writes
// g * sigmoid(alpha g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit) (glu 1), or the plain
// silu(gate) * up (glu 2: no limit, alpha 1, the up as it is): the expert's inner
// activations never exist unactivated in memory.
// ---------------------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 gg_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float gg_f32x4;
union GgFrag8 {
  gg_bf16x8 v;
  uint4 u4;
};

struct GroupsParams {
  const uint16_t* a;
  const uint16_t* w;
  uint16_t* c;
  const int* row_index;
  const int* tile_group;
  const uint16_t* gate;
  int M, N, K;
  long long lda, ldw, ldc, ldg, a_group_stride, w_group_stride, c_group_stride;
  float limit, alpha;
  float up_offset;  // what the clamped up is raised by: 1 in the clamped form, 0 in the plain one
  int vec_store;
  int c_f32;  // C holds 32-bit floats (the sums as they are) instead of bf16; strides count its elements
};

// A wave takes MT tiles of 16 tokens against NT tiles of 16 rows of W: every value it reads feeds MT or NT
// products.  Where the tokens are few (decoding) MT = NT = 1, so that a launch has every wave it can get to draw
// the memory's rate; where they are many (a prompt) MT = 4 and NT = 4 (2 gate and 2 up tiles with GLU), 16
// products for 8 reads, and the block's four waves share their tokens' values through the CU's cache.  A tile of
// rows (an entry of tile_group) is 16 MT rows.  The loop over k is written out UNROLL steps at a time with every
// read of the steps asked for before the first product, so that a wave has a dozen 16-byte reads in flight.
template <int MT, int NT, bool GLU>
__global__ void __launch_bounds__(256) gemm_groups_mfma_kernel(const GroupsParams P) {
  constexpr int UNROLL = (MT + NT * (GLU ? 2 : 1)) >= 5 ? 2 : 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  const int group = P.tile_group ? P.tile_group[blockIdx.y] : (int)blockIdx.z;
  if (group < 0) return;  // the whole block alike
  const int m0 = blockIdx.y * 16 * MT;
  const int n0 = (blockIdx.x * 4 + wave) * 16 * NT;
  if (n0 >= P.N) return;  // the whole wave
  const uint16_t* a = P.a + (size_t)group * P.a_group_stride;
  const uint16_t* w = P.w + (size_t)group * P.w_group_stride;
  const uint16_t* xr[MT];
  bool x_there[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int am = m0 + mt * 16 + r16;
    long long a_row = -1;
    if (am < P.M) a_row = P.row_index ? P.row_index[am] : am;
    x_there[mt] = a_row >= 0;
    xr[mt] = a + (size_t)(a_row >= 0 ? a_row : 0) * P.lda;
  }
  const uint16_t* wr[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int n = n0 + t * 16 + r16;
    n = n < P.N ? n : P.N - 1;  // rows past the end repeat the last one and are not stored
    wr[t] = w + (size_t)n * P.ldw;
  }
  const size_t up_rows = (size_t)P.N * P.ldw;  // GLU: the up rows follow the N gate rows
  gg_f32x4 acc[MT][NT], acc_up[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc[mt][t] = (gg_f32x4){0.f, 0.f, 0.f, 0.f};
      acc_up[mt][t] = (gg_f32x4){0.f, 0.f, 0.f, 0.f};
    }
  GgFrag8 xf[2][UNROLL][MT], wf[2][UNROLL][NT], uf[2][UNROLL][NT];
  auto ask = [&](int buf, int k0) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = k0 + u * 32 + kb * 8;
      const int kk = k < P.K ? k : 0;  // reads are unconditional, from an address that exists; what lies past K is zeroed
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xf[buf][u][mt].u4 = *(const uint4*)(xr[mt] + kk);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        wf[buf][u][t].u4 = *(const uint4*)(wr[t] + kk);
        if constexpr (GLU) uf[buf][u][t].u4 = *(const uint4*)(wr[t] + up_rows + kk);
      }
    }
  };
  auto multiply = [&](int buf, int k0) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const bool past = k0 + u * 32 + kb * 8 >= P.K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        if (past || !x_there[mt]) xf[buf][u][mt].u4 = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[buf][u][t].v, xf[buf][u][mt].v, acc[mt][t], 0, 0, 0);
          if constexpr (GLU)
            acc_up[mt][t] =
                __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[buf][u][t].v, xf[buf][u][mt].v, acc_up[mt][t], 0, 0, 0);
        }
      }
    }
  };
  constexpr int ROUND = 32 * UNROLL;
  if constexpr (MT == 1) {
    // few tokens: the next round's reads are asked for before this round's products, so that a wave waits for
    // memory once a round with a round's products to do meanwhile (gate and up of 16 tokens: 31 -> 28 us)
    ask(0, 0);
    for (int k0 = 0; k0 < P.K; k0 += 2 * ROUND) {  // written out for both buffers, so that no register is copied
      ask(1, k0 + ROUND < P.K ? k0 + ROUND : k0);  // past the end the last round is read again and not used
      multiply(0, k0);
      if (k0 + ROUND >= P.K) break;
      ask(0, k0 + 2 * ROUND < P.K ? k0 + 2 * ROUND : k0);
      multiply(1, k0 + ROUND);
    }
  } else {
    // many tokens: reading further ahead only crowds the caches (measured: 182 -> 218 us for 4 096 rows)
    for (int k0 = 0; k0 < P.K; k0 += ROUND) {
      ask(0, k0);
      multiply(0, k0);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int am = m0 + mt * 16 + r16;
    if (am >= P.M) continue;
    uint16_t* cr = P.c + (size_t)group * P.c_group_stride + (size_t)am * P.ldc;
    const uint16_t* gr = P.gate ? P.gate + (size_t)group * P.c_group_stride + (size_t)am * P.ldg : nullptr;
    if (P.c_f32) {  // no epilogue: the 32-bit sums go out unrounded
      float* cf = (float*)P.c + (size_t)group * P.c_group_stride + (size_t)am * P.ldc;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int n = n0 + t * 16 + kb * 4;
        if (P.vec_store && n + 3 < P.N) {
          *(float4*)(cf + n) = make_float4(acc[mt][t][0], acc[mt][t][1], acc[mt][t][2], acc[mt][t][3]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < P.N) cf[n + i] = acc[mt][t][i];
        }
      }
      continue;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = n0 + t * 16 + kb * 4;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[mt][t][i];
        if constexpr (GLU) {
          const float g = fminf(v[i], P.limit);
          const float u = fminf(fmaxf(acc_up[mt][t][i], -P.limit), P.limit);
          v[i] = g * (u + P.up_offset) * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * P.alpha * g));
        }
        if (gr != nullptr && n + i < P.N) {
          const float z = __uint_as_float(((uint32_t)gr[n + i]) << 16);
          v[i] *= __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
        }
      }
      if (P.vec_store && n + 3 < P.N) {
        uint2 packed;
        packed.x = rv_pack_bf16x2(v[0], v[1]);
        packed.y = rv_pack_bf16x2(v[2], v[3]);
        *(uint2*)(cr + n) = packed;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < P.N) cr[n + i] = rv_f32_to_bf16_bits(v[i]);
      }
    }
  }
}

// The experts' products of many rows, tiles staged through LDS.  A block of four waves takes a tile of 64 rows
// (one entry of tile_group) against 256 rows of its expert's matrix, 64 values of k at a time: the block copies
// both tiles from memory into LDS once (every row's 128 bytes as one run: eight lanes, 16 bytes each), and every
// wave multiplies all 64 rows against its 64 rows of the matrix from there, so a value that comes through the
// memory's caches once feeds four waves' products (read straight into registers, as the kernel above does it, the
// same product asks the CU's vector cache for 0.5 KB a product tile and keeps the matrix cores busy a tenth of the
// time).  The next 64 values of k are asked for before this round's products and written to LDS after them.
// Without GLU a wave's 64 rows of the matrix are 64 columns of C; with GLU they are 32 gate rows and their 32 up
// rows, and the activation is applied where both sums are held.  Rows of LDS are 16 bytes longer than their data,
// which spreads a fragment's sixteen rows over the banks.
#define GL_BM 64
#define GL_BW 256
#define GL_BK 64
#define GL_LD (GL_BK + 8)  // elements a row of LDS

template <bool GLU>
__global__ void __launch_bounds__(256) gemm_experts_lds_kernel(const GroupsParams P) {
  __shared__ __attribute__((aligned(16))) uint16_t xs[GL_BM * GL_LD];
  __shared__ __attribute__((aligned(16))) uint16_t ws[GL_BW * GL_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  const int group = P.tile_group[blockIdx.y];
  if (group < 0) return;  // the whole block alike, before any barrier
  constexpr int COLS = GLU ? GL_BW / 2 : GL_BW;  // columns of C a block takes
  const int m0 = blockIdx.y * GL_BM;
  const int n0 = blockIdx.x * COLS;
  const uint16_t* w = P.w + (size_t)group * P.w_group_stride;

  // what this thread copies each round: 2 pieces of 16 bytes of the rows' tile, 8 of the matrix's
  const int piece_k = (tid & 7) * 8;  // its place among a row's 64 values of k
  const uint16_t* x_src[2];
  bool x_there[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = (tid >> 3) + i * 32;
    const int am = m0 + row;
    long long a_row = -1;
    if (am < P.M) a_row = P.row_index ? P.row_index[am] : am;
    x_there[i] = a_row >= 0;
    x_src[i] = P.a + (size_t)(a_row >= 0 ? a_row : 0) * P.lda + piece_k;
  }
  const uint16_t* w_src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int row = (tid >> 3) + i * 32;  // of the block's 256 rows of the matrix
    int n;
    if constexpr (GLU) n = row < COLS ? n0 + row : P.N + n0 + (row - COLS);  // gate rows, then their up rows
    else n = n0 + row;
    const int last = GLU ? 2 * P.N - 1 : P.N - 1;
    n = n < last ? n : last;  // rows past the end repeat the last one; their columns are not stored
    w_src[i] = w + (size_t)n * P.ldw + piece_k;
  }
  uint4 x_reg[2], w_reg[8];
  auto ask = [&](int k0) {
    const bool in = k0 + piece_k < P.K;  // K is a multiple of 8: a piece lies inside or outside
    const int kk = in ? k0 : 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      x_reg[i] = *(const uint4*)(x_src[i] + kk);
      if (!in || !x_there[i]) x_reg[i] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      w_reg[i] = *(const uint4*)(w_src[i] + kk);
      if (!in) w_reg[i] = make_uint4(0, 0, 0, 0);
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i) *(uint4*)(xs + ((tid >> 3) + i * 32) * GL_LD + piece_k) = x_reg[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *(uint4*)(ws + ((tid >> 3) + i * 32) * GL_LD + piece_k) = w_reg[i];
  };

  gg_f32x4 acc[4][4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[mt][t] = (gg_f32x4){0.f, 0.f, 0.f, 0.f};
  // the wave's four tiles of 16 rows of the matrix, as rows of ws
  int w_row[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if constexpr (GLU) w_row[t] = (t < 2 ? 0 : COLS) + wave * 32 + (t & 1) * 16;
    else w_row[t] = wave * 64 + t * 16;
  }

  ask(0);
  put();
  __syncthreads();
  for (int k0 = 0; k0 < P.K; k0 += GL_BK) {
    const bool more = k0 + GL_BK < P.K;  // the same for the whole block
    if (more) ask(k0 + GL_BK);
#pragma unroll
    for (int ks = 0; ks < GL_BK / 32; ++ks) {
      GgFrag8 xf[4], wf[4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) xf[mt].u4 = *(const uint4*)(xs + (mt * 16 + r16) * GL_LD + ks * 32 + kb * 8);
#pragma unroll
      for (int t = 0; t < 4; ++t) wf[t].u4 = *(const uint4*)(ws + (w_row[t] + r16) * GL_LD + ks * 32 + kb * 8);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[t].v, xf[mt].v, acc[mt][t], 0, 0, 0);
    }
    __syncthreads();  // every wave has read this round's tiles
    if (more) put();
    __syncthreads();
  }

  constexpr int OUT_TILES = GLU ? 2 : 4;
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const int am = m0 + mt * 16 + r16;
    if (am >= P.M) continue;
    uint16_t* cr = P.c + (size_t)am * P.ldc;
#pragma unroll
    for (int t = 0; t < OUT_TILES; ++t) {
      const int n = n0 + (GLU ? wave * 32 : wave * 64) + t * 16 + kb * 4;
      float v[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[i] = acc[mt][t][i];
        if constexpr (GLU) {
          const float g = fminf(v[i], P.limit);
          const float u = fminf(fmaxf(acc[mt][t + 2][i], -P.limit), P.limit);
          v[i] = g * (u + P.up_offset) * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * P.alpha * g));
        }
      }
      if (P.vec_store && n + 3 < P.N) {
        uint2 packed;
        packed.x = rv_pack_bf16x2(v[0], v[1]);
        packed.y = rv_pack_bf16x2(v[2], v[3]);
        *(uint2*)(cr + n) = packed;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < P.N) cr[n + i] = rv_f32_to_bf16_bits(v[i]);
      }
    }
  }
}

// bf16 everywhere (c_f32: the results are the 32-bit sums).  N: columns of C; with `glu` w holds 2 N rows a group.  groups > 0: the heads' form; 0: the
// experts' form with tiles of 16 * token_tiles rows.  token_tiles: 1 (few rows) or 4 (many).  K, the leading dimensions of a and w and the group strides of a and w must
// be multiples of 8 and a, w lie on 16-byte boundaries (a lane reads 16 bytes at a time).
extern "C" int rv_gemm_groups_mfma(hipStream_t stream, const void* a, const void* w, void* c, const int* row_index,
                                   const int* tile_group, int groups, int M, int N, int K, long long lda,
                                   long long ldw, long long ldc, long long a_group_stride, long long w_group_stride,
                                   long long c_group_stride, const void* gate, long long ldg, int glu, float limit,
                                   float alpha, int token_tiles, int c_f32) {
  RV_CHECK(!c_f32 || (groups > 0 && gate == nullptr && !glu),
           "gemm_groups_mfma: 32-bit results come from the heads' form, without a gate or an activation");
  RV_CHECK(M >= 0 && N > 0 && K > 0 && groups >= 0, "gemm_groups_mfma: bad sizes M=%d N=%d K=%d groups=%d", M, N, K, groups);
  RV_CHECK((groups > 0) == (tile_group == nullptr), "gemm_groups_mfma: either a number of groups or the groups of the row tiles");
  RV_CHECK(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && a_group_stride % 8 == 0 && w_group_stride % 8 == 0 &&
               ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0,
           "gemm_groups_mfma: K, the rows' strides and the groups' strides must be multiples of 8 and the operands "
           "16-byte aligned");
  RV_CHECK(lda >= K && ldw >= K && ldc >= N && (gate == nullptr || ldg >= N), "gemm_groups_mfma: rows too short");
  RV_CHECK(!glu || (gate == nullptr && (glu == 2 || limit > 0.f)),
           "gemm_groups_mfma: the gated activation takes a limit and no gate");
  RV_CHECK(token_tiles == 1 || token_tiles == 4, "gemm_groups_mfma: 1 or 4 tiles of 16 tokens a wave, not %d", token_tiles);
  if (M == 0) return 0;
  GroupsParams P;
  P.a = (const uint16_t*)a;
  P.w = (const uint16_t*)w;
  P.c = (uint16_t*)c;
  P.row_index = row_index;
  P.tile_group = tile_group;
  P.gate = (const uint16_t*)gate;
  P.M = M, P.N = N, P.K = K;
  P.lda = lda, P.ldw = ldw, P.ldc = ldc, P.ldg = ldg;
  P.a_group_stride = a_group_stride, P.w_group_stride = w_group_stride, P.c_group_stride = c_group_stride;
  P.limit = limit, P.alpha = alpha, P.up_offset = 1.0f;
  if (glu == 2) P.limit = __builtin_inff(), P.alpha = 1.0f, P.up_offset = 0.0f;  // silu(gate) * up, nothing clamped
  P.c_f32 = c_f32;
  P.vec_store = (ldc % 4 == 0 && c_group_stride % 4 == 0 && ((uintptr_t)c & (c_f32 ? 15 : 7)) == 0) ? 1 : 0;
  if (groups == 0 && token_tiles == 4 && gate == nullptr) {  // the experts' products of many rows: tiles through LDS
    dim3 grid(rv_div_up(N, glu ? GL_BW / 2 : GL_BW), rv_div_up(M, GL_BM)), block(256);
    RV_CHECK(grid.y < 65536, "gemm_groups_mfma: too many row tiles for one launch");
    if (glu) gemm_experts_lds_kernel<true><<<grid, block, 0, stream>>>(P);
    else gemm_experts_lds_kernel<false><<<grid, block, 0, stream>>>(P);
    RV_LAUNCH_CHECK("gemm_experts_lds");
    return 0;
  }
  const int rows_of_w = token_tiles == 1 ? 16 : (glu ? 32 : 64);  // of a wave
  dim3 grid(rv_div_up(N, rows_of_w * 4), rv_div_up(M, 16 * token_tiles), groups > 0 ? groups : 1), block(256);
  RV_CHECK(grid.y < 65536 && grid.z < 65536, "gemm_groups_mfma: too many row tiles or groups for one launch");
  if (glu && token_tiles == 1) gemm_groups_mfma_kernel<1, 1, true><<<grid, block, 0, stream>>>(P);
  else if (glu) gemm_groups_mfma_kernel<4, 2, true><<<grid, block, 0, stream>>>(P);
  else if (token_tiles == 1) gemm_groups_mfma_kernel<1, 1, false><<<grid, block, 0, stream>>>(P);
  else gemm_groups_mfma_kernel<4, 4, false><<<grid, block, 0, stream>>>(P);
  RV_LAUNCH_CHECK("gemm_groups_mfma");
  return 0;
}
