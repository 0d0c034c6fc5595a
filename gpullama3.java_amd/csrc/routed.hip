// A mixture of experts: the choice of a token's experts, the rows of (token, choice) pairs ordered by expert, the
// experts' products over those rows, and the weighted sum per token.
//
// A pair's result depends on its token and its expert alone: the order of the pairs inside an expert's run and the
// tile a pair falls into change nothing, so a token's output does not depend on its batch-mates. Sums over K run in an
// order that the shapes fix.
#include "common.h"

#define ROUTE_MAX_TOP 16
#define ROUTE_MAX_EXPERTS 1024

// ----------------------------------------------------------------- the choice
// logits [T][E] float. The `top` largest (the lower number wins a tie) -> idx [T][top]; their weights are the softmax
// over the chosen logits alone -> wts [T][top]. One thread a token.
// With `scores` set the rule is another: s = softmax over all E logits; the choice goes by s + correction[e]
// (correction may be null), the weights are the chosen s themselves divided by their sum plus sum_eps.
__device__ __forceinline__ void route_choose(const float* __restrict__ logits, int t, int E, int top, int* idx,
                                             float* __restrict__ wts, int always, int scores,
                                             const float* __restrict__ correction, float sum_eps) {
  const float* z = logits + (long)t * E;
  const int stride = top + (always >= 0 ? 1 : 0);
  int chosen[ROUTE_MAX_TOP];
  float val[ROUTE_MAX_TOP];
  float z_max = -INFINITY, z_sum = 1.f;
  if (scores) {
    for (int e = 0; e < E; ++e) z_max = fmaxf(z_max, z[e]);
    z_sum = 0.f;
    for (int e = 0; e < E; ++e) z_sum += expf(z[e] - z_max);
  }
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float bv = -INFINITY, bs = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= chosen[i] == e;
      const float sc = scores ? expf(z[e] - z_max) / z_sum : z[e];
      const float v = (scores && correction) ? sc + correction[e] : sc;
      if (!taken && (best < 0 || v > bv)) {
        best = e;
        bv = v;
        bs = sc;
      }
    }
    chosen[j] = best;
    val[j] = bs;
  }
  float sum = 0.f;
  if (scores) {
    for (int j = 0; j < top; ++j) sum += val[j];
    sum += sum_eps;
  } else {
    const float largest = val[0];          // (the first chosen is the largest)
    for (int j = 0; j < top; ++j) {
      val[j] = expf(val[j] - largest);
      sum += val[j];
    }
  }
  for (int j = 0; j < top; ++j) {
    idx[(long)t * stride + j] = chosen[j];
    wts[(long)t * stride + j] = val[j] / sum;
  }
  if (always >= 0) {                     // one more pair per token: the expert that every token passes, with weight 1
    idx[(long)t * stride + top] = always;
    wts[(long)t * stride + top] = 1.0f;
  }
}

__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ logits, int T, int E, int top,
                                                         int* __restrict__ idx, float* __restrict__ wts, int always, int scores,
                                                         const float* __restrict__ correction, float sum_eps) {
  const int t = blockIdx.x * 64 + threadIdx.x;
  if (t < T) route_choose(logits, t, E, top, idx, wts, always, scores, correction, sum_eps);
}

// ----------------------------------------------------------------- pairs ordered by expert
// idx [n_pairs] -> offsets [E + 1] (the first place of each expert's run) and sorted [n_pairs] (the pairs, expert by
// expert). One block.
__device__ __forceinline__ void route_order(const int* idx, int n_pairs, int E, int* __restrict__ offsets,
                                            int* __restrict__ sorted) {
  __shared__ int count[ROUTE_MAX_EXPERTS + 1];
  __shared__ int cursor[ROUTE_MAX_EXPERTS];
  for (int e = threadIdx.x; e <= E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) atomicAdd(&count[idx[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = count[e];
      count[e] = run;
      cursor[e] = run;
      run += c;
    }
    count[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = count[e];
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) sorted[atomicAdd(&cursor[idx[i]], 1)] = i;
}

__global__ __launch_bounds__(1024) void route_sort_kernel(const int* __restrict__ idx, int n_pairs, int E,
                                                           int* __restrict__ offsets, int* __restrict__ sorted) {
  route_order(idx, n_pairs, E, offsets, sorted);
}

// Both in one launch for a step of at most 1024 tokens (a thread a token, then the block orders the pairs).
__global__ __launch_bounds__(1024) void route_few_kernel(const float* __restrict__ logits, int T, int E, int top,
                                                          int* idx, float* __restrict__ wts,
                                                          int* __restrict__ offsets, int* __restrict__ sorted, int always,
                                                          int scores, const float* __restrict__ correction, float sum_eps) {
  if ((int)threadIdx.x < T) route_choose(logits, threadIdx.x, E, top, idx, wts, always, scores, correction, sum_eps);
  __threadfence_block();
  __syncthreads();
  const int more = always >= 0 ? 1 : 0;
  route_order(idx, T * (top + more), E + more, offsets, sorted);
}

// `always` (-1: none): the number E of one more expert behind the router's, which every token passes with weight 1; idx
// and wts then have top + 1 entries a token, offsets E + 2.
extern "C" int gl3_route(const float* logits, int n_tokens, int E, int top, int* idx, float* wts, int* offsets, int* sorted,
                         int always, int scores, const float* correction, float sum_eps, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(logits && idx && wts && offsets && sorted, "gl3_route: null argument");
  const int more = always >= 0 ? 1 : 0;
  GL3_REQUIRE(n_tokens > 0 && E >= 1 && E + more <= ROUTE_MAX_EXPERTS && top >= 1 && top <= ROUTE_MAX_TOP && top <= E,
              "gl3_route: the %d largest of %d experts (at most %d of %d)", top, E, ROUTE_MAX_TOP, ROUTE_MAX_EXPERTS);
  GL3_REQUIRE(always < 0 || always == E, "gl3_route: the expert that every token passes is number %d, not %d", E, always);
  if (n_tokens <= 64) {
    route_few_kernel<<<dim3(1), dim3(1024), 0, stream>>>(logits, n_tokens, E, top, idx, wts, offsets, sorted, always, scores,
                                                         correction, sum_eps);
    GL3_LAUNCH_CHECK();
    return 0;
  }
  route_topk_kernel<<<dim3((n_tokens + 63) / 64), dim3(64), 0, stream>>>(logits, n_tokens, E, top, idx, wts, always, scores,
                                                                                 correction, sum_eps);
  GL3_LAUNCH_CHECK();
  route_sort_kernel<<<dim3(1), dim3(1024), 0, stream>>>(idx, n_tokens * (top + more), E + more, offsets, sorted);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- the experts' products
// out[pair][n] = act(sum_k A[pair / a_div][k] * W[e][n][k]) for every pair of expert e's run. offsets null: one expert
// over all n_rows rows in their own order (the expert that every token passes). Tiles of TM rows of a run x TN columns;
// a block finds its run by walking the offsets (at most n_rows / TM + E tiles exist; a block beyond them leaves).
__device__ __forceinline__ float gl3_expert_act(float v, int act) {
  if (act == 1) return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));        // gelu, the erf form
  if (act == 2) return gl3_activation<false>(v, GL3_ACT_GELU_TANH);
  if (act == 3) return gl3_activation<false>(v, GL3_ACT_SILU);
  return v;
}

// A gated expert: the rows of W are gate and up in turns (row 2 n the gate's, row 2 n + 1 the up's row n), so a lane that
// holds column c of the sums finds its partner's in the lane beside it; the even one writes column c / 2 of the
// output: act(gate) * (up + shift), both bounded by `limit` first where it is positive (gl3_gated). Every lane of a
// wave must come here (the partner's value travels from lane to lane); `ok` says whether this lane's element exists.
template <typename TO>
__device__ __forceinline__ void expert_store(TO* __restrict__ out, long ldo, int row, int n, bool ok, float v, int act,
                                             int gate_act, float limit, float shift) {
  if (gate_act < 0) {
    if (ok) out[(long)row * ldo + n] = from_f32<TO>(gl3_expert_act(v, act));
    return;
  }
  const float up = __shfl_xor(v, 1, 64);
  if (ok && !(n & 1)) out[(long)row * ldo + (n >> 1)] = from_f32<TO>(gl3_gated<false>(v, up, gate_act, limit, shift));
}

__device__ __forceinline__ bool expert_tile(const int* offsets, int E, int n_rows, int TM, int tile, int* e_out, int* lo_out,
                                            int* hi_out) {
  if (!offsets) {
    *e_out = 0;
    *lo_out = tile * TM;
    *hi_out = n_rows;
    return tile * TM < n_rows;
  }
  for (int e = 0; e < E; ++e) {
    const int lo = offsets[e], hi = offsets[e + 1];
    const int nt = (hi - lo + TM - 1) / TM;
    if (tile < nt) {
      *e_out = e;
      *lo_out = lo + tile * TM;
      *hi_out = hi;
      return true;
    }
    tile -= nt;
  }
  return false;
}

#define EG_TM 16
#define EG_TN 64
#define EG_TK 32
template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void expert_gemm_generic_kernel(const TA* __restrict__ A, long lda, int a_div,
                                                                   const TW* __restrict__ W, int N, int K,
                                                                   const int* __restrict__ offsets,
                                                                   const int* __restrict__ sorted, int E, int n_rows,
                                                                   TO* __restrict__ out, long ldo, int act, int gate_act, float limit,
                                                                   float shift) {
  __shared__ float sa[EG_TM][EG_TK + 1];
  __shared__ float sw[EG_TN][EG_TK + 1];
  __shared__ int rows[EG_TM];
  int e, lo, hi;
  if (!expert_tile(offsets, E, n_rows, EG_TM, blockIdx.x, &e, &lo, &hi)) return;
  const int m = hi - lo < EG_TM ? hi - lo : EG_TM;
  if (threadIdx.x < EG_TM) rows[threadIdx.x] = threadIdx.x < m ? (sorted ? sorted[lo + threadIdx.x] : lo + threadIdx.x) : -1;
  __syncthreads();
  const int n0 = blockIdx.y * EG_TN;
  const TW* We = W + (long)e * N * K;
  const int r = threadIdx.x / 16, cg = threadIdx.x % 16;      // this thread: row r, columns cg + 16 j
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += EG_TK) {
    for (int i = threadIdx.x; i < EG_TM * EG_TK; i += 256) {
      const int rr = i / EG_TK, kk = i % EG_TK;
      sa[rr][kk] = (rows[rr] >= 0 && k0 + kk < K) ? to_f32<TA>(A[(long)(rows[rr] / a_div) * lda + k0 + kk]) : 0.f;
    }
    for (int i = threadIdx.x; i < EG_TN * EG_TK; i += 256) {
      const int nn = i / EG_TK, kk = i % EG_TK;
      sw[nn][kk] = (n0 + nn < N && k0 + kk < K) ? to_f32<TW>(We[(long)(n0 + nn) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < EG_TK; ++kk) {
      const float a = sa[r][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, sw[cg + 16 * j][kk], acc[j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + cg + 16 * j;
    expert_store<TO>(out, ldo, rows[r], n, rows[r] >= 0 && n < N, acc[j], act, gate_act, limit, shift);
  }
}

// The same on the matrix cores for bfloat16: a block of 4 waves works a tile of 64 rows x 64 columns, wave w the
// columns 16 w .. 16 w + 15 of all four row groups; operands come straight from memory, 4 consecutive k a lane (a
// row of A or of W per lane, as v_mfma_f32_16x16x16_bf16 takes them). K must be a multiple of 16.
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short short4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float float4_t;
#define EM_TM 64
#define EM_TN 64
template <typename TO>
__global__ __launch_bounds__(256) void expert_gemm_mfma_kernel(const bf16_t* __restrict__ A, long lda, int a_div,
                                                                const bf16_t* __restrict__ W, int N, int K,
                                                                const int* __restrict__ offsets,
                                                                const int* __restrict__ sorted, int E, int n_rows,
                                                                TO* __restrict__ out, long ldo, int act, int gate_act, float limit,
                                                                   float shift) {
  __shared__ int rows[EM_TM];
  int e, lo, hi;
  if (!expert_tile(offsets, E, n_rows, EM_TM, blockIdx.x, &e, &lo, &hi)) return;
  const int m = hi - lo < EM_TM ? hi - lo : EM_TM;
  if (threadIdx.x < EM_TM) rows[threadIdx.x] = threadIdx.x < m ? (sorted ? sorted[lo + threadIdx.x] : lo + threadIdx.x) : -1;
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int li = lane & 15, kb = (lane >> 4) * 4;           // operand row / column of this lane, and its 4 k
  const int n = blockIdx.y * EM_TN + wave * 16 + li;
  const bf16_t* wp = W + ((long)e * N + (n < N ? n : 0)) * K + kb;
  const bf16_t* ap[4];
  bool a_ok[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int row = rows[g * 16 + li];
    a_ok[g] = row >= 0;
    ap[g] = A + (long)(row >= 0 ? row / a_div : 0) * lda + kb;
  }
  float4_t acc[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) acc[g] = float4_t{0.f, 0.f, 0.f, 0.f};
  const int groups = (m + 15) / 16;
  for (int k0 = 0; k0 < K; k0 += 16) {
    short4_t b = {0, 0, 0, 0};
    if (n < N) b = *reinterpret_cast<const short4_t*>(wp + k0);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      if (g < groups) {
        short4_t a = {0, 0, 0, 0};
        if (a_ok[g]) a = *reinterpret_cast<const short4_t*>(ap[g] + k0);
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, acc[g], 0, 0, 0);
      }
    }
  }
  // a lane holds column li of rows 4 (lane / 16) .. + 3 of every group
  const int nc = blockIdx.y * EM_TN + wave * 16 + li;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = rows[g * 16 + (lane >> 4) * 4 + i];
      expert_store<TO>(out, ldo, row, nc, row >= 0 && nc < N, acc[g][i], act, gate_act, limit, shift);
    }
  }
}

// For few rows (decode steps: an expert's run is a handful of pairs, and the time goes into reading its weights
// once): a block of 8 waves works a tile of 16 G rows of one run x 16 columns (G = 1, 2 or 4 by the runs' mean length,
// so that a run is mostly one tile and its weights are read once), wave w a slice of K (the slices follow from K
// alone), 32 k a step with v_mfma_f32_16x16x32_bf16: a lane holds 8 consecutive k of a row of A and of a row of W,
// read 16 bytes at a time, four steps in flight. The slices' sums are added in their order through shared memory.
typedef __bf16 bf16x8_few_t __attribute__((ext_vector_type(8)));
#define EF_WAVES 8
#define EF_TN 16
template <typename TO, int G>
__global__ __launch_bounds__(EF_WAVES * 64) void expert_gemm_few_kernel(const bf16_t* __restrict__ A, long lda, int a_div,
                                                                        const bf16_t* __restrict__ W, int N, int K,
                                                                        const int* __restrict__ offsets,
                                                                        const int* __restrict__ sorted, int E, int n_rows,
                                                                        TO* __restrict__ out, long ldo, int act, int gate_act, float limit,
                                                                   float shift) {
  constexpr int TM = 16 * G;
  __shared__ int rows[TM];
  __shared__ float part[EF_WAVES][TM][EF_TN + 1];
  int e, lo, hi;
  if (!expert_tile(offsets, E, n_rows, TM, blockIdx.x, &e, &lo, &hi)) return;
  const int m = hi - lo < TM ? hi - lo : TM;
  if (threadIdx.x < TM) rows[threadIdx.x] = (int)threadIdx.x < m ? (sorted ? sorted[lo + threadIdx.x] : lo + threadIdx.x) : -1;
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int li = lane & 15, kg = (lane >> 4) * 8;
  const int n = blockIdx.y * EF_TN + li;
  const int per = ((K + 31) / 32 + EF_WAVES - 1) / EF_WAVES * 32;       // this wave's slice of K
  const int k_lo = wave * per, k_hi = k_lo + per < K ? k_lo + per : K;
  const int groups = (m + 15) / 16;
  const bf16_t* wp = W + ((long)e * N + (n < N ? n : N - 1)) * K + kg;
  const bf16_t* ap[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int row = rows[g * 16 + li];                  // (rows beyond the run read the run's first row; their results are dropped)
    ap[g] = A + (long)((row >= 0 ? row : rows[0]) / a_div) * lda + kg;
  }
  const bf16x8_few_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  float4_t acc[G];
#pragma unroll
  for (int g = 0; g < G; ++g) acc[g] = float4_t{0.f, 0.f, 0.f, 0.f};
  int k0 = k_lo;
  for (; k0 + 128 <= k_hi; k0 += 128) {
    bf16x8_few_t a[4][G], b[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      b[u] = *reinterpret_cast<const bf16x8_few_t*>(wp + k0 + 32 * u);
#pragma unroll
      for (int g = 0; g < G; ++g)
        if (g < groups) a[u][g] = *reinterpret_cast<const bf16x8_few_t*>(ap[g] + k0 + 32 * u);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int g = 0; g < G; ++g)
        if (g < groups) acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][g], b[u], acc[g], 0, 0, 0);
  }
  for (; k0 < k_hi; k0 += 32) {
    const bool in = k0 + kg < k_hi;                     // (K is a multiple of 8: a lane's 8 k lie inside or outside)
    const bf16x8_few_t b = in ? *reinterpret_cast<const bf16x8_few_t*>(wp + k0) : zero;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g < groups) {
        const bf16x8_few_t a = in ? *reinterpret_cast<const bf16x8_few_t*>(ap[g] + k0) : zero;
        acc[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[g], 0, 0, 0);
      }
    }
  }
  // a lane holds column li of rows 4 (lane / 16) .. + 3 of every group
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][g * 16 + (lane >> 4) * 4 + i][li] = acc[g][i];
  __syncthreads();
  for (int base = 0; base < m * EF_TN; base += EF_WAVES * 64) {      // (every lane of a wave that has work walks along)
    const int idx = base + threadIdx.x;
    const bool in = idx < m * EF_TN;
    const int r = in ? idx / EF_TN : 0, c = idx % EF_TN;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < EF_WAVES; ++w) sum += part[w][r][c];
    const int nc = blockIdx.y * EF_TN + c;
    expert_store<TO>(out, ldo, rows[r], nc, in && nc < N, sum, act, gate_act, limit, shift);
  }
}

// For many rows: the tiled product of gemm_mfma.hip over an expert's run. A block of 8 waves works 128 rows of one run
// x 128 columns, a wave 32 x 64 as two tiles of the 32x32x16 instruction; K advances in steps of 64 through two buffers
// in shared memory (while a step's products run out of one, the next step's operands go from registers into the other
// and the step after that travels from memory to registers; one barrier a step; rows padded by 16 bytes against bank
// conflicts). A's rows are gathered through the run's pairs, and the results go to the pairs' own rows.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
#define ET_BM 128
#define ET_BN 128
#define ET_BK 64
#define ET_LD (ET_BK + 8)
template <typename TO>
__global__ __launch_bounds__(512) void expert_gemm_tiled_kernel(const bf16_t* __restrict__ A, long lda, int a_div,
                                                                 const bf16_t* __restrict__ W, int N, int K,
                                                                 const int* __restrict__ offsets,
                                                                 const int* __restrict__ sorted, int E, int n_rows,
                                                                 TO* __restrict__ out, long ldo, int act, int gate_act, float limit,
                                                                   float shift) {
  constexpr int NT = 512, NA = ET_BM * 8 / NT, NWC = ET_BN * 8 / NT;
  __shared__ __attribute__((aligned(16))) bf16_t As[2][ET_BM][ET_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][ET_BN][ET_LD];
  __shared__ int rows[ET_BM];
  int e, lo, hi;
  if (!expert_tile(offsets, E, n_rows, ET_BM, blockIdx.x, &e, &lo, &hi)) return;
  const int m = hi - lo < ET_BM ? hi - lo : ET_BM;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid < ET_BM) rows[tid] = tid < m ? (sorted ? sorted[lo + tid] : lo + tid) : -1;
  __syncthreads();
  const int wm = wave / 2, wn = wave % 2;
  const int lr = lane & 31, lh = lane >> 5;
  const int n0 = blockIdx.y * ET_BN;
  const bf16_t* We = W + (long)e * N * K;
  // every load is unconditional: rows beyond the run read the run's first row, columns beyond N the last one,
  // and their results are dropped
  long aoff[NA], woff[NWC];
  int arow_s[NA], wrow_s[NWC];
  const int scol = (tid & 7) * 8;
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    arow_s[i] = (tid + NT * i) >> 3;
    const int src = rows[arow_s[i]] >= 0 ? rows[arow_s[i]] : rows[0];
    aoff[i] = (long)(src / a_div) * lda;
  }
#pragma unroll
  for (int i = 0; i < NWC; ++i) {
    wrow_s[i] = (tid + NT * i) >> 3;
    woff[i] = (long)min(n0 + wrow_s[i], N - 1) * K;
  }
  const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t ra[NA], rw[NWC];
  bool r_ok = false;
  auto fetch = [&](int k0) {
    const int kf = min(k0, K - 8);                     // the step after the last one reads the last again
    r_ok = k0 + scol < K;
    const int col = min(scol, K - 8 - kf);
#pragma unroll
    for (int i = 0; i < NA; ++i) ra[i] = *(const bf16x8_t*)(A + aoff[i] + kf + col);
#pragma unroll
    for (int i = 0; i < NWC; ++i) rw[i] = *(const bf16x8_t*)(We + woff[i] + kf + col);
  };
  auto store = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NA; ++i) *(bf16x8_t*)&As[buf][arow_s[i]][scol] = r_ok ? ra[i] : zero;
#pragma unroll
    for (int i = 0; i < NWC; ++i) *(bf16x8_t*)&Ws[buf][wrow_s[i]][scol] = r_ok ? rw[i] : zero;
  };
  f32x16_t acc[2];
#pragma unroll
  for (int jn = 0; jn < 2; ++jn)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[jn][v] = 0.f;
  const int arow = wm * 32 + lr, wrow0 = wn * 64 + lr, wrow1 = wn * 64 + 32 + lr;
  fetch(0);
  store(0);
  fetch(ET_BK);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += ET_BK, buf ^= 1) {
#pragma unroll
    for (int kk = 0; kk < ET_BK / 16; ++kk) {
      const int kc = kk * 16 + lh * 8;
      const bf16x8_t b0 = *(const bf16x8_t*)&Ws[buf][wrow0][kc];
      const bf16x8_t b1 = *(const bf16x8_t*)&Ws[buf][wrow1][kc];
      const bf16x8_t a = *(const bf16x8_t*)&As[buf][arow][kc];
      acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b0, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b1, acc[1], 0, 0, 0);
      if (kk == 0) {
        __builtin_amdgcn_sched_barrier(0);
        if (k0 + ET_BK < K) store(buf ^ 1);
        fetch(k0 + 2 * ET_BK);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }
  // a lane holds C[row(v)][col]: row(v) = 8 * (v / 4) + 4 * (lane / 32) + v % 4 inside a 32 x 32 tile, col = lane % 32
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int row = rows[wm * 32 + (v >> 2) * 8 + lh * 4 + (v & 3)];
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
      const int n = n0 + wn * 64 + tn * 32 + lr;
      expert_store<TO>(out, ldo, row, n, row >= 0 && n < N, acc[tn][v], act, gate_act, limit, shift);
    }
  }
}

extern "C" int gl3_expert_gemm(const void* A, int a_dtype, long lda, int a_div, const void* W, int w_dtype, int E, int N, int K,
                               const int* offsets, const int* sorted, int n_rows, void* out, int out_dtype, long ldo, int act,
                               int use_mfma, int gate_act, float limit, float shift, hipStream_t stream) {
  if (n_rows == 0) return 0;
  GL3_REQUIRE(A && W && out && n_rows > 0 && E >= 1 && N > 0 && K > 0 && a_div >= 1 && lda >= K &&
                  ldo >= (gate_act >= 0 ? N / 2 : N),
              "gl3_expert_gemm: bad arguments");
  GL3_REQUIRE(gate_act < 0 || (GL3_ACT_KNOWN(gate_act) && N % 2 == 0),
              "gl3_expert_gemm: a gated expert has gate and up rows in turns (%d rows) and a known activation (%d)", N, gate_act);
  GL3_REQUIRE((offsets == nullptr) == (sorted == nullptr) && (offsets || E == 1),
              "gl3_expert_gemm: runs and their pairs come together; without them one expert takes every row");
  GL3_REQUIRE(act >= 0 && act <= 3, "gl3_expert_gemm: unknown activation %d", act);
  GL3_REQUIRE((N + 63) / 64 <= 65535, "gl3_expert_gemm: %d columns exceed the grid", N);
  const int e_eff = offsets ? E : 1;
  // many rows (an expert's run fills tiles of 128): the tiled kernel
  if (use_mfma && a_dtype == GL3_BF16 && w_dtype == GL3_BF16 && K % 8 == 0 && K >= 8 && lda % 8 == 0 &&
      (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(W) % 16 == 0) &&
      n_rows > 64 * e_eff && (out_dtype == GL3_BF16 || out_dtype == GL3_F32)) {
    const dim3 grid((n_rows + ET_BM - 1) / ET_BM + (offsets ? E : 0), (N + ET_BN - 1) / ET_BN), block(512);
    if (out_dtype == GL3_BF16)
      expert_gemm_tiled_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)A, lda, a_div, (const bf16_t*)W, N, K, offsets,
                                                                   sorted, E, n_rows, (bf16_t*)out, ldo, act, gate_act, limit, shift);
    else
      expert_gemm_tiled_kernel<float><<<grid, block, 0, stream>>>((const bf16_t*)A, lda, a_div, (const bf16_t*)W, N, K, offsets,
                                                                  sorted, E, n_rows, (float*)out, ldo, act, gate_act, limit, shift);
    GL3_LAUNCH_CHECK();
    return 0;
  }
  // few rows (an expert's run is a tile or two): the kernel that reads each weight row in long pieces, K in slices
  if (use_mfma && a_dtype == GL3_BF16 && w_dtype == GL3_BF16 && K % 8 == 0 && lda % 8 == 0 &&
      (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(W) % 16 == 0) &&
      n_rows <= 64 * e_eff && (N + EF_TN - 1) / EF_TN <= 65535 && (out_dtype == GL3_BF16 || out_dtype == GL3_F32)) {
    const int G = n_rows <= 16 * e_eff ? 1 : n_rows <= 32 * e_eff ? 2 : 4;      // by the runs' mean length
    const dim3 grid((n_rows + 16 * G - 1) / (16 * G) + (offsets ? E : 0), (N + EF_TN - 1) / EF_TN), block(EF_WAVES * 64);
#define EF_LAUNCH(TO, G)                                                                                                \
  expert_gemm_few_kernel<TO, G><<<grid, block, 0, stream>>>((const bf16_t*)A, lda, a_div, (const bf16_t*)W, N, K, offsets, \
                                                            sorted, E, n_rows, (TO*)out, ldo, act, gate_act, limit, shift)
    if (out_dtype == GL3_BF16) {
      if (G == 1) EF_LAUNCH(bf16_t, 1); else if (G == 2) EF_LAUNCH(bf16_t, 2); else EF_LAUNCH(bf16_t, 4);
    } else {
      if (G == 1) EF_LAUNCH(float, 1); else if (G == 2) EF_LAUNCH(float, 2); else EF_LAUNCH(float, 4);
    }
#undef EF_LAUNCH
    GL3_LAUNCH_CHECK();
    return 0;
  }
  if (use_mfma && a_dtype == GL3_BF16 && w_dtype == GL3_BF16 && K % 16 == 0 && lda % 4 == 0 &&
      (reinterpret_cast<uintptr_t>(A) % 8 == 0) && (reinterpret_cast<uintptr_t>(W) % 8 == 0)) {
    const dim3 grid((n_rows + EM_TM - 1) / EM_TM + (offsets ? E : 0), (N + EM_TN - 1) / EM_TN), block(256);
    if (out_dtype == GL3_BF16)
      expert_gemm_mfma_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)A, lda, a_div, (const bf16_t*)W, N, K, offsets,
                                                                  sorted, E, n_rows, (bf16_t*)out, ldo, act, gate_act, limit, shift);
    else if (out_dtype == GL3_F32)
      expert_gemm_mfma_kernel<float><<<grid, block, 0, stream>>>((const bf16_t*)A, lda, a_div, (const bf16_t*)W, N, K, offsets,
                                                                 sorted, E, n_rows, (float*)out, ldo, act, gate_act, limit, shift);
    else GL3_REQUIRE(false, "gl3_expert_gemm: unknown output dtype %d", out_dtype);
    GL3_LAUNCH_CHECK();
    return 0;
  }
  const dim3 grid((n_rows + EG_TM - 1) / EG_TM + (offsets ? E : 0), (N + EG_TN - 1) / EG_TN), block(256);
#define EG_LAUNCH(TA, TW, TO)                                                                                          \
  expert_gemm_generic_kernel<TA, TW, TO><<<grid, block, 0, stream>>>((const TA*)A, lda, a_div, (const TW*)W, N, K, offsets, \
                                                                     sorted, E, n_rows, (TO*)out, ldo, act, gate_act, limit, shift)
  if (a_dtype == GL3_F32 && w_dtype == GL3_F32 && out_dtype == GL3_F32) EG_LAUNCH(float, float, float);
  else if (a_dtype == GL3_BF16 && w_dtype == GL3_BF16 && out_dtype == GL3_BF16) EG_LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (a_dtype == GL3_BF16 && w_dtype == GL3_BF16 && out_dtype == GL3_F32) EG_LAUNCH(bf16_t, bf16_t, float);
  else GL3_REQUIRE(false, "gl3_expert_gemm: dtypes %d x %d -> %d are not built", a_dtype, w_dtype, out_dtype);
#undef EG_LAUNCH
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- the weighted sum
// out[t] (+)= sum_j wts[t][j] * y[t * top + j], j in order. One thread an element. With idx [T][top] and n_real: a pair
// whose expert number is n_real or more is an identity expert, whose output is the token's input row h[t] itself (y
// holds nothing for it).
template <typename TH>
__global__ void route_combine_kernel(const float* __restrict__ y, const float* __restrict__ wts, int top, int d,
                                     float* __restrict__ out, int accumulate, long n, const int* __restrict__ idx,
                                     int n_real, const TH* __restrict__ h) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / d;
  const int c = i % d;
  float s = accumulate ? out[i] : 0.f;
  for (int j = 0; j < top; ++j) {
    const float v = (idx && idx[t * top + j] >= n_real) ? to_f32<TH>(h[t * d + c]) : y[(t * top + j) * d + c];
    s = fmaf(wts[t * top + j], v, s);
  }
  out[i] = s;
}

extern "C" int gl3_route_combine(const float* y, const float* wts, int n_tokens, int top, int d, float* out, int accumulate,
                                 const int* idx, int n_real, const void* h, int h_dtype, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(y && wts && out && n_tokens > 0 && top >= 1 && d > 0, "gl3_route_combine: bad arguments");
  GL3_REQUIRE((idx == nullptr) == (h == nullptr), "gl3_route_combine: identity experts need the choices and the input rows");
  const long n = (long)n_tokens * d;
  GL3_REQUIRE((n + 255) / 256 < (1L << 31), "gl3_route_combine: too many elements");
  if (h && h_dtype == GL3_BF16)
    route_combine_kernel<bf16_t><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(y, wts, top, d, out, accumulate, n,
                                                                                            idx, n_real, (const bf16_t*)h);
  else
    route_combine_kernel<float><<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(y, wts, top, d, out, accumulate, n,
                                                                                           idx, n_real, (const float*)h);
  GL3_LAUNCH_CHECK();
  return 0;
}
