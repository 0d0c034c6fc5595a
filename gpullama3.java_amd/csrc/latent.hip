// The pieces around an attention whose keys and values are expanded from one small latent per position.
//
// Per position the cache keeps ONE row for all heads: [c (rank) | r (rot) | zeros up to a multiple of 16], c the
// normed latent and r the rotated key part that the heads share. A head's key is W_uk c beside r and its value W_uv c,
// so with the query's unrotated part taken through W_uk^T (a row of `rank` numbers per head) the scores are dot
// products with the cached rows themselves, and the weighted sum of the cached c goes through W_uv afterwards: the
// attention is one over a single key/value head whose values are the keys' first `rank` elements.
//
//   gl3_latent_prep    the two norms and the shared key part's rotation, the cache write, and the runs that let the
//                      grouped product work head by head
//   gl3_latent_query   the rotated part of every head's query into its place behind the absorbed part
//   gl3_sigmoid_gate   rows times the sigmoid of 32-bit gate columns
// Norms, angles and the rotation are 32-bit arithmetic.
#include "common.h"

// proj [T][ld] float: the query latent's sums from col_q (q_rank of them), the key/value latent's from col_kv (rank,
// then rot). cq [T][q_rank] = proj / rms * wq. The cache row (tiles of gl3_k_offset, one head of dk elements):
// [proj / rms * wkv | the rot part turned in adjacent pairs by the token's position | zeros].
// runs: offsets [H + 1] and sorted [T H] such that "expert" h owns the rows t * H + h of all tokens.
template <typename TC>
__global__ __launch_bounds__(256) void latent_prep_kernel(const float* __restrict__ proj, long ld, int col_q, int q_rank,
                                                           int col_kv, int rank, int rot, const float* __restrict__ wq,
                                                           const float* __restrict__ wkv, float eps,
                                                           const int* __restrict__ positions, const int* __restrict__ table_rows,
                                                           const int* __restrict__ block_table, int table_stride,
                                                           const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                           TC* __restrict__ cq, TC* __restrict__ k_cache, int page_size, int dk,
                                                           int T, int H, int* __restrict__ offsets, int* __restrict__ sorted) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = proj + (long)t * ld;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq = fmaf(row[col_q + i], row[col_q + i], sq);
  for (int i = threadIdx.x; i < rank; i += blockDim.x) sk = fmaf(row[col_kv + i], row[col_kv + i], sk);
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float iq = 1.0f / sqrtf(sq / (float)q_rank + eps), ik = 1.0f / sqrtf(sk / (float)rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq[(long)t * q_rank + i] = from_f32<TC>(row[col_q + i] * iq * wq[i]);
  const int p = positions[t];
  const int page = block_table[(long)table_rows[t] * table_stride + p / page_size], in_page = p % page_size;
  TC* kp = k_cache + (long)page * page_size * dk;
  for (int i = threadIdx.x; i < rank; i += blockDim.x)
    kp[gl3_k_offset(in_page, i, dk)] = from_f32<TC>(row[col_kv + i] * ik * wkv[i]);
  const int half = rot / 2;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float c = cos_t[(long)p * half + i], s = sin_t[(long)p * half + i];
    const float u = row[col_kv + rank + 2 * i], v = row[col_kv + rank + 2 * i + 1];
    kp[gl3_k_offset(in_page, rank + 2 * i, dk)] = from_f32<TC>(u * c - v * s);
    kp[gl3_k_offset(in_page, rank + 2 * i + 1, dk)] = from_f32<TC>(v * c + u * s);
  }
  for (int i = rank + rot + threadIdx.x; i < dk; i += blockDim.x) kp[gl3_k_offset(in_page, i, dk)] = from_f32<TC>(0.f);
  // the runs: token t writes its own places
  for (int h = threadIdx.x; h < H; h += blockDim.x) sorted[(long)h * T + t] = t * H + h;
  if (t == 0)
    for (int h = threadIdx.x; h <= H; h += blockDim.x) offsets[h] = h * T;
}

extern "C" int gl3_latent_prep(const float* proj, long ld, int n_tokens, int col_q, int q_rank, int col_kv, int rank, int rot,
                               const float* wq, const float* wkv, float eps, const int* positions, const int* table_rows,
                               const int* block_table, int table_stride, const float* cos_t, const float* sin_t, void* cq,
                               void* k_cache, int dtype, int page_size, int dk, int H, int* offsets, int* sorted,
                               hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(proj && wq && wkv && positions && table_rows && block_table && cq && k_cache && offsets && sorted,
              "gl3_latent_prep: null argument");
  GL3_REQUIRE(n_tokens > 0 && q_rank > 0 && rank > 0 && rot >= 0 && rot % 2 == 0 && (rot == 0 || (cos_t && sin_t)) && H > 0,
              "gl3_latent_prep: latents of %d and %d, %d rotated elements", q_rank, rank, rot);
  GL3_REQUIRE(col_q >= 0 && col_q + q_rank <= ld && col_kv >= 0 && col_kv + rank + rot <= ld, "gl3_latent_prep: columns beyond the rows");
  GL3_REQUIRE(dk >= rank + rot && dk % 16 == 0 && page_size % 32 == 0 && table_stride > 0,
              "gl3_latent_prep: cached rows of %d for %d + %d elements, pages of %d", dk, rank, rot, page_size);
  GL3_REQUIRE((long)n_tokens * H < (1L << 31), "gl3_latent_prep: too many (token, head) rows");
#define LP(TC)                                                                                                              \
  latent_prep_kernel<TC><<<dim3(n_tokens), dim3(256), 0, stream>>>(proj, ld, col_q, q_rank, col_kv, rank, rot, wq, wkv, eps,  \
                                                                   positions, table_rows, block_table, table_stride, cos_t,  \
                                                                   sin_t, (TC*)cq, (TC*)k_cache, page_size, dk, n_tokens, H, \
                                                                   offsets, sorted)
  if (dtype == GL3_F32) LP(float);
  else if (dtype == GL3_BF16) LP(bf16_t);
  else GL3_REQUIRE(false, "gl3_latent_prep: unknown dtype %d", dtype);
#undef LP
  GL3_LAUNCH_CHECK();
  return 0;
}

// q [T][H (dim + rot)]: per head [dim unrotated | rot rotated]. qa [T][H][dk]: the rotated part, turned in adjacent
// pairs by the token's position, goes to columns rank .. rank + rot, zeros behind it (columns 0 .. rank are the
// grouped product's).
template <typename TC>
__global__ __launch_bounds__(256) void latent_query_kernel(const TC* __restrict__ q, int H, int dim, int rot,
                                                            const int* __restrict__ positions, const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t, TC* __restrict__ qa, int rank, int dk) {
  const long t = blockIdx.x;
  const int p = positions[t], half = rot / 2, tail = dk - rank - rot;
  const int per = half + tail;
  for (int e = threadIdx.x; e < H * per; e += blockDim.x) {
    const int h = e / per, i = e % per;
    TC* out = qa + (t * H + h) * dk + rank;
    if (i < half) {
      const TC* in = q + (t * H + h) * (dim + rot) + dim;
      const float c = cos_t[(long)p * half + i], s = sin_t[(long)p * half + i];
      const float u = to_f32<TC>(in[2 * i]), v = to_f32<TC>(in[2 * i + 1]);
      out[2 * i] = from_f32<TC>(u * c - v * s);
      out[2 * i + 1] = from_f32<TC>(v * c + u * s);
    } else {
      out[rot + i - half] = from_f32<TC>(0.f);
    }
  }
}

extern "C" int gl3_latent_query(const void* q, int dtype, int n_tokens, int H, int dim, int rot, const int* positions,
                                const float* cos_t, const float* sin_t, void* qa, int rank, int dk, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(q && positions && qa && n_tokens > 0 && H > 0 && dim >= 0 && rot >= 0 && rot % 2 == 0 && (rot == 0 || (cos_t && sin_t)) &&
                  dk >= rank + rot,
              "gl3_latent_query: bad arguments");
  if (dk == rank && rot == 0) return 0;
  if (dtype == GL3_F32)
    latent_query_kernel<float><<<dim3(n_tokens), dim3(256), 0, stream>>>((const float*)q, H, dim, rot, positions, cos_t, sin_t,
                                                                         (float*)qa, rank, dk);
  else if (dtype == GL3_BF16)
    latent_query_kernel<bf16_t><<<dim3(n_tokens), dim3(256), 0, stream>>>((const bf16_t*)q, H, dim, rot, positions, cos_t, sin_t,
                                                                          (bf16_t*)qa, rank, dk);
  else GL3_REQUIRE(false, "gl3_latent_query: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// a [T][C] *= sigmoid(gate[t][col_g + c]), the gate's sums in 32-bit.
template <typename TC>
__global__ void sigmoid_gate_kernel(TC* __restrict__ a, const float* __restrict__ gate, long ld_g, int col_g, int C, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / C;
  const int c = i % C;
  const float g = gate[t * ld_g + col_g + c];
  a[i] = from_f32<TC>(to_f32<TC>(a[i]) / (1.0f + expf(-g)));
}

extern "C" int gl3_sigmoid_gate(void* a, int dtype, const float* gate, long ld_g, int col_g, int n_tokens, int C,
                                hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(a && gate && n_tokens > 0 && C > 0 && col_g >= 0 && col_g + C <= ld_g, "gl3_sigmoid_gate: bad arguments");
  const long n = (long)n_tokens * C;
  GL3_REQUIRE((n + 255) / 256 < (1L << 31), "gl3_sigmoid_gate: too many elements");
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (dtype == GL3_F32) sigmoid_gate_kernel<float><<<grid, block, 0, stream>>>((float*)a, gate, ld_g, col_g, C, n);
  else if (dtype == GL3_BF16) sigmoid_gate_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)a, gate, ld_g, col_g, C, n);
  else GL3_REQUIRE(false, "gl3_sigmoid_gate: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}
