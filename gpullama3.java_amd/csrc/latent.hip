// The pieces around an attention whose keys and values are expanded from one small latent per position.
//
// Per position the cache keeps ONE row for all heads: [c (rank) | r (rot) | zeros up to a multiple of 32], c the
// normed latent and r the rotated key part that the heads share. A head's key is W_uk c beside r and its value W_uv c,
// so with the query's unrotated part taken through W_uk^T (a row of `rank` numbers per head) the scores are dot
// products with the cached rows themselves, and the weighted sum of the cached c goes through W_uv afterwards: the
// attention is one over a single key/value head whose values are the keys' first `rank` elements.
//
//   gl3_latent_prep    the two norms and the shared key part's rotation, the cache write, and the runs that let the
//                      grouped product work head by head
//   gl3_latent_query   the rotated part of every head's query into its place behind the absorbed part
//   gl3_sigmoid_gate   rows times the sigmoid of 32-bit gate columns
//   gl3_latent_attention  the attention itself on the matrix cores (bfloat16; the kernel for any sizes and for 32-bit
//                      is attention_generic.hip's, which reads values out of the key rows)
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

// ----------------------------------------------------------------- the attention over the cached rows, on the matrix cores
// q [T][H dk] (the absorbed queries), the cache rows [c | r | zeros] of dk elements (a multiple of 32), values = a
// row's first `rank` elements (a multiple of 16). One key/value head for all query heads, so the rows of the first
// product are (token, head) pairs: a block of NW waves takes 16 NW consecutive pairs of one sequence (row t H + h),
// a wave 16 of them, and walks the keys 0 .. (the last pair's position) in chunks of 32 that the block stages in
// shared memory ONCE for all its heads: as rows [key][dk] for the scores' operand, and the first `rank` columns
// again transposed, [dim][key], for the second product's (the cache has no transposed copy of a latent).
// Scores S = Q K^T with v_mfma_f32_16x16x32_bf16 (a lane ends up with 4 rows x 1 key of each 16 x 16 tile), scale,
// causal mask by each pair's own position, running maximum and sum per row in 32-bit (reduced over the 16 lanes that
// share a row), the weights in bfloat16 through a wave's own patch of shared memory into operand order, O += P V.
// A decode step is the same kernel with one token a sequence (rows = heads).
typedef __bf16 la_bf16x8 __attribute__((ext_vector_type(8)));
typedef float la_f32x4 __attribute__((ext_vector_type(4)));
// A value over the 16 lanes that share a row of sums (a row of the data-parallel moves): neighbours in a quad, the
// other quad of a half, the other half; the moves are vector instructions, where a shuffle goes through shared memory.
template <int CTRL>
__device__ __forceinline__ float la_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float la_max16(float v) {
  v = fmaxf(v, la_move<0xB1>(v));       // lanes 1 0 3 2 of a quad
  v = fmaxf(v, la_move<0x4E>(v));       // lanes 2 3 0 1
  v = fmaxf(v, la_move<0x141>(v));      // a half of 8 mirrored: the other quad's (equal) values
  return fmaxf(v, la_move<0x140>(v));   // the row of 16 mirrored: the other half's
}
__device__ __forceinline__ float la_sum16(float v) {
  v += la_move<0xB1>(v);
  v += la_move<0x4E>(v);
  v += la_move<0x141>(v);
  return v + la_move<0x140>(v);
}
#define LA_LDV 40        // a transposed value row: 32 keys and 8 of padding
#define LA_LDP 40        // a row of a wave's weights

template <int NW, int RT, int MAXKS, int MAXDT>
__global__ __launch_bounds__(NW * 64) void latent_attention_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache, const int* __restrict__ cu_seqlens,
    const int* __restrict__ kv_before, const int* __restrict__ block_table, const int* __restrict__ seq_rows, int table_stride,
    bf16_t* __restrict__ out, long out_stride, int H, int dk, int rank, int page_size, float scale, int n_splits,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  // a wave takes RT tiles of 16 pairs: an operand of keys or values read from shared memory serves all of them
  constexpr int MAXP = (32 * MAXKS * 4 + NW * 64 - 1) / (NW * 64);      // pieces of a chunk that a thread carries
  constexpr int ROWS = NW * RT * 16;
  extern __shared__ __attribute__((aligned(16))) char la_smem[];
  const int s = blockIdx.y, split = blockIdx.z;
  const int tok0 = cu_seqlens[s], q_len = cu_seqlens[s + 1] - tok0, before = kv_before[s];
  const int rows_total = q_len * H;
  // A tile late in a sequence walks many keys, an early one few, and the blocks of a launch mostly run side by side:
  // the second half of the blocks takes the tiles from the end, so that blocks which share a CU (one of each half,
  // as blocks are handed out in order) carry about the same work together.
  const int nb = gridDim.x, hb = (nb + 1) / 2;
  const int tile = (int)blockIdx.x < hb ? 2 * blockIdx.x : 2 * (nb - 1 - blockIdx.x) + 1;
  const int row0 = (tile < nb ? tile : nb - 1) * ROWS;
  if (tile >= nb || row0 >= rows_total) return;
  const int* bt = block_table + (long)(seq_rows ? seq_rows[s] : s) * table_stride;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 15, lq = lane >> 4;
  const int ks = dk >> 5, dt_n = rank >> 4, ldk = dk + 8;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(la_smem);                 // [32][ldk]
  bf16_t* Vt = Ks + 32 * ldk;                                      // [rank][LA_LDV]
  bf16_t* Ps = Vt + rank * LA_LDV + wave * (RT * 16 * LA_LDP);     // [RT 16][LA_LDP], this wave's
  const la_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int wrow0 = row0 + wave * RT * 16;
  // this lane's part of the queries as the first product's operand: pair wrow0 + 16 rt + li, 8 elements at 32 step + 8 lq
  la_bf16x8 qf[RT][MAXKS];
  int pos[RT][4];
  float m_run[RT][4], l_run[RT][4];
  la_f32x4 O[RT][MAXDT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int a_row = wrow0 + 16 * rt + li;
    const bool a_ok = a_row < rows_total;
    const bf16_t* qp = q + (long)(tok0 + (a_ok ? a_row / H : 0)) * q_stride + (long)(a_ok ? a_row % H : 0) * dk + 8 * lq;
#pragma unroll
    for (int st = 0; st < MAXKS; ++st) qf[rt][st] = (st < ks && a_ok) ? *reinterpret_cast<const la_bf16x8*>(qp + 32 * st) : zero;
    // the four pairs whose sums this lane holds: rows 4 lq + i of the tile's 16
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = wrow0 + 16 * rt + 4 * lq + i;
      pos[rt][i] = r < rows_total ? before + r / H : -1;
      m_run[rt][i] = -INFINITY;
      l_run[rt][i] = 0.f;
    }
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt) O[rt][dt] = la_f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const int last = (row0 + ROWS < rows_total ? row0 + ROWS : rows_total) - 1;
  const int p_max = before + last / H;
  // this block's share of the keys: whole chunks of 32, the splits one after another
  const int chunks = p_max / 32 + 1, per = (chunks + n_splits - 1) / n_splits;
  const int k_lo = split * per * 32;
  const int k_end = (split + 1) * per * 32 - 1 < p_max ? (split + 1) * per * 32 - 1 : p_max;
  const int cbs = dk >> 3, pieces = 32 * cbs;
  const float scale2 = scale * 1.4426950408889634f;
  // a chunk travels from memory into registers while the chunk before it is worked on; piece e is 8 consecutive
  // elements of the cache in the cache's own order
  la_bf16x8 pre[MAXP];
  auto fetch = [&](int k0) {
    const bf16_t* src = k_cache + (long)bt[k0 / page_size] * page_size * dk + (long)((k0 % page_size) >> 5) * 32 * dk;
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
      const int g = threadIdx.x + u * NW * 64;      // 16 lanes a (column block, tile of 16 keys): see the staging below
      const int e = ((g >> 4) & 1) * 16 * cbs + (g >> 5) * 16 + (g & 15);
      if (g < pieces) pre[u] = *reinterpret_cast<const la_bf16x8*>(src + (long)e * 8);
    }
  };
  if (k_lo <= k_end) fetch(k_lo);
  for (int k0 = k_lo; k0 <= k_end; k0 += 32) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < MAXP; ++u) {
      // (the two tiles of a column block side by side in a wave: their transposed writes fall on banks of their own,
      // where four column blocks of one tile would share theirs)
      const int g = threadIdx.x + u * NW * 64;
      if (g < pieces) {
        const int tl = (g >> 4) & 1, cb = g >> 5, row = g & 15;
        const int p32 = ((row >> 2) << 3) | (tl << 2) | (row & 3);      // the key's place among the 32 (gl3_k_offset, inverted)
        const la_bf16x8 v = k0 + p32 <= p_max ? pre[u] : zero;
        *reinterpret_cast<la_bf16x8*>(Ks + p32 * ldk + cb * 8) = v;
        if (cb * 8 < rank) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (cb * 8 + j < rank) Vt[(cb * 8 + j) * LA_LDV + p32] = v[j];
        }
      }
    }
    __syncthreads();
    if (k0 + 32 <= k_end) fetch(k0 + 32);
    la_f32x4 S0[RT], S1[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) S0[rt] = S1[rt] = la_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < MAXKS; ++st) {
      if (st < ks) {
        const la_bf16x8 b0 = *reinterpret_cast<const la_bf16x8*>(Ks + li * ldk + 32 * st + 8 * lq);
        const la_bf16x8 b1 = *reinterpret_cast<const la_bf16x8*>(Ks + (16 + li) * ldk + 32 * st + 8 * lq);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          S0[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[rt][st], b0, S0[rt], 0, 0, 0);
          S1[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[rt][st], b1, S1[rt], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float alpha[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // (scores in units of ln 2: the weights are powers of two, one instruction each)
        const float s0 = k0 + li <= pos[rt][i] ? S0[rt][i] * scale2 : -INFINITY;
        const float s1 = k0 + 16 + li <= pos[rt][i] ? S1[rt][i] * scale2 : -INFINITY;
        const float m_new = fmaxf(m_run[rt][i], la_max16(fmaxf(s0, s1)));
        const float p0 = s0 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s0 - m_new);
        const float p1 = s1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s1 - m_new);
        const float rs = la_sum16(p0 + p1);
        alpha[i] = m_run[rt][i] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run[rt][i] - m_new);
        l_run[rt][i] = l_run[rt][i] * alpha[i] + rs;
        m_run[rt][i] = m_new;
        Ps[(16 * rt + 4 * lq + i) * LA_LDP + li] = static_cast<bf16_t>(p0);
        Ps[(16 * rt + 4 * lq + i) * LA_LDP + 16 + li] = static_cast<bf16_t>(p1);
      }
      // (the sums so far shrink only when a row's maximum has grown: rarely, once a row has seen some keys)
      if (__any(alpha[0] != 1.f || alpha[1] != 1.f || alpha[2] != 1.f || alpha[3] != 1.f)) {
#pragma unroll
        for (int dt = 0; dt < MAXDT; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) O[rt][dt][i] *= alpha[i];
      }
    }
    // (the weights of this wave's rows lie in its own patch: the wave's reads follow its writes in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    la_bf16x8 pf[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) pf[rt] = *reinterpret_cast<const la_bf16x8*>(Ps + (16 * rt + li) * LA_LDP + 8 * lq);
#pragma unroll
    for (int dt = 0; dt < MAXDT; ++dt) {
      if (dt < dt_n) {
        const la_bf16x8 b = *reinterpret_cast<const la_bf16x8*>(Vt + (16 * dt + li) * LA_LDV + 8 * lq);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) O[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[rt], b, O[rt][dt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = wrow0 + 16 * rt + 4 * lq + i;
      if (r >= rows_total) continue;
      if (n_splits > 1) {
        // this split's share as it stands: the sums under its own maximum, with that maximum and its row sum
        const long th = (long)(tok0 + r / H) * H + r % H;
        float* po = part_o + (th * n_splits + split) * rank + li;
#pragma unroll
        for (int dt = 0; dt < MAXDT; ++dt)
          if (dt < dt_n) po[16 * dt] = O[rt][dt][i];
        if (li == 0) {
          part_ml[(th * n_splits + split) * 2] = m_run[rt][i] * 0.6931471805599453f;      // (as a natural logarithm)
          part_ml[(th * n_splits + split) * 2 + 1] = l_run[rt][i];
        }
        continue;
      }
      bf16_t* op = out + (long)(tok0 + r / H) * out_stride + (long)(r % H) * rank + li;
      const float inv = 1.0f / l_run[rt][i];
#pragma unroll
      for (int dt = 0; dt < MAXDT; ++dt)
        if (dt < dt_n) op[16 * dt] = static_cast<bf16_t>(O[rt][dt][i] * inv);
    }
  }
}

// The splits of one (token, head) joined: a thread a value column; every thread works out the splits' factors itself
// (a few numbers that the whole block reads), and adds its column over the splits in their order.
__global__ __launch_bounds__(256) void latent_attention_merge_kernel(const float* __restrict__ part_o,
                                                                     const float* __restrict__ part_ml, bf16_t* __restrict__ out,
                                                                     long out_stride, int H, int rank, int n_splits) {
  const long th = blockIdx.x;
  const int d = threadIdx.x;
  const float* ml = part_ml + th * n_splits * 2;
  float M = -INFINITY;
  for (int sp = 0; sp < n_splits; ++sp) M = fmaxf(M, ml[2 * sp]);
  const float* po = part_o + th * n_splits * rank;
  float L = 0.f, acc = 0.f;
  for (int sp = 0; sp < n_splits; ++sp) {
    const float m = ml[2 * sp];
    const float f = m == -INFINITY ? 0.f : expf(m - M);
    L = fmaf(f, ml[2 * sp + 1], L);
    if (d < rank) acc = fmaf(f, po[(long)sp * rank + d], acc);
  }
  if (d < rank) out[(th / H) * out_stride + (th % H) * rank + d] = static_cast<bf16_t>(acc / L);
}

static inline size_t la_smem_bytes(int tiles, int dk, int rank) {      // tiles: the block's tiles of 16 pairs
  return ((size_t)32 * (dk + 8) + (size_t)rank * LA_LDV + (size_t)tiles * 16 * LA_LDP) * sizeof(bf16_t);
}

// Whether the kernel is built for these sizes: cached rows of a multiple of 32 up to 288 elements, values of a multiple
// of 16 up to 256, pages of a multiple of 32.
extern "C" int gl3_latent_attention_supports(int dk, int rank, int page_size) {
  return dk > 0 && dk % 32 == 0 && dk <= 288 && rank > 0 && rank % 16 == 0 && rank <= 256 && rank <= dk && page_size > 0 &&
         page_size % 32 == 0 && la_smem_bytes(8, dk, rank) <= 64000;
}

// n_splits > 1 (at most 64): the keys of every sequence are shared out over that many blocks, whose parts (part_o
// [T H][n_splits][rank], part_ml [T H][n_splits][2] floats) a second kernel joins.
extern "C" int gl3_latent_attention(const void* q, long q_stride, const void* k_cache, const int* cu_seqlens, const int* kv_before,
                                    const int* block_table, const int* seq_rows, int table_stride, void* out, long out_stride,
                                    int n_tokens, int n_seqs, int max_q_len, int H, int dk, int rank, int page_size, float scale,
                                    int n_splits, float* part_o, float* part_ml, long part_floats, hipStream_t stream) {
  if (n_seqs == 0 || max_q_len == 0) return 0;
  GL3_REQUIRE(q && k_cache && cu_seqlens && kv_before && block_table && out && table_stride > 0, "gl3_latent_attention: null argument");
  GL3_REQUIRE(gl3_latent_attention_supports(dk, rank, page_size),
              "gl3_latent_attention: cached rows of %d with values of %d in pages of %d are not built", dk, rank, page_size);
  GL3_REQUIRE(H > 0 && q_stride >= (long)H * dk && out_stride >= (long)H * rank && q_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                  (uintptr_t)k_cache % 16 == 0,
              "gl3_latent_attention: rows of %ld for %d heads of %d; queries and cache 16-byte aligned", q_stride, H, dk);
  GL3_REQUIRE(n_splits >= 1 && n_splits <= 64, "gl3_latent_attention: n_splits=%d", n_splits);
  if (n_splits > 1)
    GL3_REQUIRE(part_o && part_ml && n_tokens > 0 && part_floats >= (long)n_tokens * H * n_splits * (rank + 2),
                "gl3_latent_attention: the splits' workspace of %ld floats is too small", part_floats);
  // A tile of 16 pairs a wave; 4 waves where a sequence brings at most 64 pairs (the waves beyond them still carry
  // their share of every chunk), else 8: 128 pairs a block. (Two tiles a wave, which halve the reads of shared memory
  // per multiply-add, took 252 registers a lane and one wave a SIMD: 659 us where this takes 407, 2,048 tokens of 32
  // heads over rows of 288.)
  const long rows = (long)max_q_len * H;
  const int nw = rows <= 64 ? 4 : 8;
  const long blocks = (rows + nw * 16 - 1) / (nw * 16);
  GL3_REQUIRE(blocks < (1L << 31) && n_seqs <= 65535, "gl3_latent_attention: too many blocks");
  const dim3 grid((unsigned)blocks, n_seqs, n_splits);
  const size_t sh = la_smem_bytes(nw, dk, rank);
  const bool small = dk <= 96 && rank <= 64;
#define LA_GO(NW, KS, DT)                                                                                             \
  latent_attention_kernel<NW, 1, KS, DT><<<grid, dim3(NW * 64), sh, stream>>>(                                        \
      (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, cu_seqlens, kv_before, block_table, seq_rows, table_stride, \
      (bf16_t*)out, out_stride, H, dk, rank, page_size, scale, n_splits, part_o, part_ml)
  if (small) {
    if (nw == 4) LA_GO(4, 3, 4); else LA_GO(8, 3, 4);
  } else {
    if (nw == 4) LA_GO(4, 9, 16); else LA_GO(8, 9, 16);
  }
#undef LA_GO
  GL3_LAUNCH_CHECK();
  if (n_splits > 1) {
    latent_attention_merge_kernel<<<dim3((unsigned)((long)n_tokens * H)), dim3((rank + 63) / 64 * 64), 0, stream>>>(
        part_o, part_ml, (bf16_t*)out, out_stride, H, rank, n_splits);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}
