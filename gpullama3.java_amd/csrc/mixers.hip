// Kernels of mixers that keep a state per sequence instead of (or beside) a cache of keys and values, and of what
// stands around them: a hashed second embedding row, the mixture of the residual rows with the embedding's output,
// rotations of whole heads in place, a gate per head, the average of two normalised rows.
// Everything here computes in 32-bit; only what is handed to a matrix product is stored in the activations' type.
#include "common.h"

// ----------------------------------------------------------------- the row of a table of token pairs
// rows[t] = (previous token * mul_prev + token * mul_cur) mod buckets, or `buckets` (the table's last row) for a
// sequence's first token. The previous token of a step's first token is what the sequence's slot holds (held[0] of
// its row of `state`); the thread of that first token also leaves the step's last token there, after it has read, so
// no other thread touches the slot's row.
__global__ void pair_rows_kernel(const int* __restrict__ token_ids, const int* __restrict__ positions,
                                 const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                                 const int* __restrict__ slot_ids, int* __restrict__ state, long state_stride,
                                 long mul_prev, long mul_cur, long buckets, int* __restrict__ rows, int n_tokens) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_tokens) return;
  const int seq = seq_of_token[t];
  const int first = cu_seqlens[seq], last = cu_seqlens[seq + 1] - 1;
  int* held = state + (long)slot_ids[seq] * state_stride;
  const long prev = t > first ? token_ids[t - 1] : held[0];
  rows[t] = positions[t] == 0 ? (int)buckets : (int)((prev * mul_prev + (long)token_ids[t] * mul_cur) % buckets);
  if (t == first) held[0] = token_ids[last];
}

extern "C" int gl3_pair_rows(const int* token_ids, const int* positions, const int* seq_of_token, const int* cu_seqlens,
                             const int* slot_ids, int* state, long state_stride, long mul_prev, long mul_cur, long buckets,
                             int* rows, int n_tokens, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(token_ids && positions && seq_of_token && cu_seqlens && slot_ids && state && rows && n_tokens > 0,
              "gl3_pair_rows: bad arguments");
  GL3_REQUIRE(buckets > 0 && buckets < (1L << 31) && mul_prev >= 0 && mul_prev < (1L << 31) && mul_cur >= 0 &&
                  mul_cur < (1L << 31) && state_stride > 0,
              "gl3_pair_rows: %ld buckets, multipliers %ld and %ld", buckets, mul_prev, mul_cur);
  pair_rows_kernel<<<dim3((n_tokens + 255) / 256), dim3(256), 0, stream>>>(
      token_ids, positions, seq_of_token, cu_seqlens, slot_ids, state, state_stride, mul_prev, mul_cur, buckets, rows,
      n_tokens);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- [x; x0] as a product's input
template <typename T>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out, long n, int d) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / d;
  const int c = (int)(i - t * d);
  out[t * 2 * d + c] = from_f32<T>(a[i]);
  out[t * 2 * d + d + c] = from_f32<T>(b[i]);
}

extern "C" int gl3_concat_rows(const float* a, const float* b, void* out, int out_dtype, int n_tokens, int d,
                               hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(a && b && out && n_tokens > 0 && d > 0, "gl3_concat_rows: bad arguments");
  const long n = (long)n_tokens * d;
  const long blocks = (n + 255) / 256;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_concat_rows: %ld elements is too many", n);
  if (out_dtype == GL3_F32)
    concat_rows_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a, b, (float*)out, n, d);
  else if (out_dtype == GL3_BF16)
    concat_rows_kernel<bf16_t><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a, b, (bf16_t*)out, n, d);
  else GL3_REQUIRE(false, "gl3_concat_rows: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- heads turned in place
// Up to three runs of heads inside rows [T][ld] (queries, keys, values of one projection, or one run: an attention's
// output) are rotated by the token's position: the first rot_dim elements of every head as pairs (j, j + rot_dim/2)
// (or (2j, 2j+1)), by the angle whose cos and sin stand in the run's table [position][rot_dim/2]; `back` turns by
// minus the angle. With `gate` (rows [T][gate_ld] of the same type, head h's value at column gate_col + h; one run
// only) every element of head h, rotated or not, is multiplied by sigmoid(gate) afterwards.
// A run with norm_w (float [head_dim]) is first divided by its root mean square per head (over the head's norm_dim
// elements, eps inside the root; elements behind them are padding and hold zeros) and multiplied by norm_w.
struct RotRun {
  int col, heads, head_dim, rot_dim;
  const float* cos_tab;
  const float* sin_tab;
  const float* norm_w;
  int norm_dim;
  float norm_eps;
};

// With a cache (k_cache not null; three runs: queries, keys, values) the second and third run also go to the token's
// place in its page as they come out of the rotation: keys [page][kv head][position][head_dim], values transposed, both
// in the tiles of gl3_k_offset / gl3_v_offset; page = block_table[table_rows[t] * table_stride + position / page_size].
template <typename T>
__global__ __launch_bounds__(64) void rotate_heads_kernel(T* __restrict__ rows, long ld, const int* __restrict__ positions,
                                                           RotRun a, RotRun b, RotRun c, int adjacent, int back,
                                                           const T* __restrict__ gate, long gate_ld, int gate_col,
                                                           T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                           const int* __restrict__ table_rows,
                                                           const int* __restrict__ block_table, int table_stride,
                                                           int page_size) {
  const int t = blockIdx.x;
  int head = blockIdx.y, which = 0;
  RotRun r = a;
  if (head >= a.heads) {
    head -= a.heads;
    r = b;
    which = 1;
    if (head >= b.heads) {
      head -= b.heads;
      r = c;
      which = 2;
    }
  }
  const int pos = positions[t];
  T* p = rows + (long)t * ld + r.col + (long)head * r.head_dim;
  const int half = r.rot_dim / 2;
  const float g = gate ? 1.0f / (1.0f + expf(-to_f32<T>(gate[(long)t * gate_ld + gate_col + head]))) : 1.0f;
  T* dst = nullptr;          // the head's page of the cache, if it goes there
  const int in_page = pos % page_size;
  if (k_cache && which > 0) {
    const long page = block_table[(long)table_rows[t] * table_stride + pos / page_size];
    dst = (which == 1 ? k_cache : v_cache) + (page * r.heads + head) * (long)page_size * r.head_dim;
  }
  auto put = [&](int i, T v) {
    p[i] = v;
    if (dst) dst[which == 1 ? gl3_k_offset(in_page, i, r.head_dim) : gl3_v_offset(i, in_page, page_size)] = v;
  };
  float inv = 1.0f;
  if (r.norm_w) {      // (the whole head is read before any of it is written: the block is one wave)
    float ss = 0.f;
    for (int i = threadIdx.x; i < r.norm_dim; i += 64) {
      const float v = to_f32<T>(p[i]);
      ss += v * v;
    }
    inv = 1.0f / sqrtf(wave_sum(ss) / (float)r.norm_dim + r.norm_eps);
  }
  auto get = [&](int i) {
    const float v = to_f32<T>(p[i]);
    return r.norm_w ? v * inv * r.norm_w[i] : v;
  };
  if (r.cos_tab) {
    for (int j = threadIdx.x; j < half; j += 64) {
      const int i0 = adjacent ? 2 * j : j, i1 = adjacent ? 2 * j + 1 : j + half;
      const float cs = r.cos_tab[(long)pos * half + j];
      const float sn = back ? -r.sin_tab[(long)pos * half + j] : r.sin_tab[(long)pos * half + j];
      const float v0 = get(i0), v1 = get(i1);
      put(i0, from_f32<T>((v0 * cs - v1 * sn) * g));
      put(i1, from_f32<T>((v1 * cs + v0 * sn) * g));
    }
  }
  if (gate || dst || r.norm_w)
    for (int i = (r.cos_tab ? r.rot_dim : 0) + threadIdx.x; i < r.head_dim; i += 64) put(i, from_f32<T>(get(i) * g));
}

extern "C" int gl3_rotate_heads(void* rows, int dtype, long ld, const int* positions, int n_tokens, const int* cols,
                                const int* heads, const int* head_dims, const int* rot_dims, const float* const* cos_tabs,
                                const float* const* sin_tabs, int n_runs, int adjacent, int back, const void* gate,
                                long gate_ld, int gate_col, void* k_cache, void* v_cache, const int* table_rows,
                                const int* block_table, int table_stride, int page_size, const float* const* norm_ws,
                                const int* norm_dims, float norm_eps, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(rows && positions && n_tokens > 0 && n_runs >= 1 && n_runs <= 3, "gl3_rotate_heads: bad arguments");
  GL3_REQUIRE(!gate || n_runs == 1, "gl3_rotate_heads: a gate goes with one run of heads");
  RotRun r[3] = {};
  long total = 0;
  for (int i = 0; i < n_runs; ++i) {
    r[i] = RotRun{cols[i], heads[i], head_dims[i], rot_dims[i], cos_tabs[i], sin_tabs[i], norm_ws ? norm_ws[i] : nullptr,
                  norm_ws && norm_ws[i] ? norm_dims[i] : 0, norm_eps};
    GL3_REQUIRE(!r[i].norm_w || (r[i].norm_dim > 0 && r[i].norm_dim <= head_dims[i]),
                "gl3_rotate_heads: run %d: a norm over %d of %d elements", i, r[i].norm_dim, head_dims[i]);
    GL3_REQUIRE(heads[i] > 0 && head_dims[i] > 0 && rot_dims[i] >= 0 && rot_dims[i] % 2 == 0 && rot_dims[i] <= head_dims[i] &&
                    cols[i] >= 0 && cols[i] + (long)heads[i] * head_dims[i] <= ld && (cos_tabs[i] == nullptr) == (sin_tabs[i] == nullptr),
                "gl3_rotate_heads: run %d: %d heads of %d (%d rotated) from column %d of rows of %ld", i, heads[i],
                head_dims[i], rot_dims[i], cols[i], ld);
    total += heads[i];
  }
  GL3_REQUIRE(total <= 65535, "gl3_rotate_heads: %ld heads exceed the grid", total);
  if (k_cache) {
    GL3_REQUIRE(v_cache && table_rows && block_table && table_stride > 0 && n_runs == 3,
                "gl3_rotate_heads: a cache write takes queries, keys and values");
    GL3_REQUIRE(page_size > 0 && page_size % 32 == 0 && head_dims[1] % 16 == 0 && head_dims[2] % 16 == 0,
                "gl3_rotate_heads: the cache lies in tiles: page_size %d must be a multiple of 32, head sizes %d and %d of 16",
                page_size, head_dims[1], head_dims[2]);
  } else {
    page_size = 1;
  }
  dim3 grid(n_tokens, (unsigned)total), block(64);
  if (dtype == GL3_F32)
    rotate_heads_kernel<float><<<grid, block, 0, stream>>>((float*)rows, ld, positions, r[0], r[1], r[2], adjacent, back,
                                                           (const float*)gate, gate_ld, gate_col, (float*)k_cache,
                                                           (float*)v_cache, table_rows, block_table, table_stride, page_size);
  else if (dtype == GL3_BF16)
    rotate_heads_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)rows, ld, positions, r[0], r[1], r[2], adjacent, back,
                                                            (const bf16_t*)gate, gate_ld, gate_col, (bf16_t*)k_cache,
                                                            (bf16_t*)v_cache, table_rows, block_table, table_stride, page_size);
  else GL3_REQUIRE(false, "gl3_rotate_heads: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- x += f * (a / rms(a) * wa + b / rms(b) * wb)
// One block a token. `b` may be null (one side only). Sums in an order that depends on d and the block's size alone.
// ssq (may be null; then at most 64 tokens): ssq[t] = the sum of squares of the completed row, for a norm that is
// folded into the product that follows; with it next_weight [d] and xg [T][d]: xg = bfloat16(next_weight * row).
__global__ __launch_bounds__(1024) void sides_norm_add_kernel(float* __restrict__ x, const float* __restrict__ a,
                                                               const float* __restrict__ b, const float* __restrict__ wa,
                                                               const float* __restrict__ wb, float eps, float f, int d,
                                                               float* __restrict__ ssq, const float* __restrict__ next_weight,
                                                               bf16_t* __restrict__ xg) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const float* pa = a + t * d;
  const float* pb = b ? b + t * d : nullptr;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    const float va = pa[i];
    sa += va * va;
    if (pb) {
      const float vb = pb[i];
      sb += vb * vb;
    }
  }
  sa = block_sum(sa, scratch);
  sb = block_sum(sb, scratch);
  const float ia = 1.0f / sqrtf(sa / (float)d + eps), ib = 1.0f / sqrtf(sb / (float)d + eps);
  float ss = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = pa[i] * ia * wa[i];
    if (pb) v += pb[i] * ib * wb[i];
    const float xn = x[t * d + i] + f * v;
    x[t * d + i] = xn;
    ss += xn * xn;
    if (xg) xg[t * d + i] = static_cast<bf16_t>(next_weight[i] * xn);
  }
  if (ssq) {
    ss = block_sum(ss, scratch);
    if (threadIdx.x == 0) ssq[t] = ss;
  }
}

extern "C" int gl3_sides_norm_add(float* x, const float* a, const float* b, const float* wa, const float* wb, float eps,
                                  float f, int n_tokens, int d, float* ssq, const float* next_weight, void* xg,
                                  hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(x && a && wa && (!b || wb) && n_tokens > 0 && d > 0, "gl3_sides_norm_add: bad arguments");
  GL3_REQUIRE(!ssq || n_tokens <= 64, "gl3_sides_norm_add: sums of squares are kept for at most 64 rows");
  GL3_REQUIRE((next_weight == nullptr) == (xg == nullptr) && (!xg || ssq),
              "gl3_sides_norm_add: the next norm's weight and its rows come together, with the sums of squares");
  const int threads = d >= 1024 ? 1024 : ((d + 63) / 64) * 64;
  sides_norm_add_kernel<<<dim3(n_tokens), dim3(threads), 0, stream>>>(x, a, b, wa, wb, eps, f, d, ssq, next_weight, (bf16_t*)xg);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- out = tanh(in) in the activations' type
// in: rows of `ld` floats, `cols` of them used; out: [rows][cols] contiguous
template <typename T>
__global__ void tanh_rows_kernel(const float* __restrict__ in, long ld, int cols, T* __restrict__ out, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(tanhf(in[(i / cols) * ld + i % cols]));
}

extern "C" int gl3_tanh_rows(const float* in, long ld, int cols, void* out, int out_dtype, long n, hipStream_t stream) {
  if (n == 0) return 0;
  GL3_REQUIRE(in && out && n > 0 && cols > 0 && ld >= cols && (n + 255) / 256 < (1L << 31), "gl3_tanh_rows: bad arguments");
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_dtype == GL3_F32) tanh_rows_kernel<float><<<grid, block, 0, stream>>>(in, ld, cols, (float*)out, n);
  else if (out_dtype == GL3_BF16) tanh_rows_kernel<bf16_t><<<grid, block, 0, stream>>>(in, ld, cols, (bf16_t*)out, n);
  else GL3_REQUIRE(false, "gl3_tanh_rows: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- minGRU
// proj [T][ld] float: columns 0 .. W the update gate's sums (biased), W .. 2W the candidate's, 2W .. 3W the output
// gate's. Per sequence and channel, token by token from the state in the sequence's slot:
//   z = sigmoid(pz); c = pu >= 0 ? pu + 1/2 : sigmoid(pu); S = (1 - z) S + z c; out = S * silu(pg).
// grid (channels / 256, sequences). A step's tokens of one sequence are walked in order, so every cut of a
// sequence into steps gives the same numbers.
template <typename TO>
__global__ __launch_bounds__(256) void mingru_scan_kernel(const float* __restrict__ proj, long ld, int W,
                                                           float* __restrict__ state, long state_stride,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ slot_ids, TO* __restrict__ out) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= W) return;
  const int seq = blockIdx.y;
  float* held = state + (long)slot_ids[seq] * state_stride + c;
  float S = *held;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const float* p = proj + (long)t * ld + c;
    const float pz = p[0], pu = p[W], pg = p[2 * W];
    const float z = 1.0f / (1.0f + expf(-pz));
    const float cand = pu >= 0.f ? pu + 0.5f : 1.0f / (1.0f + expf(-pu));
    S = (1.0f - z) * S + z * cand;
    out[(long)t * W + c] = from_f32<TO>(S * (pg / (1.0f + expf(-pg))));
  }
  *held = S;
}

// The same recurrence for long prompts, in three passes over runs of MG_RUN tokens. S_t = (1 - z_t) S_(t-1) + z_t c_t
// is linear in S, so a run of tokens maps the state before it to A S + B with A = prod (1 - z), B = the run's scan
// from zero: (1) every run's A and B, all runs at once; (2) per sequence and channel the state in front of every run,
// run after run (a prompt of 2,048 tokens: 64 steps, not 2,048), and the sequence's last state into its slot; (3)
// every run again from its own start, writing the outputs. Twice the arithmetic, a thirtieth of the chain.
#define MG_RUN 32

__global__ __launch_bounds__(256) void mingru_runs_kernel(const float* __restrict__ proj, long ld, int W,
                                                           const int* __restrict__ cu_seqlens, float* __restrict__ run_a,
                                                           float* __restrict__ run_b, int n_runs) {
  const int c = blockIdx.x * 256 + threadIdx.x, run = blockIdx.y, seq = blockIdx.z;
  const int t0 = cu_seqlens[seq] + run * MG_RUN, end = cu_seqlens[seq + 1];
  if (c >= W || t0 >= end) return;
  const int t1 = t0 + MG_RUN < end ? t0 + MG_RUN : end;
  float A = 1.f, B = 0.f;
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const float* p = proj + (long)t * ld + c;
    const float pz = p[0], pu = p[W];
    const float z = 1.0f / (1.0f + expf(-pz));
    const float cand = pu >= 0.f ? pu + 0.5f : 1.0f / (1.0f + expf(-pu));
    A *= 1.0f - z;
    B = (1.0f - z) * B + z * cand;
  }
  const long at = ((long)seq * n_runs + run) * W + c;
  run_a[at] = A;
  run_b[at] = B;
}

// run_a: in A, out the state in front of the run
__global__ __launch_bounds__(256) void mingru_carry_kernel(float* __restrict__ run_a, const float* __restrict__ run_b,
                                                            float* __restrict__ state, long state_stride,
                                                            const int* __restrict__ cu_seqlens,
                                                            const int* __restrict__ slot_ids, int W, int n_runs) {
  const int c = blockIdx.x * 256 + threadIdx.x, seq = blockIdx.y;
  if (c >= W) return;
  float* held = state + (long)slot_ids[seq] * state_stride + c;
  float S = *held;
  const int n = (cu_seqlens[seq + 1] - cu_seqlens[seq] + MG_RUN - 1) / MG_RUN;
  for (int run = 0; run < n; ++run) {
    const long at = ((long)seq * n_runs + run) * W + c;
    const float A = run_a[at], B = run_b[at];
    run_a[at] = S;
    S = A * S + B;
  }
  *held = S;
}

template <typename TO>
__global__ __launch_bounds__(256) void mingru_apply_kernel(const float* __restrict__ proj, long ld, int W,
                                                            const int* __restrict__ cu_seqlens,
                                                            const float* __restrict__ run_start, int n_runs,
                                                            TO* __restrict__ out) {
  const int c = blockIdx.x * 256 + threadIdx.x, run = blockIdx.y, seq = blockIdx.z;
  const int t0 = cu_seqlens[seq] + run * MG_RUN, end = cu_seqlens[seq + 1];
  if (c >= W || t0 >= end) return;
  const int t1 = t0 + MG_RUN < end ? t0 + MG_RUN : end;
  float S = run_start[((long)seq * n_runs + run) * W + c];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const float* p = proj + (long)t * ld + c;
    const float pz = p[0], pu = p[W], pg = p[2 * W];
    const float z = 1.0f / (1.0f + expf(-pz));
    const float cand = pu >= 0.f ? pu + 0.5f : 1.0f / (1.0f + expf(-pu));
    S = (1.0f - z) * S + z * cand;
    out[(long)t * W + c] = from_f32<TO>(S * (pg / (1.0f + expf(-pg))));
  }
}

// max_q_len: the most tokens a sequence brings (host's knowledge); runs [2][n_seqs][ceil(max_q_len / 32)][W] floats of
// scratch (may be null: one pass, token by token).
extern "C" int gl3_mingru_scan(const float* proj, long ld, int W, float* state, long state_stride, const int* cu_seqlens,
                               const int* slot_ids, void* out, int out_dtype, int n_seqs, int max_q_len, float* runs,
                               hipStream_t stream) {
  if (n_seqs == 0) return 0;
  GL3_REQUIRE(proj && state && cu_seqlens && slot_ids && out && W > 0 && ld >= 3L * W && state_stride >= W &&
                  n_seqs > 0 && n_seqs <= 65535, "gl3_mingru_scan: bad arguments (W=%d ld=%ld B=%d)", W, ld, n_seqs);
  GL3_REQUIRE(out_dtype == GL3_F32 || out_dtype == GL3_BF16, "gl3_mingru_scan: unknown dtype %d", out_dtype);
  if (runs && max_q_len > MG_RUN) {
    const int n_runs = (max_q_len + MG_RUN - 1) / MG_RUN;
    GL3_REQUIRE(n_runs <= 65535, "gl3_mingru_scan: %d tokens a sequence exceed the grid", max_q_len);
    float* run_a = runs;
    float* run_b = runs + (long)n_seqs * n_runs * W;
    dim3 grid((W + 255) / 256, n_runs, n_seqs), block(256);
    mingru_runs_kernel<<<grid, block, 0, stream>>>(proj, ld, W, cu_seqlens, run_a, run_b, n_runs);
    mingru_carry_kernel<<<dim3((W + 255) / 256, n_seqs), block, 0, stream>>>(run_a, run_b, state, state_stride, cu_seqlens,
                                                                           slot_ids, W, n_runs);
    if (out_dtype == GL3_F32)
      mingru_apply_kernel<float><<<grid, block, 0, stream>>>(proj, ld, W, cu_seqlens, run_a, n_runs, (float*)out);
    else
      mingru_apply_kernel<bf16_t><<<grid, block, 0, stream>>>(proj, ld, W, cu_seqlens, run_a, n_runs, (bf16_t*)out);
    GL3_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((W + 255) / 256, n_seqs), block(256);
  if (out_dtype == GL3_F32)
    mingru_scan_kernel<float><<<grid, block, 0, stream>>>(proj, ld, W, state, state_stride, cu_seqlens, slot_ids, (float*)out);
  else
    mingru_scan_kernel<bf16_t><<<grid, block, 0, stream>>>(proj, ld, W, state, state_stride, cu_seqlens, slot_ids, (bf16_t*)out);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- blends with the previous token's row
// out[s][t] = h[t] + (h'[t] - h[t]) * mu[s] for s < n_mix, h' the row of the token before t in its sequence: row
// t - 1 of the step, or for a step's first token what the sequence's slot holds (zeros at a sequence's start).
// `inline_update` (every sequence brings one token): the thread that read element i of the held row writes the
// token's own there; otherwise gl3_keep_last_rows runs after this kernel.
template <typename T>
__global__ __launch_bounds__(256) void shift_mix_kernel(const T* __restrict__ h, int d, const float* __restrict__ mu,
                                                         int n_mix, float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ cu_seqlens,
                                                         const int* __restrict__ seq_of_token,
                                                         const int* __restrict__ slot_ids, T* __restrict__ out,
                                                         long n_tokens, int inline_update) {
  const long t = blockIdx.x;
  const int seq = seq_of_token[t];
  const bool from_step = t > cu_seqlens[seq];
  float* held = state + (long)slot_ids[seq] * state_stride;
  // (grid y: the row's elements in runs of 256, one a thread: nothing in a thread waits for an earlier trip to memory)
  for (int i = blockIdx.y * 256 + threadIdx.x; i < d; i += 256 * gridDim.y) {
    const float cur = to_f32<T>(h[t * d + i]);
    const float prev = from_step ? to_f32<T>(h[(t - 1) * d + i]) : held[i];
    const float diff = prev - cur;
    for (int s = 0; s < n_mix; ++s) out[((long)s * n_tokens + t) * d + i] = from_f32<T>(cur + diff * mu[(long)s * d + i]);
    if (inline_update) held[i] = cur;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void keep_last_rows_kernel(const T* __restrict__ h, int d, float* __restrict__ state,
                                                              long state_stride, const int* __restrict__ cu_seqlens,
                                                              const int* __restrict__ slot_ids) {
  const int seq = blockIdx.x;
  const long last = cu_seqlens[seq + 1] - 1;
  if (last < cu_seqlens[seq]) return;
  float* held = state + (long)slot_ids[seq] * state_stride;
  for (int i = threadIdx.x; i < d; i += 256) held[i] = to_f32<T>(h[last * d + i]);
}

extern "C" int gl3_shift_mix(const void* h, int dtype, int d, const float* mu, int n_mix, float* state, long state_stride,
                             const int* cu_seqlens, const int* seq_of_token, const int* slot_ids, void* out, int n_tokens,
                             int n_seqs, int one_token_each, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(h && mu && state && cu_seqlens && seq_of_token && slot_ids && out && d > 0 && n_mix > 0 && n_tokens > 0 &&
                  n_seqs > 0 && state_stride >= d && (d + 255) / 256 <= 65535, "gl3_shift_mix: bad arguments");
  const int inl = one_token_each && n_tokens == n_seqs;
  if (dtype == GL3_F32) {
    shift_mix_kernel<float><<<dim3(n_tokens, (d + 255) / 256), dim3(256), 0, stream>>>((const float*)h, d, mu, n_mix, state, state_stride,
                                                                      cu_seqlens, seq_of_token, slot_ids, (float*)out, n_tokens, inl);
    if (!inl) keep_last_rows_kernel<float><<<dim3(n_seqs), dim3(256), 0, stream>>>((const float*)h, d, state, state_stride, cu_seqlens, slot_ids);
  } else if (dtype == GL3_BF16) {
    shift_mix_kernel<bf16_t><<<dim3(n_tokens, (d + 255) / 256), dim3(256), 0, stream>>>((const bf16_t*)h, d, mu, n_mix, state, state_stride,
                                                                       cu_seqlens, seq_of_token, slot_ids, (bf16_t*)out, n_tokens, inl);
    if (!inl) keep_last_rows_kernel<bf16_t><<<dim3(n_seqs), dim3(256), 0, stream>>>((const bf16_t*)h, d, state, state_stride, cu_seqlens, slot_ids);
  } else GL3_REQUIRE(false, "gl3_shift_mix: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- the decayed matrix per head
// Per sequence and head a matrix S [D keys][D values] in 32-bit (state: [H][D][D] floats from `state_off` of the
// slot's row). r, k, v, wl are [T][H*D] float; the decay of key channel i is w = exp(-exp(wl)); bonus [H][D].
//   o_t[j] = sum_i r_t[i] (S[i][j] + bonus[i] k_t[i] v_t[j]);   S[i][j] <- w_t[i] S[i][j] + k_t[i] v_t[j]
// Tokens are walked in order from the state in the slot, so every cut of a sequence into steps gives the same sums.
//
// grid (H, sequences). A wave owns RP rows (keys) of 64 columns (values): a lane keeps its column's RP elements of S
// in registers. A round of `ch` tokens' r, k, w (the two exponentials are taken here, once an element) and v reaches
// the block through shared memory: every thread loads its share of the NEXT round into registers before it works on
// the current one, and stores it afterwards, so a trip to memory is paid once a round and hidden behind the work.
// The waves' parts of a column's sum over the rows meet in shared memory too, and are added in the order of the
// parts after the round's one barrier. Both areas have two buffers, which is why one barrier a round is enough: a
// wave writes a buffer again only after the barrier that every wave passes after its last read of it.
#define TM_MAXD 256
#define TM_LD 8           // loads a thread has on their way for the next round

// r, k, v are rows of `ld` floats, wl rows of `ld_w` (a token's H*D values from the pointer on). o (may be null): the raw
// read-outs [T][H*D]. out (may be null; then gate, rows of `ld_g`, and norm_w [H*D]): at the end of a round one wave a
// token divides the head's read-out by its root mean square and multiplies by the weight per channel and silu(gate):
// out[t, h, i] = o / sqrt(mean_i(o^2) + eps) * norm_w[h*D + i] * silu(gate[t, h*D + i]), in the activations' type.
template <int RP, typename TO>
__global__ __launch_bounds__(1024) void timemix_kernel(const float* __restrict__ r, const float* __restrict__ k,
                                                        const float* __restrict__ v, long ld, const float* __restrict__ wl,
                                                        long ld_w, const float* __restrict__ bonus, float* __restrict__ state,
                                                        long state_stride, long state_off,
                                                        const int* __restrict__ cu_seqlens,
                                                        const int* __restrict__ slot_ids, float* __restrict__ o, int H,
                                                        int D, int ch, const float* __restrict__ gate, long ld_g,
                                                        const float* __restrict__ norm_w, float eps, TO* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) float tm_shared[];
  const int head = blockIdx.x, seq = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int CG = (D + 63) / 64;                // groups of 64 columns
  const int P = (D + RP - 1) / RP;             // parts of RP rows
  const int cols = CG * 64, Dr = P * RP;       // a staged row's length: whole parts
  const int part = wave / CG, j = (wave - part * CG) * 64 + lane, i0 = part * RP;
  const bool col_ok = j < D;
  const long HD = (long)H * D;
  // shared memory: stage [2][ch][4][Dr] (r, k, w, v of a token), parts [2][ch][P * cols]
  float* stage = tm_shared;
  float* parts = tm_shared + 2 * ch * 4 * Dr;
  float* held = state + (long)slot_ids[seq] * state_stride + state_off + (long)head * D * D;
  float S[RP], ub[RP];
#pragma unroll
  for (int ii = 0; ii < RP; ++ii) {
    S[ii] = (col_ok && i0 + ii < D) ? held[(long)(i0 + ii) * D + j] : 0.f;
    ub[ii] = i0 + ii < D ? bonus[head * D + i0 + ii] : 0.f;
  }
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  float ld_[TM_LD];
  // item idx = tid + m * nt of a round: token idx / (4 D), array (idx / D) % 4, element idx % D. A thread's items are
  // the same in every round, so where they come from and go to is worked out once (the divisions are not cheap).
  const float* from[TM_LD];      // the item's address in the round that starts at token t0
  int to[TM_LD], token[TM_LD];   // its place in a stage buffer (-1 - place for a decay, which passes the exponentials)
  long step[TM_LD];              // floats from a token's row to the next token's
#pragma unroll
  for (int m = 0; m < TM_LD; ++m) {
    const int idx = tid + m * nt;
    const int tt = idx / (4 * D), rest = idx - tt * 4 * D, a = rest / D, i = rest - a * D;
    const float* src = a == 0 ? r : a == 1 ? k : a == 2 ? wl : v;
    from[m] = src + (long)(t0 + tt) * (a == 2 ? ld_w : ld) + (long)head * D + i;
    step[m] = a == 2 ? ld_w : ld;
    token[m] = tt < ch ? tt : 0x7fffffff;
    to[m] = (tt * 4 + a) * Dr + i;
    if (a == 2) to[m] = -1 - to[m];
  }
  auto fetch = [&](int tb) {
    const int n = t1 - tb;
#pragma unroll
    for (int m = 0; m < TM_LD; ++m) ld_[m] = token[m] < n ? from[m][(long)(tb - t0) * step[m]] : 0.f;
  };
  auto put = [&](int buf, int tb) {
    const int n = t1 - tb;
#pragma unroll
    for (int m = 0; m < TM_LD; ++m)
      if (token[m] < n) {
        if (to[m] >= 0) stage[buf * ch * 4 * Dr + to[m]] = ld_[m];
        else stage[buf * ch * 4 * Dr - 1 - to[m]] = expf(-expf(ld_[m]));
      }
  };
  if (t0 < t1) {
    fetch(t0);
    put(0, t0);
  }
  __syncthreads();
  int buf = 0;
  for (int tb = t0; tb < t1; tb += ch, buf ^= 1) {
    const int n = t1 - tb < ch ? t1 - tb : ch;
    if (tb + ch < t1) fetch(tb + ch);
    for (int tt = 0; tt < n; ++tt) {
      const float* row = stage + (buf * ch + tt) * 4 * Dr;
      const float vj = col_ok ? row[3 * Dr + j] : 0.f;
      float acc = 0.f;
#pragma unroll
      for (int i4 = 0; i4 < RP; i4 += 4) {
        if (i0 + i4 < D) {     // (the same for the whole wave; rows behind D inside a group of four hold what was staged: nothing they add is read)
          const float4 r4 = *(const float4*)(row + i0 + i4), k4 = *(const float4*)(row + Dr + i0 + i4),
                       w4 = *(const float4*)(row + 2 * Dr + i0 + i4);
          const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk[4] = {k4.x, k4.y, k4.z, k4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (i0 + i4 + e < D) {
              const float kv = kk[e] * vj;
              acc = fmaf(rr[e], fmaf(ub[i4 + e], kv, S[i4 + e]), acc);
              S[i4 + e] = fmaf(ww[e], S[i4 + e], kv);
            }
          }
        }
      }
      parts[(buf * ch + tt) * P * cols + part * cols + j] = acc;
    }
    if (tb + ch < t1) put(buf ^ 1, tb + ch);
    __syncthreads();
    for (int idx = tid; idx < n * D; idx += nt) {
      const int tt = idx / D, jj = idx - tt * D;
      float sum = 0.f;
      for (int p = 0; p < P; ++p) sum += parts[(buf * ch + tt) * P * cols + p * cols + jj];
      if (o) o[(long)(tb + tt) * HD + (long)head * D + jj] = sum;
      if (out) parts[(buf * ch + tt) * P * cols + jj] = sum;      // (the first part's place: only this thread reads it)
    }
    if (out) {
      __syncthreads();
      for (int tt = wave; tt < n; tt += nt >> 6) {
        const float* sums = parts + (buf * ch + tt) * P * cols;
        float ss = 0.f;
        for (int i = lane; i < D; i += 64) ss += sums[i] * sums[i];
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)D + eps);
        for (int i = lane; i < D; i += 64) {
          const float g = gate[(long)(tb + tt) * ld_g + (long)head * D + i];
          out[(long)(tb + tt) * HD + (long)head * D + i] =
              from_f32<TO>(sums[i] * inv * norm_w[head * D + i] * (g / (1.0f + expf(-g))));
        }
      }
    }
  }
#pragma unroll
  for (int ii = 0; ii < RP; ++ii)
    if (col_ok && i0 + ii < D) held[(long)(i0 + ii) * D + j] = S[ii];
}

// rows a wave owns: 8 for heads of up to 64 (eight waves a head), 16 up to 128, 64 beyond
static int timemix_rows(int D) { return D <= 64 ? 8 : D <= 128 ? 16 : 64; }

extern "C" int gl3_timemix(const float* r, const float* k, const float* v, long ld, const float* wl, long ld_w,
                           const float* bonus, float* state, long state_stride, long state_off, const int* cu_seqlens,
                           const int* slot_ids, float* o, int n_seqs, int H, int D, const float* gate, long ld_g,
                           const float* norm_w, float eps, void* out, int out_dtype, int max_q_len, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  GL3_REQUIRE(r && k && v && wl && bonus && state && cu_seqlens && slot_ids && (o || out) && n_seqs > 0 && n_seqs <= 65535 &&
                  H > 0, "gl3_timemix: bad arguments");
  GL3_REQUIRE(D >= 1 && D <= TM_MAXD, "gl3_timemix: heads of %d elements: the kernel holds up to %d", D, TM_MAXD);
  GL3_REQUIRE(ld >= (long)H * D && ld_w >= (long)H * D, "gl3_timemix: rows of %ld and %ld floats for %d heads of %d", ld, ld_w, H, D);
  GL3_REQUIRE(!out || (gate && norm_w && ld_g >= (long)H * D && (out_dtype == GL3_F32 || out_dtype == GL3_BF16)),
              "gl3_timemix: the read-outs' norm needs the gate, the weight and an output of a known type");
  GL3_REQUIRE(state_off >= 0 && state_off + (long)H * D * D <= state_stride, "gl3_timemix: the state's row of %ld floats", state_stride);
  dim3 grid(H, n_seqs);
  const int RP = timemix_rows(D), CG = (D + 63) / 64, P = (D + RP - 1) / RP;
  const int nt = 64 * CG * P, Dr = P * RP, per_token = 2 * 4 * Dr + 2 * P * CG * 64;
  // tokens a round: what 60 KB of shared memory hold, what the threads' TM_LD loads each bring, 16 at most
  int ch = 15360 / per_token;
  if (ch > TM_LD * nt / (4 * D)) ch = TM_LD * nt / (4 * D);
  if (ch > 16) ch = 16;
  // (max_q_len > 0: no sequence brings more tokens than that; a decode step's blocks then ask for a round of one token's
  // shared memory, and a CU holds as many of them as its registers allow, not two)
  if (max_q_len > 0 && ch > max_q_len) ch = max_q_len;
  GL3_REQUIRE(ch >= 1 && nt <= 1024, "gl3_timemix: heads of %d do not fit the kernel's shared memory", D);
  const size_t shared = (size_t)ch * per_token * sizeof(float);
#define TM_ARGS r, k, v, ld, wl, ld_w, bonus, state, state_stride, state_off, cu_seqlens, slot_ids, o, H, D, ch, gate, ld_g, norm_w, eps
#define TM_GO(R)                                                                                                    \
  do {                                                                                                              \
    if (out && out_dtype == GL3_BF16) timemix_kernel<R, bf16_t><<<grid, dim3(nt), shared, stream>>>(TM_ARGS, (bf16_t*)out); \
    else timemix_kernel<R, float><<<grid, dim3(nt), shared, stream>>>(TM_ARGS, (float*)out);                       \
  } while (0)
  if (RP == 8) TM_GO(8);
  else if (RP == 16) TM_GO(16);
  else TM_GO(64);
#undef TM_GO
#undef TM_ARGS
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- a norm per head, a weight per channel, a gate
// out[t, h, i] = o[t, h, i] / sqrt(mean_i(o[t, h]^2) + eps) * w[h * D + i] * silu(gate[t, h * D + i]); one wave a
// (token, head).
template <typename TO>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const float* __restrict__ gate, float eps,
                                                             TO* __restrict__ out, int H, int D) {
  const long base = ((long)blockIdx.x * H + blockIdx.y) * D;
  const int wbase = blockIdx.y * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += 64) {
    const float x = o[base + i];
    ss += x * x;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += 64) {
    const float g = gate[base + i];
    out[base + i] = from_f32<TO>(o[base + i] * inv * w[wbase + i] * (g / (1.0f + expf(-g))));
  }
}

extern "C" int gl3_head_norm_gate(const float* o, const float* w, const float* gate, float eps, void* out, int out_dtype,
                                  int n_tokens, int H, int D, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(o && w && gate && out && n_tokens > 0 && H > 0 && H <= 65535 && D > 0, "gl3_head_norm_gate: bad arguments");
  dim3 grid(n_tokens, H), block(64);
  if (out_dtype == GL3_F32) head_norm_gate_kernel<float><<<grid, block, 0, stream>>>(o, w, gate, eps, (float*)out, H, D);
  else if (out_dtype == GL3_BF16) head_norm_gate_kernel<bf16_t><<<grid, block, 0, stream>>>(o, w, gate, eps, (bf16_t*)out, H, D);
  else GL3_REQUIRE(false, "gl3_head_norm_gate: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- two score maps' outputs into one
// att [T][ld_a]: head h's output under the first map at column 2 h D, under the second at (2 h + 1) D. out [T][ld_o],
// head h at h * D: o = a1 - lambda a2, divided by its root mean square over the head's `dim` elements (eps inside
// the root; elements behind them are padding and hold zeros), times `mult`. One wave a (token, head). The maps'
// outputs may come in 32-bit where the result takes the activations' type.
template <typename TI, typename T>
__global__ __launch_bounds__(64) void diff_combine_kernel(const TI* __restrict__ att, long ld_a, T* __restrict__ out, long ld_o,
                                                           int H, int D, int dim, float lambda, float eps, float mult) {
  const long t = blockIdx.x;
  const int h = blockIdx.y;
  const TI* a1 = att + t * ld_a + (long)2 * h * D;
  const TI* a2 = a1 + D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < dim; i += 64) {
    const float o = to_f32<TI>(a1[i]) - lambda * to_f32<TI>(a2[i]);
    ss += o * o;
  }
  const float f = mult / sqrtf(wave_sum(ss) / (float)dim + eps);
  T* op = out + t * ld_o + (long)h * D;
  for (int i = threadIdx.x; i < D; i += 64) op[i] = from_f32<T>((to_f32<TI>(a1[i]) - lambda * to_f32<TI>(a2[i])) * f);
}

extern "C" int gl3_diff_combine(const void* att, int in_dtype, long ld_a, void* out, long ld_o, int dtype, int n_tokens, int H,
                                int D, int dim, float lambda, float eps, float mult, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(att && out && n_tokens > 0 && H > 0 && H <= 65535 && D > 0 && dim > 0 && dim <= D && ld_a >= 2L * H * D &&
                  ld_o >= (long)H * D,
              "gl3_diff_combine: %d heads of %d (%d used) in rows of %ld and %ld", H, D, dim, ld_a, ld_o);
  const dim3 grid(n_tokens, H), block(64);
  if (in_dtype == GL3_F32 && dtype == GL3_F32)
    diff_combine_kernel<float, float><<<grid, block, 0, stream>>>((const float*)att, ld_a, (float*)out, ld_o, H, D, dim, lambda, eps, mult);
  else if (in_dtype == GL3_BF16 && dtype == GL3_BF16)
    diff_combine_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)att, ld_a, (bf16_t*)out, ld_o, H, D, dim, lambda, eps, mult);
  else if (in_dtype == GL3_F32 && dtype == GL3_BF16)
    diff_combine_kernel<float, bf16_t><<<grid, block, 0, stream>>>((const float*)att, ld_a, (bf16_t*)out, ld_o, H, D, dim, lambda, eps, mult);
  else GL3_REQUIRE(false, "gl3_diff_combine: dtypes %d -> %d are not built", in_dtype, dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}
