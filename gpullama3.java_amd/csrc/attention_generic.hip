// Causal grouped-query attention over the paged cache for any head size up to
// 256, any number of heads and groups, float or bfloat16 storage, all arithmetic
// in 32-bit: the true 32-bit path and the fallback of the matrix-core kernels.
//
// One wave per (token, query head). Query head h reads kv head h / (H/K)
// (J/inference/InferenceCore.java:116-119). Keys lo..p are visited in chunks of 64
// that start at lo, one key per lane; score = dot(q, k) * scale with
// scale = 1/sqrt(head_dim) (:122); softmax with the running maximum
// (:128, FloatTensor.java:211-219 computes the same with the global maximum); the
// values are summed with the weights (:134-144). The chunking depends on the
// query's position alone, so a token's result is the same bit for bit whether it
// arrives with its whole prompt or alone.
//
// What other decoders ask of the same loop, all optional: values of another size than the keys
// (v_head_dim); a bias that grows with the distance, score - slopes[h] * (p - key), one slope per
// query head; and a sink, a key that every query sees with the score `sink` and whose value is
// zero, so that the weights of the real keys sum to less than one: exp(s_j) / (exp(sink) + sum exp(s)).
// The sink is the running softmax's starting point (maximum = sink, sum = 1). And a window that keeps a sequence's
// first keys visible (keep_first): query p sees key j <= p if p - j < window or j < keep_first. A chunked mask (chunk > 0, no
// window): query p sees key j <= p only if j / chunk == p / chunk. And fewer value heads than key heads (n_v): several
// score maps over the same values. With maps = n_kv / n_v, query heads and key heads lie head by head as [map 0, map 1,
// ...]: query head h is map h % maps of head h / maps, which reads key head g * maps + h % maps and value head g, g the
// head's group. The sink may be a number per query head (sinks). And values that are a part of the keys (v_in_k >= 0): a
// cache with one array per position, whose elements v_in_k .. v_in_k + v_head_dim are the values (an attention over
// cached latents); heads of up to 1024 elements then (MAXHS 1024: more registers, so a kernel of its own).
#include "common.h"

#define ATT_MAX_HS 256

template <typename T, typename TO, int MAXHS>
__global__ __launch_bounds__(64) void attention_generic_kernel(
    const T* __restrict__ q, long q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ positions, const int* __restrict__ seq_of_token, const int* __restrict__ block_table,
    int table_stride, TO* __restrict__ out, long out_stride, int n_heads, int n_kv, int head_dim, int v_head_dim,
    int page_size, int window, float scale, const float* __restrict__ slopes, int has_sink, float sink, int keep_first,
    int chunk, int n_v, const float* __restrict__ sinks, int v_in_k) {
  __shared__ float qs[MAXHS];
  __shared__ float ps[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int p = positions[t];
  const int maps = n_kv / n_v;
  const int cv = (h / maps) / ((n_heads / maps) / n_v);
  const int c = cv * maps + h % maps;
  const int* bt = block_table + (long)seq_of_token[t] * table_stride;
  const int lo = chunk > 0 ? (p / chunk) * chunk : (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const T* qp = q + (long)t * q_stride + (long)h * head_dim;
  for (int i = lane; i < head_dim; i += 64) qs[i] = to_f32<T>(qp[i]);
  __syncthreads();
  const float slope = slopes ? slopes[h] : 0.f;
  if (sinks) {
    has_sink = 1;
    sink = sinks[h];
  }
  float m = has_sink ? sink : -INFINITY, l = has_sink ? 1.f : 0.f;
  float acc[MAXHS / 64] = {};
  // with a window, the sequence's first keep_first keys stay visible: those of them that lie before the window are
  // visited first, in chunks of their own, then the window's keys
  const int kept = keep_first < lo ? keep_first : lo;
  for (int run = kept > 0 ? 0 : 1; run < 2; ++run) {
  const int from = run == 0 ? 0 : lo, to = run == 0 ? kept - 1 : p;
  for (int base = from; base <= to; base += 64) {
    const int key = base + lane;
    const bool valid = key <= to;
    float s = -INFINITY;
    if (valid) {
      const T* kp = k_cache + ((long)bt[key / page_size] * n_kv + c) * page_size * head_dim;
      const int in_page = key % page_size;
      float dot = 0.f;
      for (int i = 0; i < head_dim; ++i) dot = fmaf(qs[i], to_f32<T>(kp[gl3_k_offset(in_page, i, head_dim)]), dot);
      s = dot * scale - slope * (float)(p - key);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float pe = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(pe);
    __syncthreads();
    ps[lane] = pe;
    __syncthreads();
    const int n_valid = (to - base + 1 < 64) ? to - base + 1 : 64;
#pragma unroll
    for (int r = 0; r < MAXHS / 64; ++r) acc[r] *= alpha;
    for (int j = 0; j < n_valid; ++j) {
      const int kj = base + j;
      const int in_page = kj % page_size;
      const float w = ps[j];
      if (v_in_k >= 0) {
        // the values are elements of the key rows themselves
        const T* kp = k_cache + ((long)bt[kj / page_size] * n_kv + c) * page_size * head_dim;
#pragma unroll
        for (int r = 0; r < MAXHS / 64; ++r) {
          const int i = lane + 64 * r;
          if (i < v_head_dim) acc[r] = fmaf(w, to_f32<T>(kp[gl3_k_offset(in_page, v_in_k + i, head_dim)]), acc[r]);
        }
        continue;
      }
      // values lie transposed in a page: [head_dim][position in page], in tiles
      const T* vp = v_cache + ((long)bt[kj / page_size] * n_v + cv) * page_size * v_head_dim;
#pragma unroll
      for (int r = 0; r < MAXHS / 64; ++r) {
        const int i = lane + 64 * r;
        if (i < v_head_dim) acc[r] = fmaf(w, to_f32<T>(vp[gl3_v_offset(i, in_page, page_size)]), acc[r]);
      }
    }
    m = m_new;
  }
  }
  TO* op = out + (long)t * out_stride + (long)h * v_head_dim;
#pragma unroll
  for (int r = 0; r < MAXHS / 64; ++r) {
    const int i = lane + 64 * r;
    if (i < v_head_dim) op[i] = from_f32<TO>(acc[r] / l);
  }
}

extern "C" int gl3_attention_generic(const void* q, long q_stride, const void* k_cache, const void* v_cache, int dtype,
                                     const int* positions, const int* seq_of_token, const int* block_table,
                                     int table_stride, void* out, long out_stride, int n_tokens, int n_heads, int n_kv,
                                     int head_dim, int page_size, int window, float scale, int v_head_dim,
                                     const float* slopes, int has_sink, float sink, int keep_first, int chunk, int n_v,
                                     int out_dtype, const float* sinks, int v_in_k, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(q && k_cache && (v_cache || v_in_k >= 0) && positions && seq_of_token && block_table && out,
              "gl3_attention_generic: null argument");
  GL3_REQUIRE(n_tokens > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0,
              "gl3_attention_generic: %d heads over %d kv heads", n_heads, n_kv);
  const int most = v_in_k >= 0 ? 1024 : ATT_MAX_HS;
  GL3_REQUIRE(head_dim > 0 && head_dim <= most, "gl3_attention_generic: head_dim %d exceeds %d", head_dim, most);
  GL3_REQUIRE(v_head_dim > 0 && v_head_dim <= most && (v_head_dim % 16 == 0 || v_in_k >= 0),
              "gl3_attention_generic: v_head_dim %d is not a multiple of 16 up to %d", v_head_dim, most);
  GL3_REQUIRE(v_in_k < 0 || (v_in_k + v_head_dim <= head_dim && n_v == n_kv),
              "gl3_attention_generic: values of %d from element %d of keys of %d", v_head_dim, v_in_k, head_dim);
  GL3_REQUIRE(n_heads <= 65535, "gl3_attention_generic: %d heads exceed the grid", n_heads);
  GL3_REQUIRE(page_size > 0 && table_stride > 0, "gl3_attention_generic: bad paging");
  GL3_REQUIRE(keep_first >= 0 && (keep_first == 0 || window > 0), "gl3_attention_generic: %d kept first keys without a window", keep_first);
  GL3_REQUIRE(chunk >= 0 && (chunk == 0 || window == 0), "gl3_attention_generic: a chunked mask has no window");
  GL3_REQUIRE(n_v > 0 && n_kv % n_v == 0 && n_heads % (n_kv / n_v) == 0 && (n_heads / (n_kv / n_v)) % n_v == 0,
              "gl3_attention_generic: %d heads, %d key heads, %d value heads", n_heads, n_kv, n_v);
  GL3_REQUIRE(page_size % 32 == 0 && head_dim % 16 == 0,
              "gl3_attention_generic: the cache lies in tiles: page_size %d must be a multiple of 32, head_dim %d of 16", page_size,
              head_dim);
  dim3 grid(n_tokens, n_heads), block(64);
#define ATT_GENERIC_OF(T, TO, MAXHS)                                                                                   \
  attention_generic_kernel<T, TO, MAXHS><<<grid, block, 0, stream>>>(                                                  \
      (const T*)q, q_stride, (const T*)k_cache, (const T*)v_cache, positions, seq_of_token, block_table, table_stride, \
      (TO*)out, out_stride, n_heads, n_kv, head_dim, v_head_dim, page_size, window, scale, slopes, has_sink, sink,     \
      keep_first, chunk, n_v, sinks, v_in_k)
#define ATT_GENERIC(T, TO)                                                       \
  do {                                                                           \
    if (head_dim <= ATT_MAX_HS && v_head_dim <= ATT_MAX_HS) ATT_GENERIC_OF(T, TO, ATT_MAX_HS); \
    else ATT_GENERIC_OF(T, TO, 1024);                                            \
  } while (0)
  // (the output in 32-bit beside 16-bit operands: for a caller that goes on in 32-bit with the heads' outputs)
  if (dtype == GL3_F32 && out_dtype == GL3_F32) ATT_GENERIC(float, float);
  else if (dtype == GL3_BF16 && out_dtype == GL3_BF16) ATT_GENERIC(bf16_t, bf16_t);
  else if (dtype == GL3_BF16 && out_dtype == GL3_F32) ATT_GENERIC(bf16_t, float);
  else GL3_REQUIRE(false, "gl3_attention_generic: dtypes %d -> %d are not built", dtype, out_dtype);
#undef ATT_GENERIC
#undef ATT_GENERIC_OF
  GL3_LAUNCH_CHECK();
  return 0;
}
