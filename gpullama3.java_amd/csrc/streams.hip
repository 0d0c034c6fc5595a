// Several copies of the residual row per token ("streams"), mixed by learned numbers around every sublayer.
//
// rows [T][S][d] float: token t's S copies one after another. Around a sublayer with the numbers in[S], mix[S][S]
// (indexed [from][to]) and out[S]:
//   the sublayer reads  u = sum_s in[s] x_s          (through an RMS norm: h = u / sqrt(mean(u^2) + eps) * w)
//   and leaves          x_r <- sum_s mix[s][r] x_s + out[r] * y     for all r at once from the old copies.
// One kernel does both ends that meet between two sublayers: it takes the output y of the sublayer before (if any),
// writes the new copies, and makes the input h of the sublayer behind (if any) from them, so the copies make one
// trip to memory per sublayer. Everything is 32-bit arithmetic; h takes the activations' type. The sums run in the
// order of s, and a row's sum of squares in an order that the width alone fixes (whatever else is in the step).
#include "common.h"

#define STREAMS_MAX 16

// A block of NT threads (256 or 1024) works as 1,024 lanes, column c on lane c % 1024: a thread is R = 1024 / NT of
// them and keeps a partial sum of squares for each, a lane's sums run over its columns one after another, the lanes'
// over 64 at a time and then over the 16 groups in their order. So both block sizes give the same bits, and a step of
// few tokens (a handful of blocks, each waiting for its columns' trips to memory) takes the large one. MAXS bounds the
// copies that a thread keeps in registers (4 for the usual counts: 64 registers where 16 take 100).
template <typename TO, int NT, int MAXS>
__global__ __launch_bounds__(NT) void streams_step_kernel(float* __restrict__ rows, int S, int d,
                                                          const float* __restrict__ y, const float* __restrict__ mix,
                                                          const float* __restrict__ out_w,
                                                          const float* __restrict__ in_w,
                                                          const float* __restrict__ norm_w, float eps,
                                                          TO* __restrict__ h) {
  constexpr int R = 1024 / NT;
  extern __shared__ float u_row[];           // [d] the mixture that the next sublayer reads
  __shared__ float scratch[16];
  __shared__ float s_mix[MAXS * MAXS], s_out[MAXS], s_in[MAXS];
  const long t = blockIdx.x;
  if (threadIdx.x < S * S && y) s_mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    if (y) s_out[threadIdx.x] = out_w[threadIdx.x];
    if (in_w) s_in[threadIdx.x] = in_w[threadIdx.x];
  }
  __syncthreads();
  float* xr = rows + t * S * d;
  float ss[R];
#pragma unroll
  for (int r = 0; r < R; ++r) ss[r] = 0.f;
  for (int base = 0; base < d; base += 1024) {
    float x[R][MAXS], yv[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {            // (a thread's loads of one round are on their way together)
      const int c = base + r * NT + threadIdx.x;
#pragma unroll
      for (int s = 0; s < MAXS; ++s) x[r][s] = (s < S && c < d) ? xr[(long)s * d + c] : 0.f;
      yv[r] = (y && c < d) ? y[t * d + c] : 0.f;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int c = base + r * NT + threadIdx.x;
      if (c >= d) continue;
      if (y) {
        float nx[MAXS];
#pragma unroll
        for (int q = 0; q < MAXS; ++q) {
          if (q < S) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
              if (s < S) v = fmaf(s_mix[s * S + q], x[r][s], v);
            nx[q] = fmaf(s_out[q], yv[r], v);
          }
        }
#pragma unroll
        for (int q = 0; q < MAXS; ++q)
          if (q < S) {
            x[r][q] = nx[q];
            xr[(long)q * d + c] = nx[q];
          }
      }
      if (in_w) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
          if (s < S) v = fmaf(s_in[s], x[r][s], v);
        u_row[c] = v;
        ss[r] = fmaf(v, v, ss[r]);
      }
    }
  }
  if (!in_w) return;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const float w = wave_sum(ss[r]);
    if ((threadIdx.x & 63) == 0) scratch[(threadIdx.x >> 6) + (NT / 64) * r] = w;
  }
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) total += scratch[i];
  const float inv = 1.0f / sqrtf(total / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += NT) h[t * d + c] = from_f32<TO>(u_row[c] * inv * norm_w[c]);
}

// y null: nothing is added and the copies stay (the first sublayer of a step). in_w null: nothing is read (behind the
// last sublayer). norm_w: float [d].
extern "C" int gl3_streams_step(float* rows, int n_tokens, int S, int d, const float* y, const float* mix, const float* out_w,
                                const float* in_w, const float* norm_w, float eps, void* h, int h_dtype, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(rows && n_tokens > 0 && S >= 1 && S <= STREAMS_MAX && d > 0, "gl3_streams_step: %d tokens with %d copies (at most %d) of %d",
              n_tokens, S, STREAMS_MAX, d);
  GL3_REQUIRE(!y || (mix && out_w), "gl3_streams_step: a sublayer's output comes with the numbers that mix it in");
  GL3_REQUIRE(!in_w || (norm_w && h), "gl3_streams_step: the next sublayer's input needs its norm's weight and a place");
  GL3_REQUIRE(y || in_w, "gl3_streams_step: nothing to do");
  const size_t sh = in_w ? (size_t)d * sizeof(float) : 0;
  GL3_REQUIRE(sh <= 64000, "gl3_streams_step: rows of %d do not fit shared memory", d);
  const dim3 grid(n_tokens);
  const bool few = n_tokens <= 128 && d > 256;
#define ST_GO(TO, NT)                                                                                                   \
  do {                                                                                                                  \
    if (S <= 4) streams_step_kernel<TO, NT, 4><<<grid, dim3(NT), sh, stream>>>(rows, S, d, y, mix, out_w, in_w, norm_w, eps, (TO*)h); \
    else streams_step_kernel<TO, NT, STREAMS_MAX><<<grid, dim3(NT), sh, stream>>>(rows, S, d, y, mix, out_w, in_w, norm_w, eps,      \
                                                                                  (TO*)h);                              \
  } while (0)
  if (!in_w || h_dtype == GL3_F32) {
    if (few) ST_GO(float, 1024); else ST_GO(float, 256);
  } else if (h_dtype == GL3_BF16) {
    if (few) ST_GO(bf16_t, 1024); else ST_GO(bf16_t, 256);
  } else GL3_REQUIRE(false, "gl3_streams_step: unknown dtype %d", h_dtype);
#undef ST_GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// Every copy of a token's row takes the values of src [T][d] (a step's beginning: the embedding's output).
__global__ void streams_fill_kernel(const float* __restrict__ src, float* __restrict__ rows, int S, int d, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / d;
  const int c = i % d;
  const float v = src[i];
  for (int s = 0; s < S; ++s) rows[(t * S + s) * d + c] = v;
}

extern "C" int gl3_streams_fill(const float* src, float* rows, int n_tokens, int S, int d, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(src && rows && n_tokens > 0 && S >= 1 && d > 0, "gl3_streams_fill: bad arguments");
  const long n = (long)n_tokens * d;
  GL3_REQUIRE((n + 255) / 256 < (1L << 31), "gl3_streams_fill: too many elements");
  streams_fill_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(src, rows, S, d, n);
  GL3_LAUNCH_CHECK();
  return 0;
}

// out[r] = the sum of the copies of token which[r] (which null: token r), in the order of the copies.
__global__ void streams_sum_kernel(const float* __restrict__ rows, const int* __restrict__ which, int S, int d,
                                   float* __restrict__ out, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long r = i / d;
  const int c = i % d;
  const long t = which ? which[r] : r;
  float v = 0.f;
  for (int s = 0; s < S; ++s) v += rows[(t * S + s) * d + c];
  out[i] = v;
}

extern "C" int gl3_streams_sum(const float* rows, const int* which, int n_out, int S, int d, float* out, hipStream_t stream) {
  if (n_out == 0) return 0;
  GL3_REQUIRE(rows && out && n_out > 0 && S >= 1 && d > 0, "gl3_streams_sum: bad arguments");
  const long n = (long)n_out * d;
  GL3_REQUIRE((n + 255) / 256 < (1L << 31), "gl3_streams_sum: too many elements");
  streams_sum_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(rows, which, S, d, out, n);
  GL3_LAUNCH_CHECK();
  return 0;
}
