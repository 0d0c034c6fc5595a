// Recurrences with a matrix per head and a scalar decay: the state space's and the retention's.
//
//   S <- a S + b k v^T,   o = S^T q          S [N, P] in 32-bit per (sequence, head)
//
// a and b are numbers per (token, head) or per head; q and k may be shared by several heads (a group). A selective
// state space is k = B, q = C, v = x, a = exp(-exp(A_log) dt), b = dt; a retention is a = the head's decay, b = N^-1/2.
// Around it: the short causal convolution with silu that the state space's x, B and C pass, with the last taps - 1
// inputs of every sequence kept in its slot; the decays and step sizes; and the read-outs' gate and unit norm.
// Everything here is 32-bit arithmetic with accurate exp; only the last kernel's output takes the activations' type.
// Every kernel walks a step's tokens in order from what the slot holds, and no sum depends on what else is in the
// batch, so any cut of a sequence into steps gives the same numbers (a long step's recurrence runs in pieces joined
// through their start states: the same numbers up to 32-bit rounding).
#include "common.h"

// ----------------------------------------------------------------- convolution, decays and step sizes
// proj: [T][ld] float, the convolution's inputs from column col_x on (`channels` of them), dt from column col_dt on
// (`heads`). state: [slot][state_ld], the held inputs from state_off on as [taps - 1][channels], oldest first.
// act [T][channels] = silu(conv + bias); ab [T][2 * heads] = (exp(-exp(A_log) dt), dt), dt = softplus(dt + dt_bias).
// grid (T, blocks of 256 channels + blocks of 256 heads).
__global__ __launch_bounds__(256) void ssm_prep_kernel(const float* __restrict__ proj, long ld, int col_x, int channels,
                                                        int col_dt, int heads, const float* __restrict__ conv_w,
                                                        const float* __restrict__ conv_b, int taps,
                                                        const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                                                        const float* __restrict__ state, long state_ld, long state_off,
                                                        const int* __restrict__ cu_seqlens, const int* __restrict__ seq_of_token,
                                                        const int* __restrict__ slot_ids, float* __restrict__ act,
                                                        float* __restrict__ ab, int conv_blocks) {
  const int t = blockIdx.x;
  if ((int)blockIdx.y >= conv_blocks) {
    const int h = (blockIdx.y - conv_blocks) * 256 + threadIdx.x;
    if (h >= heads) return;
    const float z = proj[(long)t * ld + col_dt + h] + dt_bias[h];
    const float dt = z > 20.f ? z + log1pf(expf(-z)) : log1pf(expf(z));
    ab[(long)t * 2 * heads + h] = expf(-expf(A_log[h]) * dt);
    ab[(long)t * 2 * heads + heads + h] = dt;
    return;
  }
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int s = seq_of_token[t];
  const int first = cu_seqlens[s], i = t - first;
  const float* held = state + (long)slot_ids[s] * state_ld + state_off;
  float sum = conv_b ? conv_b[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int li = i - (taps - 1 - j);
    const float v = li >= 0 ? proj[(long)(first + li) * ld + col_x + c] : held[(long)(taps - 1 + li) * channels + c];
    sum = fmaf(conv_w[(long)c * taps + j], v, sum);
  }
  act[(long)t * channels + c] = sum / (1.0f + expf(-sum));
}

// The held inputs move on: after a step of n tokens a sequence holds its last taps - 1 inputs. grid (B, blocks of 256 channels)
#define SSM_MAX_TAPS 16
__global__ __launch_bounds__(256) void ssm_hold_kernel(const float* __restrict__ proj, long ld, int col_x, int channels, int taps,
                                                        float* __restrict__ state, long state_ld, long state_off,
                                                        const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids) {
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= channels) return;
  const int first = cu_seqlens[s], n = cu_seqlens[s + 1] - first;
  float* held = state + (long)slot_ids[s] * state_ld + state_off;
  float keep[SSM_MAX_TAPS];
#pragma unroll
  for (int r = 0; r < SSM_MAX_TAPS; ++r) {
    if (r < taps - 1) {
      const int li = n - (taps - 1) + r;
      keep[r] = li >= 0 ? proj[(long)(first + li) * ld + col_x + c] : held[(long)(taps - 1 + li) * channels + c];
    }
  }
#pragma unroll
  for (int r = 0; r < SSM_MAX_TAPS; ++r)
    if (r < taps - 1) held[(long)r * channels + c] = keep[r];
}

extern "C" int gl3_ssm_prep(const float* proj, long ld, int n_tokens, int n_seqs, int col_x, int channels, int col_dt, int heads,
                            const float* conv_w, const float* conv_b, int taps, const float* A_log, const float* dt_bias,
                            float* state, long state_ld, long state_off, const int* cu_seqlens, const int* seq_of_token,
                            const int* slot_ids, float* act, float* ab, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(proj && conv_w && A_log && dt_bias && state && cu_seqlens && seq_of_token && slot_ids && act && ab,
              "gl3_ssm_prep: null argument");
  GL3_REQUIRE(n_tokens > 0 && n_seqs > 0 && n_seqs <= 65535 && channels > 0 && heads > 0 && taps >= 1 && taps <= SSM_MAX_TAPS,
              "gl3_ssm_prep: %d tokens, %d sequences, %d channels, %d heads, %d taps (at most %d)", n_tokens, n_seqs, channels,
              heads, taps, SSM_MAX_TAPS);
  GL3_REQUIRE(col_x >= 0 && col_x + channels <= ld && col_dt >= 0 && col_dt + heads <= ld &&
                  state_off >= 0 && state_off + (long)(taps - 1) * channels <= state_ld,
              "gl3_ssm_prep: columns %d+%d, %d+%d of rows of %ld; state %ld+%ld of %ld", col_x, channels, col_dt, heads, ld,
              state_off, (long)(taps - 1) * channels, state_ld);
  const int conv_blocks = (channels + 255) / 256, head_blocks = (heads + 255) / 256;
  ssm_prep_kernel<<<dim3(n_tokens, conv_blocks + head_blocks), dim3(256), 0, stream>>>(
      proj, ld, col_x, channels, col_dt, heads, conv_w, conv_b, taps, A_log, dt_bias, state, state_ld, state_off, cu_seqlens,
      seq_of_token, slot_ids, act, ab, conv_blocks);
  GL3_LAUNCH_CHECK();
  if (taps > 1) {
    ssm_hold_kernel<<<dim3(n_seqs, conv_blocks), dim3(256), 0, stream>>>(proj, ld, col_x, channels, taps, state, state_ld,
                                                                         state_off, cu_seqlens, slot_ids);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// ----------------------------------------------------------------- the recurrence
// One block a (sequence, head, tile of up to 256 value columns). Thread (r, p) keeps rows r * NR .. of column p of S in
// registers; a round of tokens' q, k, v, a, b is staged through shared memory (rows of q and k padded with zeros to
// R * NR, so the inner loop has no conditions and reads four floats at a time); every thread adds its rows' part of a
// read-out, the parts of the R row groups are added in their order. The order of every sum depends on N, P and the
// launch shape alone (which follow from N and P).
//
// A long step is cut into pieces of `piece_len` tokens that run side by side (the recurrence is linear in S):
//   MODE 1  every piece but a sequence's last runs from S = 0 without read-outs and keeps its end state D_c and the
//           product A_c of its decays;
//   join    per sequence, piece after piece: the start state of piece c is kept where D_c was, S <- A_c S + D_c;
//   MODE 2  every piece runs from its start state with read-outs; a sequence's last piece leaves S in the slot.
// MODE 0 is a step in one piece, from the slot's state and back into it. How a step is cut follows from the launch
// (lengths and head count), never from the values, and changes a result by rounding alone.
struct ScanArgs {
  const float* q; long ld_q; int col_q;       // [T][ld_q], head group g at col_q + g * N
  const float* k; long ld_k; int col_k;
  const float* v; long ld_v; int col_v;       // head h at col_v + h * P
  const float* a_tok; const float* b_tok;     // [T][ld_ab] per token and head, or null
  long ld_ab;
  const float* a_head;                        // [H] when a_tok is null
  float b_const;                              // when b_tok is null
  float* state; long state_ld; long state_off;   // [slot][state_ld], S of head h at state_off + h * N * P as [N][P]
  const int* cu_seqlens; const int* slot_ids;
  float* out; long ld_o;                      // [T][ld_o], head h at h * P
  int H, heads_per_group, N, P, R, round;
  float* piece_state;                         // [sequence][piece][H][N][P]
  float* piece_decay;                         // [sequence][piece][H]
  int n_pieces, piece_len;
  int act;                                    // 1: q, k and v pass silu as they are read (a linear attention whose
                                              // projections carry an activation); 0: as they are
};

__device__ __forceinline__ float scan_in(float v, int act) { return act ? v / (1.0f + expf(-v)) : v; }

template <int NR, int MODE>
__global__ void decay_scan_kernel(ScanArgs A) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int s = MODE == 0 ? blockIdx.x : blockIdx.x / A.n_pieces, c = MODE == 0 ? 0 : blockIdx.x % A.n_pieces;
  const int h = blockIdx.y, g = h / A.heads_per_group;
  const int N = A.N, P = A.P, R = A.R, CH = A.round, NP = R * NR;
  const int first = A.cu_seqlens[s], n = A.cu_seqlens[s + 1] - first;
  const int lo = MODE == 0 ? 0 : c * A.piece_len;
  const int hi = MODE == 0 ? n : (n < lo + A.piece_len ? n : lo + A.piece_len);
  if (MODE != 0 && lo >= n) return;
  if (MODE == 1 && hi == n) return;                       // (a sequence's last piece is run once, with read-outs)
  const int pt = blockDim.x / R;                          // columns of this block's tile
  const int r = threadIdx.x / pt, pl = threadIdx.x % pt, p = blockIdx.z * pt + pl;
  const bool live = p < P;
  float* sq = smem;                       // [CH][NP]
  float* sk = sq + CH * NP;               // [CH][NP]
  float* sv = sk + CH * NP;               // [CH][pt]
  float* sa = sv + CH * pt;               // [CH]
  float* sb = sa + CH;                    // [CH]
  float* part = sb + CH;                  // [CH][R][pt]
  float* S = A.state + (long)A.slot_ids[s] * A.state_ld + A.state_off + (long)h * N * P;
  float* kept = MODE == 0 ? nullptr : A.piece_state + (((long)s * A.n_pieces + c) * A.H + h) * N * P;
  const float* from = MODE == 0 ? S : kept;
  const int n0 = r * NR;
  float acc[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) acc[i] = (MODE != 1 && live && n0 + i < N) ? from[(long)(n0 + i) * P + p] : 0.f;
  const float a_fixed = A.a_tok ? 0.f : A.a_head[h];
  float decays = 1.f;
  for (int base = lo; base < hi; base += CH) {
    const int m = hi - base < CH ? hi - base : CH;
    __syncthreads();
    for (int e = threadIdx.x; e < m * NP; e += blockDim.x) {
      const int j = e / NP, i = e % NP;
      const long t = first + base + j;
      sk[e] = i < N ? scan_in(A.k[t * A.ld_k + A.col_k + g * N + i], A.act) : 0.f;
      if (MODE != 1) sq[e] = i < N ? scan_in(A.q[t * A.ld_q + A.col_q + g * N + i], A.act) : 0.f;
    }
    for (int e = threadIdx.x; e < m * pt; e += blockDim.x) {
      const int j = e / pt, i = e % pt, col = blockIdx.z * pt + i;
      sv[j * pt + i] = col < P ? scan_in(A.v[(long)(first + base + j) * A.ld_v + A.col_v + h * P + col], A.act) : 0.f;
    }
    for (int j = threadIdx.x; j < m; j += blockDim.x) {
      const long t = first + base + j;
      sa[j] = A.a_tok ? A.a_tok[t * A.ld_ab + h] : a_fixed;
      sb[j] = A.b_tok ? A.b_tok[t * A.ld_ab + h] : A.b_const;
    }
    __syncthreads();
    for (int j = 0; j < m; ++j) {
      const float a = sa[j], bv = sb[j] * sv[j * pt + pl];
      const float4* kq = reinterpret_cast<const float4*>(sk + j * NP + n0);
      const float4* qq = reinterpret_cast<const float4*>(sq + j * NP + n0);
      if (MODE == 1) decays *= a;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < NR; i += 4) {
        const float4 kk = kq[i / 4];
        acc[i] = fmaf(a, acc[i], kk.x * bv);
        acc[i + 1] = fmaf(a, acc[i + 1], kk.y * bv);
        acc[i + 2] = fmaf(a, acc[i + 2], kk.z * bv);
        acc[i + 3] = fmaf(a, acc[i + 3], kk.w * bv);
        if (MODE != 1) {
          const float4 qv = qq[i / 4];
          o = fmaf(acc[i], qv.x, o);
          o = fmaf(acc[i + 1], qv.y, o);
          o = fmaf(acc[i + 2], qv.z, o);
          o = fmaf(acc[i + 3], qv.w, o);
        }
      }
      if (MODE != 1) part[(j * R + r) * pt + pl] = o;
    }
    if (MODE == 1) continue;
    __syncthreads();
    for (int e = threadIdx.x; e < m * pt; e += blockDim.x) {
      const int j = e / pt, i = e % pt, col = blockIdx.z * pt + i;
      float o = 0.f;
      for (int rr = 0; rr < R; ++rr) o += part[(j * R + rr) * pt + i];
      if (col < P) A.out[(long)(first + base + j) * A.ld_o + h * P + col] = o;
    }
  }
  if (MODE == 2 && hi != n) return;
  float* to = MODE == 1 ? kept : S;
#pragma unroll
  for (int i = 0; i < NR; ++i)
    if (live && n0 + i < N) to[(long)(n0 + i) * P + p] = acc[i];
  if (MODE == 1 && threadIdx.x == 0 && blockIdx.z == 0) A.piece_decay[((long)s * A.n_pieces + c) * A.H + h] = decays;
}

// The pieces' start states, sequence by sequence and piece after piece. grid (sequences, H, blocks of 256 elements of S)
__global__ __launch_bounds__(256) void decay_join_kernel(ScanArgs A) {
  const int s = blockIdx.x, h = blockIdx.y;
  const long NP = (long)A.N * A.P, e = (long)blockIdx.z * 256 + threadIdx.x;
  if (e >= NP) return;
  const int n = A.cu_seqlens[s + 1] - A.cu_seqlens[s];
  const int pieces = (n + A.piece_len - 1) / A.piece_len;
  float S = A.state[(long)A.slot_ids[s] * A.state_ld + A.state_off + (long)h * NP + e];
  for (int c = 0; c < pieces; ++c) {
    float* kept = A.piece_state + (((long)s * A.n_pieces + c) * A.H + h) * NP + e;
    if (c + 1 < pieces) {
      const float d = *kept;
      *kept = S;
      S = fmaf(A.piece_decay[((long)s * A.n_pieces + c) * A.H + h], S, d);
    } else {
      *kept = S;
    }
  }
}

// `pieces` (null: every step in one piece): room for n_seqs * n_pieces * H * (N * P + 1) floats; a step is cut when its
// longest sequence (max_len) gives at least two pieces of piece_len tokens.
extern "C" int gl3_decay_scan(const float* q, long ld_q, int col_q, const float* k, long ld_k, int col_k, const float* v,
                              long ld_v, int col_v, const float* a_tok, const float* b_tok, long ld_ab, const float* a_head,
                              float b_const, float* state, long state_ld, long state_off, const int* cu_seqlens,
                              const int* slot_ids, float* out, long ld_o, int n_seqs, int H, int heads_per_group, int N, int P,
                              float* pieces, long pieces_floats, int max_len, int piece_len, int act, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  GL3_REQUIRE(q && k && v && state && cu_seqlens && slot_ids && out && (a_tok || a_head), "gl3_decay_scan: null argument");
  GL3_REQUIRE(n_seqs > 0 && H > 0 && H <= 65535 && heads_per_group > 0 && H % heads_per_group == 0 && N > 0 && N <= 1024 && P > 0,
              "gl3_decay_scan: %d sequences, %d heads in groups of %d, keys of %d (at most 1024), values of %d", n_seqs, H,
              heads_per_group, N, P);
  const int groups = H / heads_per_group;
  GL3_REQUIRE(col_q >= 0 && col_q + (long)groups * N <= ld_q && col_k >= 0 && col_k + (long)groups * N <= ld_k && col_v >= 0 &&
                  col_v + (long)H * P <= ld_v && (long)H * P <= ld_o && (!(a_tok || b_tok) || ld_ab >= H) &&
                  state_off >= 0 && state_off + (long)H * N * P <= state_ld,
              "gl3_decay_scan: columns do not fit their rows, or the state its slot");
  // the tile of columns, the row groups and the rows a thread keeps
  const int pt = P >= 256 ? 256 : P;
  int R = 256 / pt;
  if (R > N) R = N;
  if (R < 1) R = 1;
  int nr = (N + R - 1) / R;
  while (nr > 64) {           // more rows than a thread keeps: more row groups
    R *= 2;
    nr = (N + R - 1) / R;
  }
  const int NRT = nr <= 8 ? 8 : nr <= 16 ? 16 : nr <= 32 ? 32 : 64;      // the rows a thread keeps: the kernel's template
  R = (N + NRT - 1) / NRT;
  GL3_REQUIRE(R * pt <= 1024, "gl3_decay_scan: keys of %d with values of %d need %d threads", N, P, R * pt);
  const int NP = R * NRT;
  int round = 16;
  auto bytes = [&](int ch) { return (size_t)(ch * (2 * NP + pt + 2) + ch * R * pt) * sizeof(float); };
  while (round > 1 && (bytes(round) > 60000 || (round * pt) % 4)) round /= 2;
  GL3_REQUIRE(bytes(round) <= 64000, "gl3_decay_scan: keys of %d with values of %d do not fit shared memory", N, P);
  ScanArgs A{q, ld_q, col_q, k, ld_k, col_k, v, ld_v, col_v, a_tok, b_tok, ld_ab, a_head, b_const, state, state_ld, state_off,
             cu_seqlens, slot_ids, out, ld_o, H, heads_per_group, N, P, R, round, nullptr, nullptr, 1, 0, act ? 1 : 0};
  const int ptiles = (P + pt - 1) / pt;
  const dim3 block(R * pt);
  const size_t sh = bytes(round);
#define SCAN_LAUNCH(MODE, grid)                                                          \
  do {                                                                                   \
    if (NRT == 8) decay_scan_kernel<8, MODE><<<grid, block, sh, stream>>>(A);            \
    else if (NRT == 16) decay_scan_kernel<16, MODE><<<grid, block, sh, stream>>>(A);     \
    else if (NRT == 32) decay_scan_kernel<32, MODE><<<grid, block, sh, stream>>>(A);     \
    else decay_scan_kernel<64, MODE><<<grid, block, sh, stream>>>(A);                    \
    GL3_LAUNCH_CHECK();                                                                  \
  } while (0)
  const int n_pieces = (pieces && piece_len > 0) ? (max_len + piece_len - 1) / piece_len : 1;
  if (n_pieces < 2) {
    SCAN_LAUNCH(0, dim3(n_seqs, H, ptiles));
    return 0;
  }
  const long rows = (long)n_seqs * n_pieces;
  GL3_REQUIRE(rows < (1L << 31) && rows * H * ((long)N * P + 1) <= pieces_floats,
              "gl3_decay_scan: %d sequences in %d pieces of %d heads need %ld floats, %ld given", n_seqs, n_pieces, H,
              rows * H * ((long)N * P + 1), pieces_floats);
  A.piece_state = pieces;
  A.piece_decay = pieces + rows * H * (long)N * P;
  A.n_pieces = n_pieces;
  A.piece_len = piece_len;
  const dim3 grid((unsigned)rows, H, ptiles);
  SCAN_LAUNCH(1, grid);
  decay_join_kernel<<<dim3(n_seqs, H, (unsigned)(((long)N * P + 255) / 256)), dim3(256), 0, stream>>>(A);
  GL3_LAUNCH_CHECK();
  SCAN_LAUNCH(2, grid);
#undef SCAN_LAUNCH
  return 0;
}

// ----------------------------------------------------------------- gate and unit norm of the read-outs
// y = o + skip_d[h] * skip_x (skip_d may be null); gate_first: y <- y * silu(gate) and then y / rms over each group of
// `gsize` channels; else y / rms and then times silu(gate). Times w[c] where w is given. One block a (token, group).
// o [T][C]; skip_x [T][ld_x] from col_x; gate [T][ld_g] from col_g; out [T][C] in the activations' type.
template <typename TO>
__global__ __launch_bounds__(256) void group_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ skip_x,
                                                               long ld_x, int col_x, const float* __restrict__ skip_d,
                                                               int head_dim, const float* __restrict__ gate, long ld_g,
                                                               int col_g, const float* __restrict__ w, float eps,
                                                               int gate_first, int C, int gsize, TO* __restrict__ out,
                                                               int gate_sigmoid) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const int c0 = blockIdx.y * gsize;
  float ss = 0.f;
  for (int i = threadIdx.x; i < gsize; i += blockDim.x) {
    const int c = c0 + i;
    float y = o[t * C + c];
    if (skip_d) y = fmaf(skip_d[c / head_dim], skip_x[t * ld_x + col_x + c], y);
    if (gate_first) {
      const float g = gate[t * ld_g + col_g + c];
      y *= (gate_sigmoid ? 1.0f : g) / (1.0f + expf(-g));
    }
    ss += y * y;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)gsize + eps);
  for (int i = threadIdx.x; i < gsize; i += blockDim.x) {
    const int c = c0 + i;
    float y = o[t * C + c];
    if (skip_d) y = fmaf(skip_d[c / head_dim], skip_x[t * ld_x + col_x + c], y);
    const float g = gate[t * ld_g + col_g + c];
    const float sg = (gate_sigmoid ? 1.0f : g) / (1.0f + expf(-g));      // silu of the gate, or its sigmoid
    y = gate_first ? y * sg * inv : y * inv * sg;
    if (w) y *= w[c];
    out[t * C + c] = from_f32<TO>(y);
  }
}

extern "C" int gl3_group_norm_gate(const float* o, const float* skip_x, long ld_x, int col_x, const float* skip_d, int head_dim,
                                   const float* gate, long ld_g, int col_g, const float* w, float eps, int gate_first,
                                   int n_tokens, int C, int gsize, void* out, int out_dtype, int gate_sigmoid,
                                   hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(o && gate && out && n_tokens > 0 && C > 0 && gsize > 0 && C % gsize == 0 && C / gsize <= 65535,
              "gl3_group_norm_gate: %d channels in groups of %d", C, gsize);
  GL3_REQUIRE(!skip_d || (skip_x && head_dim > 0 && C % head_dim == 0 && col_x >= 0 && col_x + C <= ld_x),
              "gl3_group_norm_gate: the skipped input's columns");
  GL3_REQUIRE(col_g >= 0 && col_g + C <= ld_g, "gl3_group_norm_gate: the gate's columns");
  const int threads = gsize >= 256 ? 256 : ((gsize + 63) / 64) * 64;
  const dim3 grid(n_tokens, C / gsize), block(threads);
  if (out_dtype == GL3_F32)
    group_norm_gate_kernel<float><<<grid, block, 0, stream>>>(o, skip_x, ld_x, col_x, skip_d, head_dim, gate, ld_g, col_g, w, eps,
                                                              gate_first, C, gsize, (float*)out, gate_sigmoid);
  else if (out_dtype == GL3_BF16)
    group_norm_gate_kernel<bf16_t><<<grid, block, 0, stream>>>(o, skip_x, ld_x, col_x, skip_d, head_dim, gate, ld_g, col_g, w, eps,
                                                               gate_first, C, gsize, (bf16_t*)out, gate_sigmoid);
  else GL3_REQUIRE(false, "gl3_group_norm_gate: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}
