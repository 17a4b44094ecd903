// Mixers that carry a state of fixed size from token to token, and the short causal convolution in front of them.
//
//   short_conv         y_t[c] = act(bias[c] + sum_j w[c][j] u_(t - taps + 1 + j)[c]) over each sequence's own tokens; the
//                      last taps - 1 inputs of a sequence are kept in its state row, so a step goes on where the last
//                      one stopped (zeros before a sequence's first token: a fresh state row is zero)
//   state_space_scan   a scalar decay a head:   S <- exp(-exp(A) dt) S + dt B x^T,  y = S^T C + D x      (S: N x P)
//   channel_delta_scan a decay for every key channel and the delta rule:
//                      S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q                 (S: D x P)
//   diff_heads         two softmax maps over the same values, o = rms_norm(a1 - lambda a2) (1 - c)
//
// Everything here is 32-bit FMA: inputs are the float sums of the projections, states are float.  The scans walk a
// sequence's tokens in order; what runs side by side is (sequence, head, columns of the state): a wave holds some columns
// of a head's state in registers, several lanes a column, each with its share of the rows.  A workgroup's waves (64
// columns of one head) share the token's vectors, which are staged through LDS up to 32 tokens at a time; the next
// tokens' vectors are asked for from memory before this chunk's tokens are walked.
#include "common.h"

#define RC_MAX_TAPS 16
#define RC_TB 32            // the most tokens staged at a time (fewer where LDS would not hold them)
#define RC_ROWS_MAX 256     // rows of a head's state (N of the state space, key size of the delta rule)

__device__ __forceinline__ float rc_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float rc_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------- short causal convolution
// u: float rows of u_stride values (columns of a fused projection); state [rows][taps - 1][C]; out [N][C].
// One thread a (token, channel).  A sequence's tokens lie one after another, so the input `back` tokens earlier is
// `back` rows up, or, before the step's first token, in the state.
__global__ void __launch_bounds__(256)
short_conv_kernel(const float* __restrict__ u, int u_stride, const float* __restrict__ w, const float* __restrict__ bias,
                  int act, const float* __restrict__ state, int state_rows, const int* __restrict__ tok_seq,
                  const int* __restrict__ tok_pos, const int* __restrict__ seq_past, const int* __restrict__ seq_slot,
                  float* __restrict__ out, int N, int C, int taps) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x, n = blockIdx.x;     // (tokens along x: any number of them)
  if (c >= C) return;
  const int seq = tok_seq[n], in_step = tok_pos[n] - seq_past[seq];       // new tokens of the sequence before this one
  int slot = seq_slot[seq];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const float* st = state + (size_t)slot * (taps - 1) * C;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    const float v = back <= in_step ? u[(size_t)(n - back) * u_stride + c] : st[(size_t)(taps - 1 - (back - in_step)) * C + c];
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  out[(size_t)n * C + c] = act ? rc_silu(acc) : acc;
}

// The state after the step: the last taps - 1 inputs of (old state, the step's inputs).  One thread a (sequence,
// channel) reads what it keeps before it writes.
__global__ void __launch_bounds__(256)
short_conv_state_kernel(const float* __restrict__ u, int u_stride, float* __restrict__ state, int state_rows,
                        const int* __restrict__ seq_start, const int* __restrict__ seq_slot, int C, int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
  if (c >= C) return;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int s0 = seq_start[b], n_new = seq_start[b + 1] - s0, keep = taps - 1;
  float* st = state + (size_t)slot * keep * C;
  float v[RC_MAX_TAPS];
#pragma unroll
  for (int i = 0; i < RC_MAX_TAPS; ++i) {
    if (i < keep) {
      const int from_end = keep - i;            // the value that ends up in place i is this many inputs from the end
      v[i] = from_end <= n_new ? u[(size_t)(s0 + n_new - from_end) * u_stride + c] : st[(size_t)(i + n_new) * C + c];
    }
  }
#pragma unroll
  for (int i = 0; i < RC_MAX_TAPS; ++i)
    if (i < keep) st[(size_t)i * C + c] = v[i];
}

// Single tokens (every sequence of the step brings one): output and the state's shift in one pass, one thread a
// (sequence, channel), which reads what it needs before it writes.
__global__ void __launch_bounds__(256)
short_conv_single_kernel(const float* __restrict__ u, int u_stride, const float* __restrict__ w, const float* __restrict__ bias,
                         int act, float* __restrict__ state, int state_rows, const int* __restrict__ seq_start,
                         const int* __restrict__ seq_slot, float* __restrict__ out, int C, int taps) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x, b = blockIdx.x;
  if (c >= C) return;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int n = seq_start[b], keep = taps - 1;
  float* st = state + (size_t)slot * keep * C;
  const float now = u[(size_t)n * u_stride + c];
  float v[RC_MAX_TAPS];
  float acc = bias ? bias[c] : 0.f;
#pragma unroll
  for (int i = 0; i < RC_MAX_TAPS; ++i)
    if (i < keep) {
      v[i] = st[(size_t)i * C + c];
      acc = fmaf(w[(size_t)c * taps + i], v[i], acc);
    }
  acc = fmaf(w[(size_t)c * taps + keep], now, acc);
  out[(size_t)n * C + c] = act ? rc_silu(acc) : acc;
#pragma unroll
  for (int i = 0; i < RC_MAX_TAPS; ++i)
    if (i < keep) st[(size_t)i * C + c] = i + 1 < keep ? v[i + 1 < RC_MAX_TAPS ? i + 1 : i] : now;
}

SYN_EXPORT int syn_short_conv(const float* u, int u_stride, const float* w, const float* bias, int act, float* state,
                              int state_rows, const int* tok_seq, const int* tok_pos, const int* seq_start,
                              const int* seq_past, const int* seq_slot, float* out, int n_tokens, int n_seqs, int C,
                              int taps, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && n_seqs > 0 && C > 0, "short_conv: empty input");
  SYN_CHECK(taps >= 1 && taps <= RC_MAX_TAPS, "short_conv: %d taps (1 to %d)", taps, RC_MAX_TAPS);
  SYN_CHECK(u_stride >= C && state_rows > 0, "short_conv: rows of %d values for %d channels", u_stride, C);
  const int bx = (C + 255) / 256;
  if (n_tokens == n_seqs) {      // (a step brings at least one token for each of its sequences: here exactly one)
    short_conv_single_kernel<<<dim3(n_seqs, bx), 256, 0, stream>>>(u, u_stride, w, bias, act, state, state_rows, seq_start,
                                                                  seq_slot, out, C, taps);
    SYN_LAUNCH_CHECK("short_conv_single");
    return 0;
  }
  short_conv_kernel<<<dim3(n_tokens, bx), 256, 0, stream>>>(u, u_stride, w, bias, act, state, state_rows, tok_seq, tok_pos,
                                                           seq_past, seq_slot, out, n_tokens, C, taps);
  SYN_LAUNCH_CHECK("short_conv");
  if (taps > 1) {
    short_conv_state_kernel<<<dim3(bx, n_seqs), 256, 0, stream>>>(u, u_stride, state, state_rows, seq_start, seq_slot, C, taps);
    SYN_LAUNCH_CHECK("short_conv_state");
  }
  return 0;
}

// ---------------------------------------------------------------- what the two scans share
// A wave holds 64 / SL columns of a head's state, SL lanes a column (SL = 4 or 16 slices), and a lane holds the rows
// slice * R .. slice * R + R - 1 of its column (R = rows / SL rounded up to a multiple of 4; rows beyond the state's are
// zeros that stay zeros).
//   SL = 4:  lane = 16 * slice + column.  The state is read and written in pieces of 64 bytes: for single tokens, where
//            the state is all that moves.
//   SL = 16: lane = slice + 16 * column.  A token's chain of operations is a quarter as long, there are four times as many
//            waves, and the sum over a column's slices stays inside a row of 16 lanes (four DPP additions, no trip through
//            LDS): for prompts, whose tokens come one after another and wait for one another.
// A token's vectors over the rows lie in LDS as SL pieces of R values, each followed by four unused ones, so that the
// slices' 16-byte reads spread over the banks and no read needs a bound.
#define RC_LD(R, SL) ((SL) * ((R) + 4))
#define RC_LDS_BUDGET (60 * 1024)
#define RC_PF(R) ((R) <= 8 ? 8 : 4)   // row values (each of two vectors) that a thread of the state space's scan holds of the next chunk
#define RC_PFX 2     // column values likewise
#define RC_TPW 2     // tokens that a wave of the delta rule's scan holds of the next chunk
__device__ __forceinline__ int rc_at(int n, int R) { return (n / R) * (R + 4) + n % R; }
template <int CTRL>
__device__ __forceinline__ float rc_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
// the sum over the lanes that hold a column's slices, in all of them
template <int SL>
__device__ __forceinline__ float rc_sum_slices(float v) {
  if constexpr (SL == 16) {
    v += rc_dpp<0xB1>(v);       // lanes 1 0 3 2 of every four
    v += rc_dpp<0x4E>(v);       // lanes 2 3 0 1
    v += rc_dpp<0x141>(v);      // the other four of every eight (mirrored)
    v += rc_dpp<0x140>(v);      // the other eight of the row (mirrored)
  } else {
#pragma unroll
    for (int off = 64 / SL; off < SYN_WAVE; off <<= 1) v += __shfl_xor(v, off, SYN_WAVE);
  }
  return v;
}
template <int SL> __device__ __forceinline__ int rc_slice(int lane) { return SL == 16 ? lane % 16 : lane / (64 / SL); }
template <int SL> __device__ __forceinline__ int rc_col(int lane) { return SL == 16 ? lane / 16 : lane % (64 / SL); }

// How many of a head's columns a workgroup takes (64, 32 or 16): a token's work for one head is bounded by what one
// compute unit issues, so a prompt's heads are spread over as many compute units as there are (their workgroups then
// stage the same row vectors each for itself); single tokens keep 64.
static int rc_block_columns(long heads, int cols, int longest) {
  if (longest <= 1) return 64;
  const long units = syn_compute_units();
  for (int cb = 64; cb > 16; cb /= 2)
    if (heads * ((cols + cb - 1) / cb) >= units) return cb;
  return 16;
}
// Four slices a wave (a lane then does four times the rows for the same overhead a token) also for prompts, where the
// chip has two waves a SIMD even so.
static bool rc_few_slices(long heads, int cols) { return heads * ((cols + 15) / 16) >= 8L * syn_compute_units(); }

// ---------------------------------------------------------------- state space with a scalar decay a head
// xbc [N][inner + 2 G Ns] float: x (H x P), B (G x Ns), C (G x Ns) behind the convolution; dt: float rows of dt_stride
// values, one a head, before bias and softplus; state [rows][H][Ns][P]; y [N][H * P] float (D x included).
template <int R, int SL>
__global__ void __launch_bounds__(64 * SL)
state_space_scan_kernel(const float* __restrict__ xbc, const float* __restrict__ dt, int dt_stride,
                        const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                        float* __restrict__ state, int state_rows, const int* __restrict__ seq_start,
                        const int* __restrict__ seq_slot, float* __restrict__ y, int H, int P, int Ns, int G, int tb_max) {
  constexpr int LD = RC_LD(R, SL), COLS = 64 / SL;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* Bs = lds;                          // [tb_max][LD]
  float* Cs = Bs + tb_max * LD;             // [tb_max][LD]
  float* xs = Cs + tb_max * LD;             // [tb_max][64]   dt * x of the workgroup's columns
  float* xr = xs + tb_max * 64;             // [tb_max][64]   x itself
  float* dec = xr + tb_max * 64;            // [tb_max]
  const int CB = blockDim.x / SYN_WAVE * (64 / SL);      // columns of this workgroup
  const int head = blockIdx.x, b = blockIdx.y, p0 = blockIdx.z * CB;
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, slice = rc_slice<SL>(lane);
  const int mine = wave * COLS + rc_col<SL>(lane), p = p0 + mine;       // this lane's column: of the workgroup's 64, of the head
  const bool col_ok = p < P;
  const int s0 = seq_start[b], n_new = seq_start[b + 1] - s0;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int inner = H * P, width = inner + 2 * G * Ns, grp = head / (H / G);
  float* S = state + ((size_t)slot * H + head) * Ns * P;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice * R + i;
    s[i] = (col_ok && n < Ns) ? S[(size_t)n * P + p] : 0.f;
  }
  const float A = -expf(a_log[head]), bias = dt_bias[head], D = d_skip[head];
  // a chunk's values on their way from memory: asked for while the chunk before is walked (the host keeps a chunk within
  // RC_PF(R) row values and RC_PFX column values a thread)
  float pb[RC_PF(R)], pc[RC_PF(R)], px[RC_PFX], pd[RC_PFX];
  auto fetch = [&](int t0) {
    const int tb = min(tb_max, n_new - t0);
#pragma unroll
    for (int j = 0; j < RC_PF(R); ++j) {
      const int e = tid + j * blockDim.x, t = e / (SL * R), n = e % (SL * R);
      pb[j] = pc[j] = 0.f;
      if (e < tb * SL * R && n < Ns) {
        const float* row = xbc + (size_t)(s0 + t0 + t) * width + inner + grp * Ns;
        pb[j] = row[n];
        pc[j] = row[G * Ns + n];
      }
    }
#pragma unroll
    for (int j = 0; j < RC_PFX; ++j) {
      const int e = tid + j * blockDim.x, t = e / CB, pp = p0 + e % CB;
      px[j] = pd[j] = 0.f;
      if (e < tb * CB) {
        const size_t tok = s0 + t0 + t;
        pd[j] = dt[tok * dt_stride + head];
        if (pp < P) px[j] = xbc[tok * width + head * P + pp];
      }
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n_new; t0 += tb_max) {
    const int tb = min(tb_max, n_new - t0);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < RC_PF(R); ++j) {
      const int e = tid + j * blockDim.x, t = e / (SL * R), n = e % (SL * R);
      if (e < tb * SL * R) {
        Bs[t * LD + rc_at(n, R)] = pb[j];
        Cs[t * LD + rc_at(n, R)] = pc[j];
      }
    }
#pragma unroll
    for (int j = 0; j < RC_PFX; ++j) {
      const int e = tid + j * blockDim.x;
      if (e < tb * CB) {
        const float step = rc_softplus(pd[j] + bias);
        const int at = (e / CB) * 64 + e % CB;
        xs[at] = step * px[j];
        xr[at] = px[j];
        if (e % CB == 0) dec[e / CB] = expf(A * step);
      }
    }
    __syncthreads();
    if (t0 + tb_max < n_new) fetch(t0 + tb_max);
#pragma unroll 2
    for (int t = 0; t < tb; ++t) {
      const float a = dec[t], bx = xs[t * 64 + mine];
      const float4* Bt = (const float4*)(Bs + t * LD + slice * (R + 4));
      const float4* Ct = (const float4*)(Cs + t * LD + slice * (R + 4));
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 bv = Bt[i / 4], cv = Ct[i / 4];
        s[i] = fmaf(a, s[i], bx * bv.x), acc[0] = fmaf(s[i], cv.x, acc[0]);
        s[i + 1] = fmaf(a, s[i + 1], bx * bv.y), acc[1] = fmaf(s[i + 1], cv.y, acc[1]);
        s[i + 2] = fmaf(a, s[i + 2], bx * bv.z), acc[2] = fmaf(s[i + 2], cv.z, acc[2]);
        s[i + 3] = fmaf(a, s[i + 3], bx * bv.w), acc[3] = fmaf(s[i + 3], cv.w, acc[3]);
      }
      const float sum = rc_sum_slices<SL>((acc[0] + acc[1]) + (acc[2] + acc[3]));
      if (slice == 0 && col_ok)
        y[(size_t)(s0 + t0 + t) * inner + head * P + p] = fmaf(D, xr[t * 64 + mine], sum);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice * R + i;
    if (col_ok && n < Ns) S[(size_t)n * P + p] = s[i];
  }
}

SYN_EXPORT int syn_state_space_scan(const float* xbc, const float* dt, int dt_stride, const float* dt_bias,
                                    const float* a_log, const float* d_skip, float* state, int state_rows,
                                    const int* seq_start, const int* seq_slot, int n_seqs, int longest, float* y, int H,
                                    int P, int Ns, int G, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && longest > 0 && H > 0 && P > 0 && Ns > 0 && G > 0, "state_space_scan: empty input");
  SYN_CHECK(H % G == 0, "state_space_scan: %d heads do not divide into %d groups", H, G);
  SYN_CHECK(Ns <= RC_ROWS_MAX, "state_space_scan: a state of %d rows (at most %d)", Ns, RC_ROWS_MAX);
  SYN_CHECK(dt_stride >= H && state_rows > 0, "state_space_scan: step rows of %d values for %d heads", dt_stride, H);
  const int block_cols = rc_block_columns((long)H * n_seqs, P, longest);
  // single tokens: four slices a wave (the state moves in pieces of 64 bytes); tokens in a row: sixteen
#define SYN_SS(R, SL)                                                                                                   \
  do {                                                                                                                  \
    const int per_token = (2 * RC_LD(R, SL) + 2 * 64 + 1) * (int)sizeof(float);                                         \
    const int waves = (min(P, block_cols) + 64 / SL - 1) / (64 / SL), cb = waves * (64 / SL);                           \
    const dim3 grid(H, n_seqs, (P + cb - 1) / cb);                                                                      \
    int tb = min(min(RC_TB, longest), RC_LDS_BUDGET / per_token);                                                       \
    tb = max(1, min(tb, min(RC_PF(R) * waves * SYN_WAVE / (SL * R), RC_PFX * waves * SYN_WAVE / cb)));                  \
    state_space_scan_kernel<R, SL><<<grid, waves * SYN_WAVE, (size_t)tb * per_token, stream>>>(                         \
        xbc, dt, dt_stride, dt_bias, a_log, d_skip, state, state_rows, seq_start, seq_slot, y, H, P, Ns, G, tb);        \
  } while (0)
  if (longest <= 1 || rc_few_slices((long)H * n_seqs, P)) {
    if (Ns <= 32) SYN_SS(8, 4);
    else if (Ns <= 64) SYN_SS(16, 4);
    else if (Ns <= 128) SYN_SS(32, 4);
    else SYN_SS(64, 4);
  } else {
    if (Ns <= 64) SYN_SS(4, 16);
    else if (Ns <= 128) SYN_SS(8, 16);
    else SYN_SS(16, 16);
  }
#undef SYN_SS
  SYN_LAUNCH_CHECK("state_space_scan");
  return 0;
}

// ---------------------------------------------------------------- delta rule with a decay for every key channel
// qkv [N][(2 K + H E)] float behind the convolution: q (K heads x D), k (K x D), v (H x E); beta: float rows, one a head,
// before the sigmoid; a: float rows of a_stride values, H * D of them used, before bias and softplus; state
// [rows][H][D][E]; o [N][H * E] float.
// Staged for each token: q and k as unit vectors (q also times q_scale), the decays, k . q.
template <int R, int SL>
__global__ void __launch_bounds__(64 * SL)
channel_delta_scan_kernel(const float* __restrict__ qkv, const float* __restrict__ beta, int beta_stride,
                          const float* __restrict__ a, int a_stride, const float* __restrict__ a_bias,
                          const float* __restrict__ a_log, float q_scale, float unit_eps, float* __restrict__ state,
                          int state_rows, const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
                          float* __restrict__ o, int H, int K, int D, int E, int tb_max) {
  constexpr int LD = RC_LD(R, SL), COLS = 64 / SL;
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                          // [tb_max][LD]
  float* ks = qs + tb_max * LD;             // [tb_max][LD]
  float* gs = ks + tb_max * LD;             // [tb_max][LD]
  float* vs = gs + tb_max * LD;             // [tb_max][64]
  float* kq = vs + tb_max * 64;             // [tb_max]
  float* bt = kq + tb_max;                  // [tb_max]
  const int CB = blockDim.x / SYN_WAVE * (64 / SL);      // columns of this workgroup
  const int head = blockIdx.x, b = blockIdx.y, p0 = blockIdx.z * CB;
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, slice = rc_slice<SL>(lane);
  const int n_waves = blockDim.x / SYN_WAVE;
  const int mine = wave * COLS + rc_col<SL>(lane), p = p0 + mine;
  const bool col_ok = p < E;
  const int s0 = seq_start[b], n_new = seq_start[b + 1] - s0;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int kvh = head / (H / K), width = 2 * K * D + H * E;
  float* S = state + ((size_t)slot * H + head) * D * E;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice * R + i;
    s[i] = (col_ok && n < D) ? S[(size_t)n * E + p] : 0.f;
  }
  const float A = -expf(a_log[head]);
  // a chunk's values on their way from memory: a wave stages the tokens wave, wave + n_waves (the host keeps a chunk within
  // RC_TPW tokens a wave), asked for while the chunk before is walked
  constexpr int DL = (SL * R + 63) / 64;
  float pq[RC_TPW][DL], pk[RC_TPW][DL], pa[RC_TPW][DL], pv[RC_TPW], pbeta[RC_TPW];
  auto fetch = [&](int t0) {
    const int tb = min(tb_max, n_new - t0);
#pragma unroll
    for (int j = 0; j < RC_TPW; ++j) {
      const int t = wave + j * n_waves;
      pv[j] = pbeta[j] = 0.f;
#pragma unroll
      for (int i = 0; i < DL; ++i) pq[j][i] = pk[j][i] = pa[j][i] = 0.f;
      if (t < tb) {
        const size_t tok = s0 + t0 + t;
        const float* qr = qkv + tok * width + kvh * D;
        const float* kr = qr + K * D;
#pragma unroll
        for (int i = 0; i < DL; ++i) {
          const int d = lane + 64 * i;
          if (d < D) {
            pq[j][i] = qr[d], pk[j][i] = kr[d];
            pa[j][i] = a[tok * (size_t)a_stride + head * D + d] + a_bias[head * D + d];
          }
        }
        if (lane < CB && p0 + lane < E) pv[j] = qkv[tok * width + 2 * K * D + head * E + p0 + lane];
        pbeta[j] = beta[tok * beta_stride + head];
      }
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n_new; t0 += tb_max) {
    const int tb = min(tb_max, n_new - t0);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < RC_TPW; ++j) {
      const int t = wave + j * n_waves;
      if (t < tb) {
        float sq = 0.f, sk = 0.f, dot = 0.f;
#pragma unroll
        for (int i = 0; i < DL; ++i)
          sq = fmaf(pq[j][i], pq[j][i], sq), sk = fmaf(pk[j][i], pk[j][i], sk), dot = fmaf(pq[j][i], pk[j][i], dot);
        sq = wave_sum(sq), sk = wave_sum(sk), dot = wave_sum(dot);
        const float iq = q_scale / sqrtf(sq + unit_eps), ik = 1.f / sqrtf(sk + unit_eps);
#pragma unroll
        for (int i = 0; i < DL; ++i) {      // (rows beyond the keys: zeros, and a decay of one)
          const int d = lane + 64 * i;
          if (d < SL * R) {
            const int at = t * LD + rc_at(d, R);
            qs[at] = pq[j][i] * iq;
            ks[at] = pk[j][i] * ik;
            gs[at] = d < D ? expf(A * rc_softplus(pa[j][i])) : 1.f;
          }
        }
        if (lane == 0) {
          kq[t] = dot * iq * ik;
          bt[t] = 1.f / (1.f + expf(-pbeta[j]));
        }
        vs[t * 64 + lane] = pv[j];
      }
    }
    __syncthreads();
    if (t0 + tb_max < n_new) fetch(t0 + tb_max);
#pragma unroll 1
    for (int t = 0; t < tb; ++t) {
      const float4* qt = (const float4*)(qs + t * LD + slice * (R + 4));
      const float4* kt = (const float4*)(ks + t * LD + slice * (R + 4));
      const float4* gt = (const float4*)(gs + t * LD + slice * (R + 4));
      float rk[4] = {0.f, 0.f, 0.f, 0.f}, rq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 gv = gt[i / 4], kv = kt[i / 4], qv = qt[i / 4];
        s[i] *= gv.x, rk[0] = fmaf(s[i], kv.x, rk[0]), rq[0] = fmaf(s[i], qv.x, rq[0]);
        s[i + 1] *= gv.y, rk[1] = fmaf(s[i + 1], kv.y, rk[1]), rq[1] = fmaf(s[i + 1], qv.y, rq[1]);
        s[i + 2] *= gv.z, rk[2] = fmaf(s[i + 2], kv.z, rk[2]), rq[2] = fmaf(s[i + 2], qv.z, rq[2]);
        s[i + 3] *= gv.w, rk[3] = fmaf(s[i + 3], kv.w, rk[3]), rq[3] = fmaf(s[i + 3], qv.w, rq[3]);
      }
      const float rks = rc_sum_slices<SL>((rk[0] + rk[1]) + (rk[2] + rk[3]));
      const float rqs = rc_sum_slices<SL>((rq[0] + rq[1]) + (rq[2] + rq[3]));
      const float u = bt[t] * (vs[t * 64 + mine] - rks);
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 kv = kt[i / 4];
        s[i] = fmaf(kv.x, u, s[i]), s[i + 1] = fmaf(kv.y, u, s[i + 1]);
        s[i + 2] = fmaf(kv.z, u, s[i + 2]), s[i + 3] = fmaf(kv.w, u, s[i + 3]);
      }
      // the read-out sees this token's write: (S + k u^T)^T q = S^T q + u (k . q)
      if (slice == 0 && col_ok) o[(size_t)(s0 + t0 + t) * H * E + head * E + p] = fmaf(u, kq[t], rqs);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice * R + i;
    if (col_ok && n < D) S[(size_t)n * E + p] = s[i];
  }
}

SYN_EXPORT int syn_channel_delta_scan(const float* qkv, const float* beta, int beta_stride, const float* a, int a_stride,
                                      const float* a_bias, const float* a_log, float q_scale, float unit_eps, float* state,
                                      int state_rows, const int* seq_start, const int* seq_slot, int n_seqs, int longest,
                                      float* o, int H, int K, int D, int E, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && longest > 0 && H > 0 && K > 0 && D > 0 && E > 0, "channel_delta_scan: empty input");
  SYN_CHECK(H % K == 0, "channel_delta_scan: %d heads do not divide into %d key heads", H, K);
  SYN_CHECK(D <= RC_ROWS_MAX, "channel_delta_scan: keys of %d values (at most %d)", D, RC_ROWS_MAX);
  SYN_CHECK(beta_stride >= H && state_rows > 0, "channel_delta_scan: rows of %d values for %d heads", beta_stride, H);
  SYN_CHECK(a_stride >= H * D, "channel_delta_scan: decay rows of %d values for %d heads of %d", a_stride, H, D);
  // (always 64 columns a workgroup: staging a token here means norms and decays, which workgroups that split a head's
  // columns would each do again; measured at 32 heads over 2,048 tokens: 1.18 ms with 64 columns, 1.46 ms with 16)
  const int block_cols = 64;
#define SYN_CD(R, SL)                                                                                                   \
  do {                                                                                                                  \
    const int per_token = (3 * RC_LD(R, SL) + 64 + 2) * (int)sizeof(float);                                             \
    const int waves = (min(E, block_cols) + 64 / SL - 1) / (64 / SL), cb = waves * (64 / SL);                           \
    const dim3 grid(H, n_seqs, (E + cb - 1) / cb);                                                                      \
    const int tb = max(1, min(min(min(RC_TB, longest), RC_LDS_BUDGET / per_token), RC_TPW * waves));                    \
    channel_delta_scan_kernel<R, SL><<<grid, waves * SYN_WAVE, (size_t)tb * per_token, stream>>>(                       \
        qkv, beta, beta_stride, a, a_stride, a_bias, a_log, q_scale, unit_eps, state, state_rows, seq_start, seq_slot,  \
        o, H, K, D, E, tb);                                                                                             \
  } while (0)
  if (longest <= 1 || rc_few_slices((long)H * n_seqs, E)) {
    if (D <= 32) SYN_CD(8, 4);
    else if (D <= 64) SYN_CD(16, 4);
    else if (D <= 128) SYN_CD(32, 4);
    else SYN_CD(64, 4);
  } else {
    if (D <= 64) SYN_CD(4, 16);
    else if (D <= 128) SYN_CD(8, 16);
    else SYN_CD(16, 16);
  }
#undef SYN_CD
  SYN_LAUNCH_CHECK("channel_delta_scan");
  return 0;
}

// ---------------------------------------------------------------- two softmax maps over the same values
// a [N][G][2][Rq][E]: for each kv head the heads' results of the first map, then of the second (the order in which
// grouped-query attention over 2 G key heads leaves them); out [N][G * Rq][E] = rms_norm(a1 - lambda a2) * post.
// One wave a (token, head).
template <typename T>
__global__ void diff_heads_kernel(const T* __restrict__ a, T* __restrict__ out, float lambda, float eps, float post,
                                  int n_items, int G, int Rq, int E) {
  const int item = blockIdx.x * (blockDim.x / SYN_WAVE) + threadIdx.x / SYN_WAVE;
  if (item >= n_items) return;
  const int lane = threadIdx.x % SYN_WAVE;
  const int H = G * Rq, tok = item / H, h = item % H, g = h / Rq, r = h % Rq;
  const T* a1 = a + (((size_t)tok * G + g) * 2 * Rq + r) * E;
  const T* a2 = a1 + (size_t)Rq * E;
  float ss = 0.f;
  for (int d = lane; d < E; d += SYN_WAVE) {
    const float v = to_f32<T>(a1[d]) - lambda * to_f32<T>(a2[d]);
    ss = fmaf(v, v, ss);
  }
  const float f = post / sqrtf(wave_sum(ss) / (float)E + eps);
  for (int d = lane; d < E; d += SYN_WAVE)
    out[((size_t)tok * H + h) * E + d] = from_f32<T>((to_f32<T>(a1[d]) - lambda * to_f32<T>(a2[d])) * f);
}

SYN_EXPORT int syn_diff_heads(const void* a, void* out, int is_f32, float lambda, float eps, float post, int n_tokens, int G,
                              int Rq, int E, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && G > 0 && Rq > 0 && E > 0, "diff_heads: empty input");
  const int wpb = 4, items = n_tokens * G * Rq, grid = (items + wpb - 1) / wpb;
  if (is_f32)
    diff_heads_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>((const float*)a, (float*)out, lambda, eps, post, items, G, Rq, E);
  else
    diff_heads_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>((const bf16*)a, (bf16*)out, lambda, eps, post, items, G, Rq, E);
  SYN_LAUNCH_CHECK("diff_heads");
  return 0;
}
