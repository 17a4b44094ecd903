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
// sequence's tokens in order; what runs side by side is (sequence, head, tile of 16 state columns): a wave holds 16
// columns of a head's state in registers, four lanes a column, each with every fourth row.  A workgroup's waves (up to
// four tiles of one head) share the token's vectors, which are staged through LDS sixteen tokens at a time.
#include "common.h"

#define RC_MAX_TAPS 16
#define RC_TB 16            // tokens staged at a time
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
  const int c = blockIdx.x * blockDim.x + threadIdx.x, n = blockIdx.y;
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

SYN_EXPORT int syn_short_conv(const float* u, int u_stride, const float* w, const float* bias, int act, float* state,
                              int state_rows, const int* tok_seq, const int* tok_pos, const int* seq_start,
                              const int* seq_past, const int* seq_slot, float* out, int n_tokens, int n_seqs, int C,
                              int taps, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && n_seqs > 0 && C > 0, "short_conv: empty input");
  SYN_CHECK(taps >= 1 && taps <= RC_MAX_TAPS, "short_conv: %d taps (1 to %d)", taps, RC_MAX_TAPS);
  SYN_CHECK(u_stride >= C && state_rows > 0, "short_conv: rows of %d values for %d channels", u_stride, C);
  const int bx = (C + 255) / 256;
  short_conv_kernel<<<dim3(bx, n_tokens), 256, 0, stream>>>(u, u_stride, w, bias, act, state, state_rows, tok_seq, tok_pos,
                                                           seq_past, seq_slot, out, n_tokens, C, taps);
  SYN_LAUNCH_CHECK("short_conv");
  if (taps > 1) {
    short_conv_state_kernel<<<dim3(bx, n_seqs), 256, 0, stream>>>(u, u_stride, state, state_rows, seq_start, seq_slot, C, taps);
    SYN_LAUNCH_CHECK("short_conv_state");
  }
  return 0;
}

// ---------------------------------------------------------------- what the two scans share
// lane = 16 * slice + column: the lane holds rows slice, slice + 4, ... of its column; R = rows / 4 rounded up
__device__ __forceinline__ float rc_sum_slices(float v) {
  v += __shfl_xor(v, 16, SYN_WAVE);
  v += __shfl_xor(v, 32, SYN_WAVE);
  return v;
}

// ---------------------------------------------------------------- state space with a scalar decay a head
// xbc [N][inner + 2 G Ns] float: x (H x P), B (G x Ns), C (G x Ns) behind the convolution; dt: float rows of dt_stride
// values, one a head, before bias and softplus; state [rows][H][Ns][P]; y [N][H * P] float (D x included).
template <int R>
__global__ void __launch_bounds__(256)
state_space_scan_kernel(const float* __restrict__ xbc, const float* __restrict__ dt, int dt_stride,
                        const float* __restrict__ dt_bias, const float* __restrict__ a_log, const float* __restrict__ d_skip,
                        float* __restrict__ state, int state_rows, const int* __restrict__ seq_start,
                        const int* __restrict__ seq_slot, float* __restrict__ y, int H, int P, int Ns, int G) {
  extern __shared__ float lds[];
  float* Bs = lds;                          // [RC_TB][Ns]
  float* Cs = Bs + RC_TB * Ns;              // [RC_TB][Ns]
  float* xs = Cs + RC_TB * Ns;              // [RC_TB][64]   dt * x of the workgroup's columns
  float* xr = xs + RC_TB * 64;              // [RC_TB][64]   x itself
  float* dec = xr + RC_TB * 64;             // [RC_TB]
  const int head = blockIdx.x, b = blockIdx.y, p0 = blockIdx.z * 64;
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, slice = lane / 16;
  const int p = p0 + wave * 16 + lane % 16;
  const bool col_ok = p < P;
  const int s0 = seq_start[b], n_new = seq_start[b + 1] - s0;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int inner = H * P, width = inner + 2 * G * Ns, grp = head / (H / G);
  float* S = state + ((size_t)slot * H + head) * Ns * P;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice + 4 * i;
    s[i] = (col_ok && n < Ns) ? S[(size_t)n * P + p] : 0.f;
  }
  const float A = -expf(a_log[head]), bias = dt_bias[head], D = d_skip[head];
  for (int t0 = 0; t0 < n_new; t0 += RC_TB) {
    const int tb = min(RC_TB, n_new - t0);
    __syncthreads();
    for (int e = tid; e < tb * Ns; e += blockDim.x) {
      const int t = e / Ns, n = e % Ns;
      const float* row = xbc + (size_t)(s0 + t0 + t) * width + inner + grp * Ns;
      Bs[e] = row[n];
      Cs[e] = row[G * Ns + n];
    }
    for (int e = tid; e < tb * 64; e += blockDim.x) {
      const int t = e / 64, pp = p0 + e % 64;
      const size_t tok = s0 + t0 + t;
      const float step = rc_softplus(dt[tok * dt_stride + head] + bias);
      const float x = pp < P ? xbc[tok * width + head * P + pp] : 0.f;
      xs[e] = step * x;
      xr[e] = x;
      if (e % 64 == 0) dec[t] = expf(A * step);
    }
    __syncthreads();
    for (int t = 0; t < tb; ++t) {
      const float a = dec[t], bx = xs[t * 64 + wave * 16 + lane % 16];
      const float* Bt = Bs + t * Ns;
      const float* Ct = Cs + t * Ns;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int n = slice + 4 * i;
        if (n < Ns) {
          s[i] = fmaf(a, s[i], bx * Bt[n]);
          acc = fmaf(s[i], Ct[n], acc);
        }
      }
      acc = rc_sum_slices(acc);
      if (slice == 0 && col_ok)
        y[(size_t)(s0 + t0 + t) * inner + head * P + p] = fmaf(D, xr[t * 64 + wave * 16 + lane % 16], acc);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice + 4 * i;
    if (col_ok && n < Ns) S[(size_t)n * P + p] = s[i];
  }
}

SYN_EXPORT int syn_state_space_scan(const float* xbc, const float* dt, int dt_stride, const float* dt_bias,
                                    const float* a_log, const float* d_skip, float* state, int state_rows,
                                    const int* seq_start, const int* seq_slot, int n_seqs, float* y, int H, int P, int Ns,
                                    int G, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && H > 0 && P > 0 && Ns > 0 && G > 0, "state_space_scan: empty input");
  SYN_CHECK(H % G == 0, "state_space_scan: %d heads do not divide into %d groups", H, G);
  SYN_CHECK(Ns <= RC_ROWS_MAX, "state_space_scan: a state of %d rows (at most %d)", Ns, RC_ROWS_MAX);
  SYN_CHECK(dt_stride >= H && state_rows > 0, "state_space_scan: step rows of %d values for %d heads", dt_stride, H);
  const int waves = min(4, (P + 15) / 16);
  const dim3 grid(H, n_seqs, (P + 63) / 64);
  const size_t lds = (size_t)(2 * RC_TB * Ns + 2 * RC_TB * 64 + RC_TB) * sizeof(float);
#define SYN_SS(R)                                                                                                     \
  state_space_scan_kernel<R><<<grid, waves * SYN_WAVE, lds, stream>>>(xbc, dt, dt_stride, dt_bias, a_log, d_skip, state, \
                                                                      state_rows, seq_start, seq_slot, y, H, P, Ns, G)
  if (Ns <= 64) SYN_SS(16);
  else if (Ns <= 128) SYN_SS(32);
  else SYN_SS(64);
#undef SYN_SS
  SYN_LAUNCH_CHECK("state_space_scan");
  return 0;
}

// ---------------------------------------------------------------- delta rule with a decay for every key channel
// qkv [N][(2 K + H E)] float behind the convolution: q (K heads x D), k (K x D), v (H x E); beta: float rows, one a head,
// before the sigmoid; a: float rows of a_stride values, H * D of them used, before bias and softplus; state [rows][H][D][E]; o [N][H * E] float.
// Staged for each token: q and k as unit vectors (q also times q_scale), the decays, k . q.
template <int R>
__global__ void __launch_bounds__(256)
channel_delta_scan_kernel(const float* __restrict__ qkv, const float* __restrict__ beta, int beta_stride,
                          const float* __restrict__ a, int a_stride, const float* __restrict__ a_bias,
                          const float* __restrict__ a_log, float q_scale, float unit_eps, float* __restrict__ state, int state_rows,
                          const int* __restrict__ seq_start, const int* __restrict__ seq_slot, float* __restrict__ o,
                          int H, int K, int D, int E) {
  extern __shared__ float lds[];
  float* qs = lds;                          // [RC_TB][D]
  float* ks = qs + RC_TB * D;               // [RC_TB][D]
  float* gs = ks + RC_TB * D;               // [RC_TB][D]
  float* vs = gs + RC_TB * D;               // [RC_TB][64]
  float* kq = vs + RC_TB * 64;              // [RC_TB]
  float* bt = kq + RC_TB;                   // [RC_TB]
  const int head = blockIdx.x, b = blockIdx.y, p0 = blockIdx.z * 64;
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, slice = lane / 16;
  const int n_waves = blockDim.x / SYN_WAVE;
  const int p = p0 + wave * 16 + lane % 16;
  const bool col_ok = p < E;
  const int s0 = seq_start[b], n_new = seq_start[b + 1] - s0;
  int slot = seq_slot[b];
  if (slot < 0 || slot >= state_rows) slot = state_rows - 1;
  const int kvh = head / (H / K), width = 2 * K * D + H * E;
  float* S = state + ((size_t)slot * H + head) * D * E;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice + 4 * i;
    s[i] = (col_ok && n < D) ? S[(size_t)n * E + p] : 0.f;
  }
  const float A = -expf(a_log[head]);
  for (int t0 = 0; t0 < n_new; t0 += RC_TB) {
    const int tb = min(RC_TB, n_new - t0);
    __syncthreads();
    for (int t = wave; t < tb; t += n_waves) {
      const size_t tok = s0 + t0 + t;
      const float* qr = qkv + tok * width + kvh * D;
      const float* kr = qr + K * D;
      float sq = 0.f, sk = 0.f, dot = 0.f;
      for (int d = lane; d < D; d += SYN_WAVE) {
        const float qv = qr[d], kv = kr[d];
        sq = fmaf(qv, qv, sq), sk = fmaf(kv, kv, sk), dot = fmaf(qv, kv, dot);
      }
      sq = wave_sum(sq), sk = wave_sum(sk), dot = wave_sum(dot);
      const float iq = q_scale / sqrtf(sq + unit_eps), ik = 1.f / sqrtf(sk + unit_eps);
      for (int d = lane; d < D; d += SYN_WAVE) {
        qs[t * D + d] = qr[d] * iq;
        ks[t * D + d] = kr[d] * ik;
        gs[t * D + d] = expf(A * rc_softplus(a[tok * (size_t)a_stride + head * D + d] + a_bias[head * D + d]));
      }
      if (lane == 0) {
        kq[t] = dot * iq * ik;
        bt[t] = 1.f / (1.f + expf(-beta[tok * beta_stride + head]));
      }
      {
        const int pp = p0 + lane;
        vs[t * 64 + lane] = pp < E ? qkv[tok * width + 2 * K * D + head * E + pp] : 0.f;
      }
    }
    __syncthreads();
    for (int t = 0; t < tb; ++t) {
      const float* qt = qs + t * D;
      const float* kt = ks + t * D;
      const float* gt = gs + t * D;
      float rk = 0.f, rq = 0.f;
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int n = slice + 4 * i;
        if (n < D) {
          s[i] *= gt[n];
          rk = fmaf(s[i], kt[n], rk);
          rq = fmaf(s[i], qt[n], rq);
        }
      }
      rk = rc_sum_slices(rk), rq = rc_sum_slices(rq);
      const float u = bt[t] * (vs[t * 64 + wave * 16 + lane % 16] - rk);
#pragma unroll
      for (int i = 0; i < R; ++i) {
        const int n = slice + 4 * i;
        if (n < D) s[i] = fmaf(kt[n], u, s[i]);
      }
      // the read-out sees this token's write: (S + k u^T)^T q = S^T q + u (k . q)
      if (slice == 0 && col_ok) o[(size_t)(s0 + t0 + t) * H * E + head * E + p] = fmaf(u, kq[t], rq);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = slice + 4 * i;
    if (col_ok && n < D) S[(size_t)n * E + p] = s[i];
  }
}

SYN_EXPORT int syn_channel_delta_scan(const float* qkv, const float* beta, int beta_stride, const float* a, int a_stride,
                                      const float* a_bias, const float* a_log, float q_scale, float unit_eps, float* state,
                                      int state_rows, const int* seq_start, const int* seq_slot, int n_seqs, float* o, int H,
                                      int K, int D, int E, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && H > 0 && K > 0 && D > 0 && E > 0, "channel_delta_scan: empty input");
  SYN_CHECK(H % K == 0, "channel_delta_scan: %d heads do not divide into %d key heads", H, K);
  SYN_CHECK(D <= RC_ROWS_MAX, "channel_delta_scan: keys of %d values (at most %d)", D, RC_ROWS_MAX);
  SYN_CHECK(beta_stride >= H && state_rows > 0, "channel_delta_scan: rows of %d values for %d heads", beta_stride, H);
  SYN_CHECK(a_stride >= H * D, "channel_delta_scan: decay rows of %d values for %d heads of %d", a_stride, H, D);
  const int waves = min(4, (E + 15) / 16);
  const dim3 grid(H, n_seqs, (E + 63) / 64);
  const size_t lds = (size_t)(3 * RC_TB * D + RC_TB * 64 + 2 * RC_TB) * sizeof(float);
#define SYN_CD(R)                                                                                                       \
  channel_delta_scan_kernel<R><<<grid, waves * SYN_WAVE, lds, stream>>>(qkv, beta, beta_stride, a, a_stride, a_bias, a_log, q_scale, \
                                                                        unit_eps, state, state_rows, seq_start, seq_slot, \
                                                                        o, H, K, D, E)
  if (D <= 64) SYN_CD(16);
  else if (D <= 128) SYN_CD(32);
  else SYN_CD(64);
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
