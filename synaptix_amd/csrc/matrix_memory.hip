// A matrix memory with exponential gates and a running maximum (the mLSTM cell), one state for each sequence and head:
//
//   i_t = cap tanh((i~ + b_i) / cap)                      log input gate   (cap <= 0: no cap)
//   f_t = logsigmoid(cap tanh((f~ + b_f) / cap))          log forget gate
//   m_t = max(f_t + m_(t-1), i_t)                         m_0 = 0
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T         S [dim][vdim], S_0 = 0
//   n_t = exp(f_t + m_(t-1) - m_t) n_(t-1) + exp(i_t - m_t) k_t               n [dim],       n_0 = 0
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),                   q_t = q~_t * q_scale
//
// All of it in 32-bit.  The state of a (slot, head) is dim * vdim + dim + 1 floats: S by rows, n, m.
// proj [N][width] float is the fused projection [q: H x dim | k: H x dim | v: H x vdim | gate: H x vdim | i~: H | f~: H].
#include "common.h"

#define MM_TC 16        // tokens whose q, k and gates are staged in LDS together
#define MM_VT 64        // columns of S a workgroup keeps (one a lane)
#define MM_DG 4         // waves of a workgroup; wave w keeps the rows d = w, w + 4, ... of its columns
#define MM_MAX_DIM 256

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One workgroup for each (sequence of the step, head); it walks the sequence's new tokens in order with 64 columns of S
// in registers, one tile of 64 columns after another.  n and m are read once, carried anew from there in every pass over
// a tile (the same values each time), and stored after the last: no other workgroup reads or writes this head's state.
template <int DPT>   // rows of S a thread keeps: dim <= 4 * DPT
__global__ void __launch_bounds__(MM_DG * SYN_WAVE)
matrix_memory_scan_kernel(const float* __restrict__ proj, int width, const float* __restrict__ i_bias,
                          const float* __restrict__ f_bias, float cap, float q_scale, float* __restrict__ state,
                          int spare_row, const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
                          float* __restrict__ out, int H, int dim, int vdim) {
  __shared__ float qs[MM_TC][MM_MAX_DIM];
  __shared__ float ks[MM_TC][MM_MAX_DIM];
  __shared__ float gs[MM_TC][2];
  __shared__ float red[2][MM_DG][MM_VT];
  __shared__ float red_n[2][MM_DG];
  const int b = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int t0 = seq_start[b], t1 = seq_start[b + 1];
  if (t0 >= t1) return;     // a sequence without tokens in this step (the spare ones of a padded step): nothing moves
  const int slot = seq_slot[b];
  const size_t per_head = (size_t)dim * vdim + dim + 1;
  float* st = state + ((size_t)(slot < 0 ? spare_row : slot) * H + h) * per_head;
  const int q_col = h * dim, k_col = H * dim + h * dim, v_col = 2 * H * dim + h * vdim;
  const int i_col = 2 * H * dim + 2 * H * vdim + h, f_col = i_col + H;
  const float bi = i_bias ? i_bias[h] : 0.f, bf = f_bias ? f_bias[h] : 0.f;
  const int dn = wave + MM_DG * lane;          // the entry of n this thread keeps
  const float n_before = dn < dim ? st[(size_t)dim * vdim + dn] : 0.f;
  const float m_before = st[(size_t)dim * vdim + dim];
  float n = n_before, m = m_before;

  for (int vt = 0; vt * MM_VT < vdim; ++vt) {
    const int v = vt * MM_VT + lane;
    const bool v_ok = v < vdim;
    n = n_before, m = m_before;
    float S[DPT];
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
      const int d = wave + MM_DG * j;
      S[j] = (d < dim && v_ok) ? st[(size_t)d * vdim + v] : 0.f;
    }
    for (int c0 = t0; c0 < t1; c0 += MM_TC) {
      const int nc = min(MM_TC, t1 - c0);
      __syncthreads();
      for (int idx = threadIdx.x; idx < nc * dim; idx += blockDim.x) {
        const int t = idx / dim, d = idx % dim;
        const float* row = proj + (size_t)(c0 + t) * width;
        qs[t][d] = row[q_col + d] * q_scale;
        ks[t][d] = row[k_col + d];
      }
      if (threadIdx.x < nc * 2) {
        const int t = threadIdx.x / 2, which = threadIdx.x % 2;
        const float raw = proj[(size_t)(c0 + t) * width + (which ? f_col : i_col)] + (which ? bf : bi);
        const float capped = cap > 0.f ? cap * tanhf(raw / cap) : raw;
        gs[t][which] = which ? log_sigmoid(capped) : capped;
      }
      float vv[MM_TC];
#pragma unroll
      for (int t = 0; t < MM_TC; ++t) vv[t] = (t < nc && v_ok) ? proj[(size_t)(c0 + t) * width + v_col + v] : 0.f;
      __syncthreads();
#pragma unroll
      for (int t = 0; t < MM_TC; ++t) {
        if (t < nc) {
          const float ig = gs[t][0], fg = gs[t][1];
          const float m_new = fmaxf(fg + m, ig);
          const float a = expf(fg + m - m_new), bb = expf(ig - m_new);
          m = m_new;
          float num = 0.f;
#pragma unroll
          for (int j = 0; j < DPT; ++j) {
            const int d = wave + MM_DG * j;
            if (d < dim) {
              S[j] = a * S[j] + (bb * ks[t][d]) * vv[t];
              num = fmaf(S[j], qs[t][d], num);
            }
          }
          float nq = 0.f;
          if (dn < dim) {
            n = a * n + bb * ks[t][dn];
            nq = n * qs[t][dn];
          }
          nq = wave_sum(nq);
          const int buf = t & 1;
          red[buf][wave][lane] = num;
          if (lane == 0) red_n[buf][wave] = nq;
          __syncthreads();
          if (wave == 0 && v_ok) {
            float total = 0.f, nqt = 0.f;
#pragma unroll
            for (int w = 0; w < MM_DG; ++w) total += red[buf][w][lane], nqt += red_n[buf][w];
            const float den = fmaxf(fabsf(nqt), expf(-m)) + 1e-6f;
            out[(size_t)(c0 + t) * H * vdim + (size_t)h * vdim + v] = total / den;
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
      const int d = wave + MM_DG * j;
      if (d < dim && v_ok) st[(size_t)d * vdim + v] = S[j];
    }
  }
  if (dn < dim) st[(size_t)dim * vdim + dn] = n;
  if (threadIdx.x == 0) st[(size_t)dim * vdim + dim] = m;
}

// The same cell for prompts, in chunks of MMC_L tokens that are worked on side by side.  Inside a chunk, with b_t the
// sum of f from the chunk's first token to t, a_s = i_s - b_s, P_t = max_(s <= t) a_s, and m_0, S_0, n_0 the state
// before the chunk:
//   m_t = b_t + M_t,  M_t = max(m_0, P_t)                                         (the recurrence of m, unrolled)
//   A[t][s] = (q_t . k_s) exp(a_s - M_t) for s <= t,   g_t = exp(m_0 - M_t)
//   S_t^T q_t = sum_s A[t][s] v_s + g_t S_0^T q_t,      n_t . q_t = sum_s A[t][s] + g_t n_0 . q_t
//   S_L = exp(m_0 - M_L) S_0 + exp(P_L - M_L) U,        U = sum_s exp(a_s - P_L) k_s v_s^T          (n likewise)
// Every exponent is at most 0, as in the step-by-step form; all sums are 32-bit FMA; b, a, P and M are kept in 64-bit
// inside the chunk (b grows to 32 log gates, and the exponents are small differences).  Three launches:
//   local: for every chunk U and its n-part, b_L and P_L           (chunks side by side)
//   carry: for every sequence, chunk after chunk: the state before each chunk is stored, then carried over it
//   out:   for every chunk its tokens' results from q, k, v and the state before it  (chunks side by side)
// Chunk c of the step is the c-th in the order of the sequences; a workgroup finds its sequence from seq_start.
#define MMC_L 32

struct ChunkWork {     // scratch of one call; `chunks` is the most chunks the step can have
  float* U;            // [chunks][H][dim][vdim]
  float* un;           // [chunks][H][dim]
  float* stat;         // [chunks][H][2]   b_L, P_L
  float* S0;           // [chunks][H][dim][vdim]  the state before the chunk
  float* n0;           // [chunks][H][dim]
  float* m0;           // [chunks][H]
  float* m_end;        // [sequences][H]  m behind a sequence's last chunk
};

// which sequence and which tokens chunk `c` of the step holds; false: there is no such chunk
__device__ __forceinline__ bool chunk_of(const int* __restrict__ seq_start, int n_seqs, int c, int& seq, int& first, int& count) {
  for (int b = 0; b < n_seqs; ++b) {
    const int s0 = seq_start[b], n = seq_start[b + 1] - s0, chunks = (n + MMC_L - 1) / MMC_L;
    if (c < chunks) {
      seq = b, first = s0 + c * MMC_L, count = min(MMC_L, n - c * MMC_L);
      return true;
    }
    c -= chunks;
  }
  return false;
}

// The gates of a chunk's tokens by one wave, a token a lane: b_t and a_t in 64-bit, P_t along the lanes.
struct ChunkGates {
  double b, a, P;      // of this lane's token (lanes beyond the chunk: a = -inf, b and P of the last token)
  float ig;
};
__device__ __forceinline__ ChunkGates chunk_gates(const float* __restrict__ proj, int width, int first, int nc, int lane,
                                                  int i_col, int f_col, float bi, float bf, float cap) {
  ChunkGates g;
  g.ig = -INFINITY;
  float fg = 0.f;
  if (lane < nc) {
    const float* row = proj + (size_t)(first + lane) * width;
    const float ri = row[i_col] + bi, rf = row[f_col] + bf;
    g.ig = cap > 0.f ? cap * tanhf(ri / cap) : ri;
    fg = log_sigmoid(cap > 0.f ? cap * tanhf(rf / cap) : rf);
  }
  g.b = fg;
#pragma unroll
  for (int off = 1; off < MMC_L; off <<= 1) {
    const double x = __shfl_up(g.b, off, SYN_WAVE);
    if (lane >= off) g.b += x;
  }
  g.a = lane < nc ? (double)g.ig - g.b : -INFINITY;
  g.P = g.a;
#pragma unroll
  for (int off = 1; off < MMC_L; off <<= 1) {
    const double x = __shfl_up(g.P, off, SYN_WAVE);
    if (lane >= off) g.P = fmax(g.P, x);
  }
  return g;
}

template <int DPT>   // rows of S a thread keeps: dim <= 4 * DPT
__global__ void __launch_bounds__(MM_DG * SYN_WAVE)
mm_chunk_local_kernel(const float* __restrict__ proj, int width, const float* __restrict__ i_bias,
                      const float* __restrict__ f_bias, float cap, const int* __restrict__ seq_start, int n_seqs,
                      ChunkWork work, int H, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int L = MMC_L;
  const int DP = dim + 1;
  float* ks = lds;                 // [L][DP]
  float* vs = ks + L * DP;         // [L][64]
  float* ws = vs + L * MM_VT;      // [L] exp(a_s - P_L)
  const int c = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
  int seq, first, nc;
  if (!chunk_of(seq_start, n_seqs, c, seq, first, nc)) return;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, tid = threadIdx.x;
  const int v = vt * MM_VT + lane;
  const int k_col = H * dim + h * dim, v_col = 2 * H * dim + h * vdim;
  const int i_col = 2 * H * dim + 2 * H * vdim + h, f_col = i_col + H;
  for (int idx = tid; idx < L * dim; idx += blockDim.x) {
    const int t = idx / dim, d = idx % dim;
    ks[t * DP + d] = t < nc ? proj[(size_t)(first + t) * width + k_col + d] : 0.f;
  }
  for (int idx = tid; idx < L * MM_VT; idx += blockDim.x) {
    const int t = idx / MM_VT, cc = idx % MM_VT;
    vs[idx] = (t < nc && vt * MM_VT + cc < vdim) ? proj[(size_t)(first + t) * width + v_col + vt * MM_VT + cc] : 0.f;
  }
  if (wave == 0) {
    const ChunkGates g = chunk_gates(proj, width, first, nc, lane, i_col, f_col, i_bias ? i_bias[h] : 0.f,
                                     f_bias ? f_bias[h] : 0.f, cap);
    const double PL = __shfl(g.P, nc - 1, SYN_WAVE), bL = __shfl(g.b, nc - 1, SYN_WAVE);
    if (lane < L) ws[lane] = lane < nc ? expf((float)(g.a - PL)) : 0.f;
    if (lane == 0 && vt == 0) {
      work.stat[((size_t)c * H + h) * 2] = (float)bL;
      work.stat[((size_t)c * H + h) * 2 + 1] = (float)PL;
    }
  }
  __syncthreads();
  float U[DPT];
#pragma unroll
  for (int j = 0; j < DPT; ++j) U[j] = 0.f;
  for (int s = 0; s < nc; ++s) {
    const float wv = ws[s] * vs[s * MM_VT + lane];
#pragma unroll
    for (int j = 0; j < DPT; ++j) {
      const int d = wave + MM_DG * j;
      if (d < dim) U[j] = fmaf(ks[s * DP + d], wv, U[j]);
    }
  }
  float* Uc = work.U + ((size_t)c * H + h) * dim * vdim;
#pragma unroll
  for (int j = 0; j < DPT; ++j) {
    const int d = wave + MM_DG * j;
    if (d < dim && v < vdim) Uc[(size_t)d * vdim + v] = U[j];
  }
  if (vt == 0) {
    for (int d = tid; d < dim; d += blockDim.x) {
      float nn = 0.f;
      for (int s = 0; s < nc; ++s) nn = fmaf(ws[s], ks[s * DP + d], nn);
      work.un[((size_t)c * H + h) * dim + d] = nn;
    }
  }
}

// Elementwise over the chunks of a sequence, in order: a thread carries one element of S (or of n) from chunk to
// chunk, so that a (sequence, head) is spread over as many workgroups as its state has elements / 256.  m after the
// last chunk goes to work.m_end (other workgroups still read the old m from the state): the out kernel stores it.
__global__ void __launch_bounds__(256)
mm_chunk_carry_kernel(float* __restrict__ state, int spare_row, const int* __restrict__ seq_start,
                      const int* __restrict__ seq_slot, ChunkWork work, int H, int dim, int vdim) {
  const int b = blockIdx.x, h = blockIdx.y;
  const long SV = (long)dim * vdim, total = SV + dim;
  const long e = (long)blockIdx.z * 256 + threadIdx.x;
  const int n_new = seq_start[b + 1] - seq_start[b];
  if (n_new <= 0) return;
  int c = 0;                      // the step's chunks before this sequence's
  for (int x = 0; x < b; ++x) c += (seq_start[x + 1] - seq_start[x] + MMC_L - 1) / MMC_L;
  const int n_chunks = (n_new + MMC_L - 1) / MMC_L;
  const int slot = seq_slot[b];
  float* st = state + ((size_t)(slot < 0 ? spare_row : slot) * H + h) * (total + 1);
  const bool on = e < total, is_s = e < SV, first = blockIdx.z == 0 && threadIdx.x == 0;
  float x = on ? st[e] : 0.f;
  float m = st[total];
  constexpr int AHEAD = 4;         // chunks whose sums are asked for together
  for (int k0 = 0; k0 < n_chunks; k0 += AHEAD) {
    float u[AHEAD], bL[AHEAD], PL[AHEAD];
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      const size_t ch = (size_t)(c + min(k0 + a, n_chunks - 1)) * H + h;
      u[a] = !on ? 0.f : (is_s ? work.U[ch * SV + e] : work.un[ch * dim + (e - SV)]);
      bL[a] = work.stat[ch * 2], PL[a] = work.stat[ch * 2 + 1];
    }
#pragma unroll
    for (int a = 0; a < AHEAD; ++a) {
      if (k0 + a < n_chunks) {
        const size_t ch = (size_t)(c + k0 + a) * H + h;
        if (on) {
          if (is_s) work.S0[ch * SV + e] = x;
          else work.n0[ch * dim + (e - SV)] = x;
        }
        if (first) work.m0[ch] = m;
        const float M = fmaxf(m, PL[a]);
        x = expf(m - M) * x + expf(PL[a] - M) * u[a];
        m = bL[a] + M;
      }
    }
  }
  if (on) st[e] = x;
  if (first) work.m_end[(size_t)b * H + h] = m;
}

__host__ __device__ inline size_t mmc_out_lds_floats(int dim) {
  return (size_t)6 * MMC_L + 2 * MMC_L * (dim + 1) + MMC_L * MM_VT + MMC_L * (MMC_L + 1) + (size_t)dim * MM_VT + dim + 3 * MMC_L;
}

__global__ void __launch_bounds__(MM_DG * SYN_WAVE)
mm_chunk_out_kernel(const float* __restrict__ proj, int width, const float* __restrict__ i_bias,
                    const float* __restrict__ f_bias, float cap, float q_scale, const int* __restrict__ seq_start,
                    int n_seqs, ChunkWork work, float* __restrict__ out, int H, int dim, int vdim,
                    float* __restrict__ state, int spare_row, const int* __restrict__ seq_slot) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int L = MMC_L;
  const int DP = dim + 1;
  double* as = (double*)lds;             // [L] a_s
  double* Ms = as + L;                   // [L] M_t
  double* bs = Ms + L;                   // [L] b_t
  float* qs = (float*)(bs + L);          // [L][DP]  q, scaled
  float* ks = qs + L * DP;               // [L][DP]
  float* vs = ks + L * DP;               // [L][64]
  float* As = vs + L * MM_VT;            // [L][L + 1]
  float* Cs = As + L * (L + 1);          // [dim][64]  S before the chunk
  float* ns = Cs + (size_t)dim * MM_VT;  // [dim]
  float* gq = ns + dim;                  // [L] g_t
  float* rs = gq + L;                    // [L] n_t . q_t
  const int c = blockIdx.x, h = blockIdx.y, vt = blockIdx.z;
  int seq, first, nc;
  if (!chunk_of(seq_start, n_seqs, c, seq, first, nc)) return;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, tid = threadIdx.x;
  const int v = vt * MM_VT + lane;
  const bool v_ok = v < vdim;
  const size_t ch = (size_t)c * H + h;
  if (first == seq_start[seq] && vt == 0 && tid == 0) {
    // the sequence's m behind this step, which the carry left aside
    const int slot = seq_slot[seq];
    state[((size_t)(slot < 0 ? spare_row : slot) * H + h) * ((size_t)dim * vdim + dim + 1) + (size_t)dim * vdim + dim] =
        work.m_end[(size_t)seq * H + h];
  }
  const int q_col = h * dim, k_col = H * dim + h * dim, v_col = 2 * H * dim + h * vdim;
  const int i_col = 2 * H * dim + 2 * H * vdim + h, f_col = i_col + H;
  for (int idx = tid; idx < L * dim; idx += blockDim.x) {
    const int t = idx / dim, d = idx % dim;
    const float* row = proj + (size_t)(first + min(t, nc - 1)) * width;
    qs[t * DP + d] = t < nc ? row[q_col + d] * q_scale : 0.f;
    ks[t * DP + d] = t < nc ? row[k_col + d] : 0.f;
  }
  for (int idx = tid; idx < L * MM_VT; idx += blockDim.x) {
    const int t = idx / MM_VT, cc = idx % MM_VT;
    vs[idx] = (t < nc && vt * MM_VT + cc < vdim) ? proj[(size_t)(first + t) * width + v_col + vt * MM_VT + cc] : 0.f;
  }
  {
    const float* S0 = work.S0 + ch * dim * vdim;
    for (int idx = tid; idx < dim * MM_VT; idx += blockDim.x) {
      const int d = idx / MM_VT, cc = idx % MM_VT;
      Cs[idx] = vt * MM_VT + cc < vdim ? S0[(size_t)d * vdim + vt * MM_VT + cc] : 0.f;
    }
    for (int d = tid; d < dim; d += blockDim.x) ns[d] = work.n0[ch * dim + d];
  }
  if (wave == 0) {
    const float m0 = work.m0[ch];
    const ChunkGates g = chunk_gates(proj, width, first, nc, lane, i_col, f_col, i_bias ? i_bias[h] : 0.f,
                                     f_bias ? f_bias[h] : 0.f, cap);
    const double M = fmax((double)m0, g.P);
    if (lane < L) {
      as[lane] = g.a, Ms[lane] = M, bs[lane] = g.b;
      gq[lane] = expf((float)((double)m0 - M));
    }
  }
  __syncthreads();
  {
    // A[t][s]: thread tid takes t = tid / 8 and the four s = 4 (tid % 8) ..
    const int t = tid / 8, s0 = 4 * (tid % 8);
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    if (s0 <= t) {
      const float* qr = qs + t * DP;
      const float* kr = ks + s0 * DP;
      for (int d = 0; d < dim; ++d) {
        const float qv = qr[d];
        a0 = fmaf(qv, kr[d], a0), a1 = fmaf(qv, kr[DP + d], a1);
        a2 = fmaf(qv, kr[2 * DP + d], a2), a3 = fmaf(qv, kr[3 * DP + d], a3);
      }
    }
    const double Mt = Ms[t];
    float* ar = As + t * (L + 1) + s0;
    const bool row_ok = t < nc;
    ar[0] = (row_ok && s0 <= t) ? a0 * expf((float)(as[s0] - Mt)) : 0.f;
    ar[1] = (row_ok && s0 + 1 <= t) ? a1 * expf((float)(as[s0 + 1] - Mt)) : 0.f;
    ar[2] = (row_ok && s0 + 2 <= t) ? a2 * expf((float)(as[s0 + 2] - Mt)) : 0.f;
    ar[3] = (row_ok && s0 + 3 <= t) ? a3 * expf((float)(as[s0 + 3] - Mt)) : 0.f;
  }
  __syncthreads();
  // wave w takes the tokens 8 w .. 8 w + 7: their n . q first, then this lane's column of S^T q
  constexpr int R = L / MM_DG;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int t = wave * R + r;
    float part = lane < L ? As[t * (L + 1) + lane] : 0.f;
    float nq0 = 0.f;
    for (int d = lane; d < dim; d += SYN_WAVE) nq0 = fmaf(ns[d], qs[t * DP + d], nq0);
    part = wave_sum(part + gq[t] * nq0);
    if (lane == 0) rs[t] = part;
  }
  float acc[R], acc0[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f, acc0[r] = 0.f;
  for (int s = 0; s < nc; ++s) {
    const float vv = vs[s * MM_VT + lane];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = fmaf(As[(wave * R + r) * (L + 1) + s], vv, acc[r]);
  }
#pragma unroll 4
  for (int d = 0; d < dim; ++d) {
    const float cv = Cs[(size_t)d * MM_VT + lane];
#pragma unroll
    for (int r = 0; r < R; ++r) acc0[r] = fmaf(qs[(wave * R + r) * DP + d], cv, acc0[r]);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // rs[t] of this wave's tokens, written by its lane 0
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int t = wave * R + r;
    if (t < nc && v_ok) {
      const float den = fmaxf(fabsf(rs[t]), expf(-(float)(bs[t] + Ms[t]))) + 1e-6f;
      out[(size_t)(first + t) * H * vdim + (size_t)h * vdim + v] = (acc[r] + gq[t] * acc0[r]) / den;
    }
  }
}

static hipError_t raise_chunk_out_lds() {
  static OncePerDevice once;
  return once_per_device(once, [] {
    return hipFuncSetAttribute((const void*)mm_chunk_out_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)(mmc_out_lds_floats(MM_MAX_DIM) * sizeof(float)));
  });
}

// floats of scratch memory that a chunked call over n_tokens tokens in n_seqs sequences needs
SYN_EXPORT long syn_matrix_memory_chunk_scratch(int n_tokens, int n_seqs, int H, int dim, int vdim) {
  const long chunks = (n_tokens + MMC_L - 1) / MMC_L + n_seqs;
  return chunks * H * (2L * dim * vdim + 2L * dim + 3) + (long)n_seqs * H;
}

// out [N][H * vdim] float: o_t of every token, before the heads' norm
// chunked: 0 = token by token (single tokens), 1 = in chunks (prompts; scratch: syn_matrix_memory_chunk_scratch floats)
SYN_EXPORT int syn_matrix_memory_scan(const float* proj, int width, const float* i_bias, const float* f_bias, float cap,
                                      float q_scale, float* state, int state_rows, const int* seq_start,
                                      const int* seq_slot, int n_seqs, float* out, int H, int dim, int vdim,
                                      int chunked, int n_tokens, float* scratch, hipStream_t stream) {
  SYN_CHECK(n_seqs > 0 && H > 0, "matrix_memory_scan: empty input");
  SYN_CHECK(dim > 0 && dim <= MM_MAX_DIM && vdim > 0, "matrix_memory_scan: sizes %d x %d (keys up to %d)", dim, vdim,
            MM_MAX_DIM);
  SYN_CHECK(width >= 2 * H * dim + 2 * H * vdim + 2 * H, "matrix_memory_scan: rows of %d values do not hold q, k, v, "
            "the gate and the two gates of the cell", width);
  SYN_CHECK(state_rows >= 1, "matrix_memory_scan: no state rows");
  const dim3 grid(n_seqs, H, (vdim + MM_VT - 1) / MM_VT);
  const int dpt = (dim + MM_DG - 1) / MM_DG;
  if (chunked) {
    SYN_CHECK(scratch != nullptr, "matrix_memory_scan: prompts in chunks need scratch memory");
    const long chunks = (n_tokens + MMC_L - 1) / MMC_L + n_seqs;
    ChunkWork w;
    w.U = scratch;
    w.S0 = w.U + chunks * H * dim * vdim;
    w.un = w.S0 + chunks * H * dim * vdim;
    w.n0 = w.un + chunks * H * dim;
    w.stat = w.n0 + chunks * H * dim;
    w.m0 = w.stat + chunks * H * 2;
    w.m_end = w.m0 + chunks * H;
    const dim3 carry_grid(n_seqs, H, (unsigned)(((long)dim * vdim + dim + 255) / 256));
    const dim3 per_chunk((unsigned)chunks, H, (vdim + MM_VT - 1) / MM_VT);
    const size_t local_lds = ((size_t)MMC_L * (dim + 1) + MMC_L * MM_VT + MMC_L) * sizeof(float);
    const size_t out_lds = mmc_out_lds_floats(dim) * sizeof(float);
    const hipError_t e = raise_chunk_out_lds();
    SYN_CHECK(e == hipSuccess, "matrix_memory_scan: the chunk kernel's LDS: %s", hipGetErrorString(e));
#define SYN_MMC(D)                                                                                                       \
  do {                                                                                                                   \
    mm_chunk_local_kernel<D><<<per_chunk, MM_DG * SYN_WAVE, local_lds, stream>>>(proj, width, i_bias, f_bias, cap,        \
                                                                                 seq_start, n_seqs, w, H, dim, vdim);     \
  } while (0)
    if (dpt <= 8) SYN_MMC(8);
    else if (dpt <= 16) SYN_MMC(16);
    else if (dpt <= 32) SYN_MMC(32);
    else SYN_MMC(64);
#undef SYN_MMC
    mm_chunk_carry_kernel<<<carry_grid, 256, 0, stream>>>(state, state_rows - 1, seq_start, seq_slot, w, H, dim, vdim);
    mm_chunk_out_kernel<<<per_chunk, MM_DG * SYN_WAVE, out_lds, stream>>>(proj, width, i_bias, f_bias, cap, q_scale,
                                                                          seq_start, n_seqs, w, out, H, dim, vdim, state,
                                                                          state_rows - 1, seq_slot);
    SYN_LAUNCH_CHECK("matrix_memory_scan (chunks)");
    return 0;
  }
  const dim3 per_head(n_seqs, H);
#define SYN_MM(D)                                                                                                       \
  matrix_memory_scan_kernel<D><<<per_head, MM_DG * SYN_WAVE, 0, stream>>>(proj, width, i_bias, f_bias, cap, q_scale, state, \
                                                                          state_rows - 1, seq_start, seq_slot, out, H, dim, \
                                                                          vdim)
  if (dpt <= 8) SYN_MM(8);
  else if (dpt <= 16) SYN_MM(16);
  else if (dpt <= 32) SYN_MM(32);
  else SYN_MM(64);
#undef SYN_MM
  SYN_LAUNCH_CHECK("matrix_memory_scan");
  return 0;
}

// Each head's o divided by its root mean square, times a gain over all heads' values, times sigmoid(gate):
// one wave for each (token, head).  gate: float rows of gate_stride values (the fused projection from its gate on).
// silu_first: the gate acts before the norm instead, as o * silu(gate), and the norm sees the gated values.
template <typename TOut>
__global__ void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gain, float eps,
                                      const float* __restrict__ gate, int gate_stride, TOut* __restrict__ out,
                                      int n_items, int H, int vdim, int silu_first) {
  const int item = blockIdx.x * (blockDim.x / SYN_WAVE) + threadIdx.x / SYN_WAVE;
  if (item >= n_items) return;
  const int lane = threadIdx.x % SYN_WAVE;
  const int tok = item / H, h = item % H;
  const float* x = o + ((size_t)tok * H + h) * vdim;
  const float* g = gate ? gate + (size_t)tok * gate_stride + (size_t)h * vdim : nullptr;
  const bool first = silu_first && g;
  float ss = 0.f;
  for (int d = lane; d < vdim; d += SYN_WAVE) {
    const float v = first ? x[d] * (g[d] / (1.f + expf(-g[d]))) : x[d];
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)vdim + eps);
  for (int d = lane; d < vdim; d += SYN_WAVE) {
    float v = (first ? x[d] * (g[d] / (1.f + expf(-g[d]))) : x[d]) * inv;
    if (gain) v *= gain[h * vdim + d];
    if (g && !first) v *= 1.f / (1.f + expf(-g[d]));
    out[((size_t)tok * H + h) * vdim + d] = from_f32<TOut>(v);
  }
}

SYN_EXPORT int syn_head_norm_gate(const float* o, const float* gain, float eps, const float* gate, int gate_stride,
                                  void* out, int out_is_f32, int n_tokens, int H, int vdim, int silu_first,
                                  hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && H > 0 && vdim > 0, "head_norm_gate: empty input");
  SYN_CHECK(gate == nullptr || gate_stride >= H * vdim, "head_norm_gate: gate rows of %d values", gate_stride);
  const int wpb = 4, items = n_tokens * H;
  const int grid = (items + wpb - 1) / wpb;
  if (out_is_f32)
    head_norm_gate_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>(o, gain, eps, gate, gate_stride, (float*)out, items,
                                                                      H, vdim, silu_first);
  else
    head_norm_gate_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>(o, gain, eps, gate, gate_stride, (bf16*)out, items,
                                                                     H, vdim, silu_first);
  SYN_LAUNCH_CHECK("head_norm_gate");
  return 0;
}
