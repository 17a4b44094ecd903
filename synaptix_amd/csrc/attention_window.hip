// Attention over the paged cache for mixers whose scores, mask and softmax differ from the plain causal ones:
//
//   score(i, j) = scale (q_i . k_j) [soft cap] - slope_h (i - j) - r1_h ln(1 + r2_h (i - j))
//   key j is visible to the query at i iff  j <= i  and  (window <= 0 or i - j < window or j < keep_first)
//       and (chunk <= 0 or j / chunk == i / chunk or j < keep_first):
//       a sliding window that never loses the first keep_first keys, which keep their true positions, and/or runs of
//       `chunk` positions counted from the sequence's first token, whose keys only their own run's queries see;
//   p_j = exp(score_j) / (sink + sum_j exp(score_j)),  sink = exp(sinks[h]) with `sinks` (a learned score a head of a
//       further key that has no value), 1 with `sink_one` (that score is 0), else 0;
//   head h reads kv head h / (heads / kv heads); keys have `dim` values, values `vdim`;
//   v_share > 1: that many neighbouring kv heads read the values of one value head (kv heads / v_share of them are
//       stored), as the maps of a differential attention do, which have keys of their own and the values in common;
//   the heads' results may be multiplied by sigmoid(gate) before they are stored: a gate for every value, or with
//       `gate_per_head` one for each head.
// Scores, weights and sums are 32-bit whatever the cache's type; the weights are not rounded before they meet V.
//
// Cache pages hold 64 tokens: k_pages[page, kv_head, token, dim], v_pages[page, kv_head, vdim, token] (plain rows in
// both types).  One wave for each (token, head), plain FMA, online softmax over blocks of 64 keys: prompts and single
// tokens alike.
#include "common.h"

#define AW_MAX_DIM 640      // (instantiations for head sizes up to 256 and up to 640)

struct WindowTerms {
  const float* slopes;   // [heads] or nullptr
  const float* r1;       // [heads] or nullptr (with r2)
  const float* r2;
  float softcap;         // 0: none
  int window;            // 0: every key
  int keep_first;
  int sink_one;
  int v_share;           // this many neighbouring kv heads read one value head (1: each its own)
  const float* sinks;    // [heads] or nullptr: the score of a key without a value in every softmax
  int chunk;             // 0: none
  int gate_per_head;     // the gate's rows hold one number a head (else one for each value)
};

// the first key that the query at `pos` sees (kept first keys aside); it never falls as pos grows
__device__ __forceinline__ int first_visible(int pos, const WindowTerms& t) {
  int lo = t.window > 0 ? max(0, pos - t.window + 1) : 0;
  if (t.chunk > 0) lo = max(lo, pos / t.chunk * t.chunk);
  return lo;
}

// ---------------------------------------------------------------- intake: bias, q/k norm, cache write
// proj [N][width] float holds the fused projection  [q heads x dim | k heads x dim | v heads x vdim | ...]; what lies
// behind v (a gate) is left where it is.  One wave for each (token, q head | k head | v head); there are nv value
// heads (nkv, unless several kv heads share a value head).
// cos_t, sin_t [positions][rot / 2] (or null): after the norm the first `rot` values of a q or k head are turned, value
// i < rot / 2 paired with value i + rot / 2 (with `pairs`: value 2 i with value 2 i + 1), by the angle whose cosine
// and sine stand at [position][i].  Without write_kv the rows hold queries only (keys and values are another layer's).
template <typename T>
__global__ void window_intake_kernel(const float* __restrict__ proj, int width, const float* __restrict__ bias,
                                     T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     const int* __restrict__ page_table, int table_stride,
                                     const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                     const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int pairs,
                                     int nh, int nkv, int nv, int dim, int vdim, int write_kv) {
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int tok = blockIdx.x;
  const int item = blockIdx.y * (blockDim.x / SYN_WAVE) + wave;
  if (item >= (write_kv ? nh + nkv + nv : nh)) return;
  const bool is_q = item < nh, is_k = !is_q && item < nh + nkv;
  const int len = (is_q || is_k) ? dim : vdim;
  const int col = is_q ? item * dim : (is_k ? nh * dim + (item - nh) * dim : (nh + nkv) * dim + (item - nh - nkv) * vdim);
  const float* src = proj + (size_t)tok * width + col;
  const float* b = bias ? bias + col : nullptr;
  const float* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);
  float inv = 1.f;
  if (gain) {
    float ss = 0.f;
    for (int d = lane; d < len; d += SYN_WAVE) {
      const float v = src[d] + (b ? b[d] : 0.f);
      ss += v * v;
    }
    inv = 1.f / sqrtf(wave_sum(ss) / (float)len + eps);
  }
  const int pos = tok_pos[tok];
  T* dst;
  size_t stride = 1;
  if (is_q) {
    dst = q_out + ((size_t)tok * nh + item) * dim;
  } else {
    const int page = page_table[(size_t)tok_seq[tok] * table_stride + pos / SYN_PAGE];
    if (is_k) {
      dst = k_pages + (((size_t)page * nkv + (item - nh)) * SYN_PAGE + pos % SYN_PAGE) * dim;
    } else {
      dst = v_pages + ((size_t)page * nv + (item - nh - nkv)) * vdim * SYN_PAGE + pos % SYN_PAGE;
      stride = SYN_PAGE;
    }
  }
  const int half = (cos_t && (is_q || is_k)) ? rot / 2 : 0;
  for (int d = lane; d < len; d += SYN_WAVE) {
    float v = src[d] + (b ? b[d] : 0.f);
    if (gain) v = v * inv * gain[d];
    if (d < 2 * half) {
      const bool first = pairs ? d % 2 == 0 : d < half;
      const int i = pairs ? d / 2 : (first ? d : d - half);
      const int mate = pairs ? (d ^ 1) : (first ? d + half : d - half);
      float o = src[mate] + (b ? b[mate] : 0.f);
      if (gain) o = o * inv * gain[mate];
      const float c = cos_t[(size_t)pos * half + i], sn = sin_t[(size_t)pos * half + i];
      v = first ? v * c - o * sn : v * c + o * sn;
    }
    dst[(size_t)d * stride] = from_f32<T>(v);
  }
}

SYN_EXPORT int syn_window_intake(const float* proj, int width, const float* bias, void* q_out, void* k_pages,
                                 void* v_pages, int is_f32, const int* page_table, int table_stride, const int* tok_seq,
                                 const int* tok_pos, const float* q_gain, const float* k_gain, float eps,
                                 const float* cos_t, const float* sin_t, int rot, int pairs, int n_tokens,
                                 int nh, int nkv, int nv, int dim, int vdim, int write_kv, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0 && nv > 0 && dim > 0 && vdim > 0, "window_intake: empty input");
  SYN_CHECK(width >= (write_kv ? (nh + nkv) * dim + nv * vdim : nh * dim), "window_intake: rows of %d values do not hold q%s",
            width, write_kv ? ", k and v" : "");
  SYN_CHECK((q_gain == nullptr) == (k_gain == nullptr), "window_intake: q and k gains come together");
  SYN_CHECK((cos_t == nullptr) == (sin_t == nullptr) && (cos_t == nullptr || (rot > 0 && rot % 2 == 0 && rot <= dim)),
            "window_intake: a rotation of %d of %d values", rot, dim);
  const int wpb = 4, items = write_kv ? nh + nkv + nv : nh;
  const dim3 grid(n_tokens, (items + wpb - 1) / wpb);
  if (is_f32)
    window_intake_kernel<float><<<grid, wpb * SYN_WAVE, 0, stream>>>(proj, width, bias, (float*)q_out, (float*)k_pages,
                                                                     (float*)v_pages, page_table, table_stride, tok_seq,
                                                                     tok_pos, q_gain, k_gain, eps, cos_t, sin_t, rot, pairs,
                                                                     nh, nkv, nv, dim, vdim, write_kv);
  else
    window_intake_kernel<bf16><<<grid, wpb * SYN_WAVE, 0, stream>>>(proj, width, bias, (bf16*)q_out, (bf16*)k_pages,
                                                                    (bf16*)v_pages, page_table, table_stride, tok_seq,
                                                                    tok_pos, q_gain, k_gain, eps, cos_t, sin_t, rot, pairs,
                                                                    nh, nkv, nv, dim, vdim, write_kv);
  SYN_LAUNCH_CHECK("window_intake");
  return 0;
}

// ---------------------------------------------------------------- attention, one wave a (token, head)
__device__ __forceinline__ float window_score(float dot, float scale, const WindowTerms& t, float slope, float r1,
                                              float r2, int pos, int key) {
  float s = dot * scale;
  if (t.softcap > 0.f) s = t.softcap * tanhf(s / t.softcap);
  const float dist = (float)(pos - key);
  s -= slope * dist;
  if (t.r1) s -= r1 * logf(1.f + r2 * dist);
  return s;
}

// eight consecutive values of a cache row as floats: one 16-byte load in bf16, two in 32-bit
template <typename T> __device__ __forceinline__ void load8(const T* p, float (&o)[8]);
template <> __device__ __forceinline__ void load8<bf16>(const bf16* p, float (&o)[8]) {
  const bf16x8 v = *(const bf16x8*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (float)v[e];
}
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&o)[8]) {
  const float4 a = ((const float4*)p)[0], b = ((const float4*)p)[1];
  o[0] = a.x, o[1] = a.y, o[2] = a.z, o[3] = a.w, o[4] = b.x, o[5] = b.y, o[6] = b.z, o[7] = b.w;
}

// WAVES waves a (token, head): wave w takes every WAVES-th of the visible blocks of 64 keys, and the waves' partial
// results (maximum, sum, weighted values) are merged through LDS at the end.  One wave is enough where a step has many
// tokens; single tokens over a long window get eight.
// MAXD: the largest head size that the registers and LDS of this instantiation hold (a multiple of 64).
template <typename T, int WAVES, int MAXD>
__global__ void __launch_bounds__(WAVES * SYN_WAVE)
window_attention_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                        const int* __restrict__ page_table, int table_stride, const int* __restrict__ tok_seq,
                        const int* __restrict__ tok_pos, const float* __restrict__ gate, int gate_stride,
                        const float* __restrict__ gate_bias, T* __restrict__ out, float scale, int nh, int nkv, int dim,
                        int vdim, WindowTerms terms) {
  __shared__ float qs[MAXD];
  __shared__ float ps[WAVES][SYN_PAGE];
  __shared__ float part_o[WAVES][MAXD];
  __shared__ float part_ml[WAVES][2];
  const int tok = blockIdx.x, head = blockIdx.y;
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  const int seq = tok_seq[tok], pos = tok_pos[tok];
  const int kvh = head / (nh / nkv);
  const T* qr = q + ((size_t)tok * nh + head) * dim;
  for (int d = threadIdx.x; d < dim; d += WAVES * SYN_WAVE) qs[d] = to_f32<T>(qr[d]);
  __syncthreads();

  const int lo = first_visible(pos, terms);
  const int kept = min(terms.keep_first, lo);        // keys below `kept` are seen although the window has passed them
  const int n_kept_blocks = kept > 0 ? (kept - 1) / SYN_PAGE + 1 : 0;
  const int first_window_block = max(lo / SYN_PAGE, n_kept_blocks);
  const int n_blocks = n_kept_blocks + (pos / SYN_PAGE - first_window_block + 1);
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;
  const float r1 = terms.r1 ? terms.r1[head] : 0.f, r2 = terms.r1 ? terms.r2[head] : 0.f;
  // the sink is a key without a value whose score is sinks[head], or 0: the first wave's running maximum and sum
  // start from it
  const bool sink_here = (terms.sink_one || terms.sinks) && wave == 0;
  float m = sink_here ? (terms.sinks ? terms.sinks[head] : 0.f) : -INFINITY, l = sink_here ? 1.f : 0.f;
  float o[MAXD / SYN_WAVE] = {};
  for (int idx = wave; idx < n_blocks; idx += WAVES) {
    const int kb = idx < n_kept_blocks ? idx : first_window_block + (idx - n_kept_blocks);
    const int page = page_table[(size_t)seq * table_stride + kb];
    const size_t kbase = ((size_t)page * nkv + kvh) * SYN_PAGE * dim;
    const size_t vbase = ((size_t)page * (nkv / terms.v_share) + kvh / terms.v_share) * SYN_PAGE * vdim;
    const int key = kb * SYN_PAGE + lane;
    const bool valid = key <= pos && (key >= lo || key < kept);
    float s = -INFINITY;
    if (valid) {
      const T* kr = k_pages + kbase + (size_t)lane * dim;
      float dot = 0.f;
      if (dim % 8 == 0) {
        for (int d = 0; d < dim; d += 8) {
          float kv[8];
          load8<T>(kr + d, kv);
#pragma unroll
          for (int e = 0; e < 8; ++e) dot = fmaf(qs[d + e], kv[e], dot);
        }
      } else {
        for (int d = 0; d < dim; ++d) dot = fmaf(qs[d], to_f32<T>(kr[d]), dot);
      }
      s = window_score(dot, scale, terms, slope, r1, r2, pos, key);
    }
    const float m_new = fmaxf(m, wave_max(s));   // every block that is visited holds a visible key
    const float alpha = expf(m - m_new);
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
    // the wave's own lanes exchange their weights through LDS: a barrier of the wave, not of the workgroup (the
    // waves walk different numbers of blocks)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    ps[wave][lane] = p;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < MAXD / SYN_WAVE; ++i) {
      const int d = lane + i * SYN_WAVE;
      if (d < vdim) {
        const T* vr = v_pages + vbase + (size_t)d * SYN_PAGE;
        float acc = o[i] * alpha;
        for (int j = 0; j < SYN_PAGE; j += 8) {
          float vv[8];
          load8<T>(vr + j, vv);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float pj = ps[wave][j + e];
            acc = fmaf(pj, pj != 0.f ? vv[e] : 0.f, acc);   // slots past the sequence's end may hold anything
          }
        }
        o[i] = acc;
      }
    }
  }
  if (WAVES > 1) {
    // merge in the waves' order: the largest maximum, every wave's sum and values scaled to it
    if (lane == 0) part_ml[wave][0] = m, part_ml[wave][1] = l;
#pragma unroll
    for (int i = 0; i < MAXD / SYN_WAVE; ++i)
      if (lane + i * SYN_WAVE < vdim) part_o[wave][lane + i * SYN_WAVE] = o[i];
    __syncthreads();
    if (wave != 0) return;
    float mm = -INFINITY;
    for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, part_ml[w][0]);
    l = 0.f;
#pragma unroll
    for (int i = 0; i < MAXD / SYN_WAVE; ++i) o[i] = 0.f;
    for (int w = 0; w < WAVES; ++w) {
      const float f = part_ml[w][0] == -INFINITY ? 0.f : expf(part_ml[w][0] - mm);
      l += f * part_ml[w][1];
#pragma unroll
      for (int i = 0; i < MAXD / SYN_WAVE; ++i)
        if (lane + i * SYN_WAVE < vdim) o[i] += f * part_o[w][lane + i * SYN_WAVE];
    }
  }
  T* orow = out + ((size_t)tok * nh + head) * vdim;
  const int per_head = terms.gate_per_head;
  const float* g = gate ? gate + (size_t)tok * gate_stride + (per_head ? head : (size_t)head * vdim) : nullptr;
#pragma unroll
  for (int i = 0; i < MAXD / SYN_WAVE; ++i) {
    const int d = lane + i * SYN_WAVE;
    if (d < vdim) {
      float v = o[i] / l;
      if (g) {
        const float z = g[per_head ? 0 : d] + (gate_bias ? gate_bias[per_head ? head : head * vdim + d] : 0.f);
        v *= 1.f / (1.f + expf(-z));
      }
      orow[d] = from_f32<T>(v);
    }
  }
}

// gate: float rows of gate_stride values whose first nh * vdim are the gate of each value (or null)
SYN_EXPORT int syn_window_attention(const void* q, const void* k_pages, const void* v_pages, int is_f32,
                                    const int* page_table, int table_stride, const int* tok_seq, const int* tok_pos,
                                    const float* gate, int gate_stride, const float* gate_bias, void* out, float scale,
                                    int n_tokens, int nh, int nkv, int dim, int vdim, const float* slopes,
                                    const float* r1, const float* r2, float softcap, int window, int keep_first,
                                    int sink_one, int v_share, const float* sinks, int chunk, int gate_per_head,
                                    hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && nh > 0 && nkv > 0, "window_attention: empty input");
  SYN_CHECK(chunk >= 0 && !(sinks && sink_one), "window_attention: chunks of %d, or two sinks", chunk);
  SYN_CHECK(v_share > 0 && nkv % v_share == 0, "window_attention: %d kv heads in shares of %d", nkv, v_share);
  SYN_CHECK(nh % nkv == 0, "window_attention: %d heads do not divide into %d kv heads", nh, nkv);
  SYN_CHECK(dim > 0 && dim <= AW_MAX_DIM && vdim > 0 && vdim <= AW_MAX_DIM,
            "window_attention: head sizes %d and %d are outside 1..%d", dim, vdim, AW_MAX_DIM);
  SYN_CHECK(softcap >= 0.f && window >= 0 && keep_first >= 0, "window_attention: soft cap %g, window %d, kept %d",
            (double)softcap, window, keep_first);
  SYN_CHECK((r1 == nullptr) == (r2 == nullptr), "window_attention: r1 and r2 come together");
  SYN_CHECK(gate == nullptr || gate_stride >= (gate_per_head ? nh : nh * vdim), "window_attention: gate rows of %d values",
            gate_stride);
  const WindowTerms terms = {slopes, r1, r2, softcap, window, keep_first, sink_one, v_share, sinks, chunk, gate_per_head};
  const dim3 grid(n_tokens, nh);
  // few (token, head) pairs (single tokens of a few sequences): eight waves share each pair's keys
  const bool many_waves = (long)n_tokens * nh < 8L * syn_compute_units();
  const bool large = dim > 256 || vdim > 256;
#define SYN_AW2(T, W, D)                                                                                              \
  window_attention_kernel<T, W, D><<<grid, W * SYN_WAVE, 0, stream>>>((const T*)q, (const T*)k_pages, (const T*)v_pages, \
                                                                      page_table, table_stride, tok_seq, tok_pos, gate, \
                                                                      gate_stride, gate_bias, (T*)out, scale, nh, nkv,  \
                                                                      dim, vdim, terms)
#define SYN_AW(T, W) do { if (large) SYN_AW2(T, W, 640); else SYN_AW2(T, W, 256); } while (0)
  if (is_f32) {
    if (many_waves) SYN_AW(float, 8); else SYN_AW(float, 1);
  } else {
    if (many_waves) SYN_AW(bf16, 8); else SYN_AW(bf16, 1);
  }
#undef SYN_AW
#undef SYN_AW2
  SYN_LAUNCH_CHECK("window_attention");
  return 0;
}

// ---------------------------------------------------------------- prompts in bf16 on the matrix cores
// One wave for 16 queries of one (sequence, head), four such waves a workgroup: the workgroup walks the pages that its
// 64 queries see, a page of 64 keys at a time through LDS, and a wave leaves out a page none of whose keys it sees.
// S^T = K Q^T (MFMA 16x16: a lane then holds four keys of ONE query, so
// the softmax's statistics are a lane's own plus two exchanges across the lane groups), and the accumulator's layout
// is the B operand of O^T += V^T P^T, whose A operand are 8-byte pieces of the V page's rows.  The weights meet V as
// two bf16 numbers each (the weight rounded, and what the rounding left), so that they count with 16 bits of mantissa
// although the product runs in bf16.  Head sizes in steps of 16 up to 128 (keys in steps of 32 take k-steps of 32).
#define AWP_TILES 8
typedef __attribute__((ext_vector_type(4))) __bf16 awp_bf16x4;

__device__ __forceinline__ f32x4 awp_mfma16(bf16x4 a, bf16x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 awp_mfma32(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 awp_join(bf16x4 lo, bf16x4 hi) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = lo[e], r[4 + e] = hi[e];
  return r;
}

#define AWP_KPAD 8      // bf16 values behind a K row in LDS, so that the 16 rows of a fragment fall into different banks
#define AWP_VPAD 4      // the same for a V row (64 tokens)

template <bool X32>
__global__ void __launch_bounds__(256, 2)      // (two waves a SIMD: the registers are bounded for that)
window_prefill_bf16_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pages, const bf16* __restrict__ v_pages,
                           const int* __restrict__ page_table, int table_stride, const int* __restrict__ seq_start,
                           const int* __restrict__ seq_past, int n_seqs, const float* __restrict__ gate, int gate_stride,
                           const float* __restrict__ gate_bias, bf16* __restrict__ out, float scale, int nh, int nkv,
                           int dim, int vdim, WindowTerms terms) {
  __shared__ __attribute__((aligned(16))) bf16 Ks[SYN_PAGE * (16 * AWP_TILES + AWP_KPAD)];
  __shared__ __attribute__((aligned(16))) bf16 Vs[16 * AWP_TILES * (SYN_PAGE + AWP_VPAD)];
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE, i = lane % 16, g = lane / 16;
  int bt = blockIdx.x, seq = -1, n_new = 0, start = 0;
  for (int b = 0; b < n_seqs; ++b) {
    const int s0 = seq_start[b], n = seq_start[b + 1] - s0, tiles = (n + 63) / 64;
    if (bt < tiles) {
      seq = b, n_new = n, start = s0;
      break;
    }
    bt -= tiles;
  }
  if (seq < 0) return;                              // (the whole workgroup: no barrier has been reached yet)
  const int nb = bt * 64, n0 = nb + wave * 16;       // the workgroup's and this wave's first query
  const bool wave_on = n0 < n_new;                   // a wave without queries still helps to stage the pages
  const int head = blockIdx.y, kvh = head / (nh / nkv);
  const int past = seq_past[seq];
  const bool q_ok = n0 + i < n_new;
  const int my_n = min(n0 + i, n_new - 1);       // (rows beyond the sequence's tokens repeat its last one and are not stored)
  const int qpos = past + my_n;
  const int vt = vdim / 16, KLD = dim + AWP_KPAD, VLD = SYN_PAGE + AWP_VPAD;
  const bf16* qrow = q + ((size_t)(start + my_n) * nh + head) * dim;
  bf16x8 qf8[AWP_TILES / 2];
  bf16x4 qf4[AWP_TILES];
  if constexpr (X32) {
#pragma unroll
    for (int s = 0; s < AWP_TILES / 2; ++s)
      if (s < dim / 32) qf8[s] = *(const bf16x8*)(qrow + 32 * s + 8 * g);
  } else {
#pragma unroll
    for (int s = 0; s < AWP_TILES; ++s)
      if (s < dim / 16) qf4[s] = *(const bf16x4*)(qrow + 16 * s + 4 * g);
  }
  const int lo_q = first_visible(qpos, terms);                                // this lane's query
  const int lo_wave = first_visible(past + n0, terms);                        // this wave's first query
  const int kmax_wave = past + min(n0 + 15, n_new - 1);
  const int lo_last = first_visible(kmax_wave, terms);                        // this wave's last query
  // the pages that the workgroup's 64 queries see together
  const int lo_first = first_visible(past + nb, terms);
  const int kmax = past + min(nb + 63, n_new - 1);
  const int kept = min(terms.keep_first, lo_first);
  const int n_kept_blocks = kept > 0 ? (kept - 1) / SYN_PAGE + 1 : 0;
  const int first_window_block = max(lo_first / SYN_PAGE, n_kept_blocks);
  const int n_blocks = n_kept_blocks + (kmax / SYN_PAGE - first_window_block + 1);
  const float slope = terms.slopes ? terms.slopes[head] : 0.f;
  const float r1 = terms.r1 ? terms.r1[head] : 0.f, r2 = terms.r1 ? terms.r2[head] : 0.f;
  constexpr float LOG2E = 1.4426950408889634f;
  const float scale2 = scale * LOG2E, slope2 = slope * LOG2E, cap2 = terms.softcap * LOG2E;
  // (the sink's score in units of ln 2; a score of 0 is 0 in any unit)
  float m = terms.sinks ? terms.sinks[head] * LOG2E : (terms.sink_one ? 0.f : -INFINITY);
  float l = (terms.sinks || terms.sink_one) ? 1.f : 0.f;
  f32x4 O[AWP_TILES];
#pragma unroll
  for (int j = 0; j < AWP_TILES; ++j) O[j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // A page's K and V go from memory to registers in whole 16-byte pieces, a row piece after another (every thread
  // up to four of each), one page ahead of the page that is being multiplied, and from there into LDS.
  constexpr int PIECES = 16 * AWP_TILES * SYN_PAGE / 8 / 256;      // 4
  uint4 kreg[PIECES], vreg[PIECES];
  int k_at[PIECES], v_at[PIECES];       // where this thread's pieces go in LDS (-1: the page has fewer pieces)
#pragma unroll
  for (int r = 0; r < PIECES; ++r) {
    const int it = tid + 256 * r;
    k_at[r] = it < SYN_PAGE * dim / 8 ? (it / (dim / 8)) * KLD + 8 * (it % (dim / 8)) : -1;
    v_at[r] = it < SYN_PAGE * vdim / 8 ? (it / 8) * VLD + 8 * (it % 8) : -1;
  }
  auto block_of = [&](int idx) { return idx < n_kept_blocks ? idx : first_window_block + (idx - n_kept_blocks); };
  auto fetch = [&](int idx) {
    const int page = page_table[(size_t)seq * table_stride + block_of(idx)];
    const uint4* kp = (const uint4*)(k_pages + ((size_t)page * nkv + kvh) * SYN_PAGE * dim);
    const uint4* vp = (const uint4*)(v_pages + ((size_t)page * (nkv / terms.v_share) + kvh / terms.v_share) * SYN_PAGE * vdim);
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
      const int it = tid + 256 * r;
      if (k_at[r] >= 0) kreg[r] = kp[it];
      if (v_at[r] >= 0) vreg[r] = vp[it];
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int r = 0; r < PIECES; ++r) {
      if (k_at[r] >= 0) *(uint4*)(Ks + k_at[r]) = kreg[r];
      if (v_at[r] >= 0) {
        uint2* dst = (uint2*)(Vs + v_at[r]);       // (a V row in LDS begins at a multiple of 8 bytes only)
        dst[0] = make_uint2(vreg[r].x, vreg[r].y);
        dst[1] = make_uint2(vreg[r].z, vreg[r].w);
      }
    }
  };
  fetch(0);
  for (int idx = 0; idx < n_blocks; ++idx) {
    const int kb = block_of(idx);
    __syncthreads();          // every wave has left the page before
    stage();
    __syncthreads();
    if (idx + 1 < n_blocks) fetch(idx + 1);
    const int page_lo = kb * SYN_PAGE, page_hi = page_lo + SYN_PAGE - 1;
    if (!wave_on || page_lo > kmax_wave || (page_hi < lo_wave && page_lo >= terms.keep_first)) continue;   // none of it is seen
    f32x4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16* krow = Ks + (16 * t + i) * KLD;
      if constexpr (X32) {
#pragma unroll
        for (int c = 0; c < AWP_TILES / 2; ++c)
          if (c < dim / 32) s[t] = awp_mfma32(*(const bf16x8*)(krow + 32 * c + 8 * g), qf8[c], s[t]);
      } else {
#pragma unroll
        for (int c = 0; c < AWP_TILES; ++c)
          if (c < dim / 16) s[t] = awp_mfma16(*(const bf16x4*)(krow + 16 * c + 4 * g), qf4[c], s[t]);
      }
    }
    // the terms and the mask on this lane's 16 scores (keys 16 t + 4 g + e of the page, all of query i); a page that
    // lies behind the wave's first query and inside its last query's window and chunk is seen whole by all of them: no mask
    const bool whole = page_hi <= past + n0 && page_lo >= lo_last;
    const float dist0 = (float)(qpos - page_lo - 4 * g);
    // scores in units of ln 2 from here on (scale, slope and cap carry log2 e; r1 ln(x) = r1 log2(x) ln 2): the
    // exponentials below are bare exp2
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = s[t][e] * scale2;
        if (terms.softcap > 0.f) v = cap2 * tanhf(s[t][e] * scale / terms.softcap);
        const float dist = dist0 - (float)(16 * t + e);          // query position - key position
        if (slope2 != 0.f) v -= slope2 * dist;
        if (terms.r1) v -= r1 * __builtin_amdgcn_logf(fmaf(r2, dist, 1.f));
        if (!whole) {
          const int key = page_lo + 16 * t + 4 * g + e;
          v = (key <= qpos && (key >= lo_q || key < terms.keep_first)) ? v : -INFINITY;
        }
        s[t][e] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, SYN_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, SYN_WAVE));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;     // nothing seen yet: every weight below is zero
    const float alpha = __builtin_amdgcn_exp2f(m - m_use);
    float sum = 0.f;
    // a weight as two bf16 numbers: its upper 16 bits, and the upper 16 bits of what they leave (16 bits of mantissa
    // together); two neighbours share a register
    unsigned hi[4][2], lw[4][2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int e = 0; e < 4; e += 2) {
        const float p0 = __builtin_amdgcn_exp2f(s[t][e] - m_use), p1 = __builtin_amdgcn_exp2f(s[t][e + 1] - m_use);
        sum += p0 + p1;                                           // exp2(-inf) = 0 for what is hidden
        const unsigned b0 = __float_as_uint(p0) & 0xffff0000u, b1 = __float_as_uint(p1) & 0xffff0000u;
        hi[t][e / 2] = (b0 >> 16) | b1;
        const unsigned r0 = __float_as_uint(p0 - __uint_as_float(b0)), r1b = __float_as_uint(p1 - __uint_as_float(b1));
        lw[t][e / 2] = (r0 >> 16) | (r1b & 0xffff0000u);
      }
    sum += __shfl_xor(sum, 16, SYN_WAVE);
    sum += __shfl_xor(sum, 32, SYN_WAVE);
    l = l * alpha + sum;
    m = m_new;
    const bool rescale = __any(alpha != 1.f);       // (the maximum moves in the first pages and then seldom)
#pragma unroll
    for (int pr = 0; pr < 2; ++pr) {
      // k index 8 g + e stands for key 32 pr + 4 g + e, 8 g + 4 + e for key 32 pr + 16 + 4 g + e: both operands agree
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
      const bf16x8 b_hi = __builtin_bit_cast(bf16x8, (u32x4){hi[2 * pr][0], hi[2 * pr][1], hi[2 * pr + 1][0], hi[2 * pr + 1][1]});
      const bf16x8 b_lo = __builtin_bit_cast(bf16x8, (u32x4){lw[2 * pr][0], lw[2 * pr][1], lw[2 * pr + 1][0], lw[2 * pr + 1][1]});
#pragma unroll
      for (int j = 0; j < AWP_TILES; ++j) {
        if (j < vt) {
          const bf16* vrow = Vs + (16 * j + i) * VLD + 32 * pr + 4 * g;
          const bf16x8 a = awp_join(*(const bf16x4*)vrow, *(const bf16x4*)(vrow + 16));
          if (pr == 0 && rescale) O[j] *= alpha;
          O[j] = awp_mfma32(a, b_hi, O[j]);
          O[j] = awp_mfma32(a, b_lo, O[j]);
        }
      }
    }
  }
  if (!q_ok) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const size_t tok = (size_t)(start + my_n);
#pragma unroll
  for (int j = 0; j < AWP_TILES; ++j) {
    if (j < vt) {
      const int col = head * vdim + 16 * j + 4 * g;
      bf16x4 o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = O[j][e] * inv;
        if (gate) {
          const int at = terms.gate_per_head ? head : col + e;
          const float z = gate[tok * gate_stride + at] + (gate_bias ? gate_bias[at] : 0.f);
          v *= 1.f / (1.f + __expf(-z));
        }
        o4[e] = (bf16)v;
      }
      *(bf16x4*)(out + tok * nh * vdim + col) = o4;
    }
  }
}

// Prompts (and any step that is not single tokens only) in bf16: seq_start [n_seqs + 1] offsets of the sequences' new
// tokens in q, seq_past [n_seqs] tokens cached before.  Head sizes that are multiples of 16 up to 128.
SYN_EXPORT int syn_window_attention_prefill_bf16(const void* q, const void* k_pages, const void* v_pages,
                                                 const int* page_table, int table_stride, const int* seq_start,
                                                 const int* seq_past, int n_seqs, int n_tokens, const float* gate,
                                                 int gate_stride, const float* gate_bias, void* out, float scale, int nh,
                                                 int nkv, int dim, int vdim, const float* slopes, const float* r1,
                                                 const float* r2, float softcap, int window, int keep_first, int sink_one,
                                                 int v_share, const float* sinks, int chunk, int gate_per_head,
                                                 hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && n_seqs > 0 && nh > 0 && nkv > 0, "window_attention_prefill: empty input");
  SYN_CHECK(v_share > 0 && nkv % v_share == 0, "window_attention_prefill: %d kv heads in shares of %d", nkv, v_share);
  SYN_CHECK(nh % nkv == 0, "window_attention_prefill: %d heads do not divide into %d kv heads", nh, nkv);
  SYN_CHECK(dim % 16 == 0 && vdim % 16 == 0 && dim >= 16 && vdim >= 16 && dim <= 16 * AWP_TILES && vdim <= 16 * AWP_TILES,
            "window_attention_prefill: head sizes %d and %d (multiples of 16 up to %d)", dim, vdim, 16 * AWP_TILES);
  SYN_CHECK(softcap >= 0.f && window >= 0 && keep_first >= 0, "window_attention_prefill: soft cap %g, window %d, kept %d",
            (double)softcap, window, keep_first);
  SYN_CHECK((r1 == nullptr) == (r2 == nullptr), "window_attention_prefill: r1 and r2 come together");
  SYN_CHECK(gate == nullptr || gate_stride >= (gate_per_head ? nh : nh * vdim), "window_attention_prefill: gate rows of %d values",
            gate_stride);
  SYN_CHECK(chunk >= 0 && !(sinks && sink_one), "window_attention_prefill: chunks of %d, or two sinks", chunk);
  SYN_CHECK((uintptr_t)q % 16 == 0 && (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0 && (uintptr_t)out % 8 == 0,
            "window_attention_prefill: operands are not aligned");
  const WindowTerms terms = {slopes, r1, r2, softcap, window, keep_first, sink_one, v_share, sinks, chunk, gate_per_head};
  const dim3 grid((n_tokens + 63) / 64 + n_seqs, nh);      // at most this many tiles of 64 queries; the rest leave at once
  if (dim % 32 == 0)
    window_prefill_bf16_kernel<true><<<grid, 256, 0, stream>>>(
        (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
        gate, gate_stride, gate_bias, (bf16*)out, scale, nh, nkv, dim, vdim, terms);
  else
    window_prefill_bf16_kernel<false><<<grid, 256, 0, stream>>>(
        (const bf16*)q, (const bf16*)k_pages, (const bf16*)v_pages, page_table, table_stride, seq_start, seq_past, n_seqs,
        gate, gate_stride, gate_bias, (bf16*)out, scale, nh, nkv, dim, vdim, terms);
  SYN_LAUNCH_CHECK("window_attention_prefill");
  return 0;
}
