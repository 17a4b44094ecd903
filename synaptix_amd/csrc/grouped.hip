// Products of rows with one of several weight matrices, chosen by the row's group:
//
//   out[orow(r), b, n] = epilogue( sum_k A[arow(r), b, k] * W[b, n, k] )         b: the group (an expert, a head)
//
// Two ways to say which rows meet which matrix:
//   * segments: seg_start[b] <= r < seg_start[b + 1] are the rows of group b (tokens sorted by expert), with
//     arow(r) = a_rows[r] and orow(r) = o_rows[r] gathered through index lists;
//   * every group takes all M rows (a linear map for each head of a token): A, W and out move on by a fixed
//     number of elements from one group to the next.
// Epilogue, in this order and each optional: the exact GELU 0.5 z (1 + erf(z / sqrt 2)); a weight of the row;
// sigmoid of a gate value read from float rows.  Or, with `pair`: W's rows come in pairs (2 j: the gate row of output j,
// 2 j + 1: its up row) and what is stored is the gated activation of the two sums (gated, csrc/common.h), N / 2 columns.  Sums are 32-bit.  bf16 operands whose K is a multiple of 32 run on
// the matrix cores: with few rows a group 16x16x32 with operands straight from memory as 16-byte pieces of rows (no
// LDS: a wave computes 32 rows x 64 columns), with many rows tiles of 128 x 128 through LDS (any K that is a multiple
// of 8); everything else, and all of the 32-bit path, is plain FMA with one wave a (row, 8 columns).
//
// Beside it: the choice of a mixture's router (the largest `top` logits of a token, softmax over those) and the
// counting sort that turns the choices into segments.
#include "common.h"

struct GroupedArgs {
  const void* a;
  long lda, a_group;        // A[row, group, k] = a[row * lda + group * a_group + k]
  const void* w;
  long w_group, ldw;        // W[group, n, k] = w[group * w_group + n * ldw + k]
  void* out;
  long ldo, o_group;        // out[row, group, n] = out[row * ldo + group * o_group + n]
  int out_is_f32;
  const int* seg_start;     // [groups + 1], or null: every group takes rows 0 .. M - 1
  const int* a_rows;        // [rows] or null
  const int* o_rows;        // [rows] or null
  const float* row_weight;  // [rows] or null
  const float* gate;        // or null: gate[row * gate_ld + group * gate_group + n * gate_col]
  long gate_ld, gate_group;
  int gate_col;
  int act;                  // 0: none, 1: exact GELU
  int pair;                 // 0: none; else 1 + the code of the gated activation over pairs of rows of W
  float limit;              // that activation's bound, if it has one
  int M, N, K, groups;
  int w_packed;             // W[group] lies in the order of the fragments: [N / 16][K / 32][64 lanes][8] with
                            // lane = 16 (k % 32 / 8) + n % 16 (bf16, N a multiple of 16, K of 32); 0: plain rows
};

// element (n, k) of a matrix in fragment order, K32 = K / 32
__device__ __forceinline__ size_t packed_at(int n, int k, int K32) {
  return ((size_t)(n >> 4) * K32 + (k >> 5)) * 512 + (((k & 31) >> 3) << 7) + ((n & 15) << 3) + (k & 7);
}

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }

__device__ __forceinline__ float grouped_epilogue(const GroupedArgs& g, float v, int r, int b, int n) {
  if (g.act == 1) v = gelu_erf(v);
  if (g.row_weight) v *= g.row_weight[r];
  if (g.gate) {
    const float z = g.gate[(size_t)r * g.gate_ld + (size_t)b * g.gate_group + (size_t)n * g.gate_col];
    v *= 1.f / (1.f + expf(-z));
  }
  return v;
}

// the pair (gate sum, up sum) of output column n / 2 (n even)
__device__ __forceinline__ float grouped_pair(const GroupedArgs& g, float gate, float up, int r) {
  float v = gated(g.pair - 1, gate, up, g.limit);
  if (g.row_weight) v *= g.row_weight[r];
  return v;
}

__device__ __forceinline__ void grouped_store(const GroupedArgs& g, int r, int b, int n, float v) {
  const int orow = g.o_rows ? g.o_rows[r] : r;
  const size_t at = (size_t)orow * g.ldo + (size_t)b * g.o_group + n;
  if (g.out_is_f32) ((float*)g.out)[at] = v;
  else ((bf16*)g.out)[at] = (bf16)v;
}

// ---------------------------------------------------------------- plain FMA: one wave a (row, 8 columns)
template <typename T>
__global__ void __launch_bounds__(256) grouped_product_simt_kernel(GroupedArgs g) {
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE;
  int r = blockIdx.x, b = blockIdx.z;
  if (g.seg_start) {
    // the group whose segment holds row r (segments are in order and cover 0 .. seg_start[groups] - 1)
    if (r >= g.seg_start[g.groups]) return;
    int lo = 0, hi = g.groups;
    while (hi - lo > 1) {
      const int mid = (lo + hi) / 2;
      if (g.seg_start[mid] <= r) lo = mid; else hi = mid;
    }
    b = lo;
  }
  const int n0 = (blockIdx.y * 4 + wave) * 8;
  if (n0 >= g.N) return;
  const int arow = g.a_rows ? g.a_rows[r] : r;
  const T* a = (const T*)g.a + (size_t)arow * g.lda + (size_t)b * g.a_group;
  const T* w = (const T*)g.w + (size_t)b * g.w_group;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int k = lane; k < g.K; k += SYN_WAVE) {
    const float x = to_f32<T>(a[k]);
#pragma unroll
    for (int c = 0; c < 8; ++c)
      if (n0 + c < g.N)
        acc[c] = fmaf(x, to_f32<T>(w[g.w_packed ? packed_at(n0 + c, k, g.K / 32) : (size_t)(n0 + c) * g.ldw + k]), acc[c]);
  }
  if (g.pair) {
#pragma unroll
    for (int c = 0; c < 8; c += 2) {
      const float gate = wave_sum(acc[c]), up = wave_sum(acc[c + 1]);
      if (lane == 0 && n0 + c < g.N) grouped_store(g, r, b, (n0 + c) / 2, grouped_pair(g, gate, up, r));
    }
    return;
  }
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    const float v = wave_sum(acc[c]);
    if (lane == 0 && n0 + c < g.N) grouped_store(g, r, b, n0 + c, grouped_epilogue(g, v, r, b, n0 + c));
  }
}

// ---------------------------------------------------------------- bf16 on the matrix cores
// D = W_tile (16 outputs x 32 k) . A_tile^T (32 k x 16 rows): a lane then holds four consecutive outputs of one row.
// Both operands are 16-byte pieces of rows (8 k-values of lane group lane / 16), so whatever order the instruction
// gives the k-values inside a lane group, the two operands agree.
#define GP_TM 32
// NB: blocks of 16 outputs a wave (4: 64 outputs; 1: 16 outputs, four times the waves, where few groups have rows and
// each group's matrix has to be streamed by more than a few waves).
template <int NB>
__global__ void __launch_bounds__(256) grouped_product_mfma_kernel(GroupedArgs g) {
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, i = lane % 16, q = lane / 16;
  int b = blockIdx.z, row0, row_end;
  if (g.seg_start) {
    int t = blockIdx.x;
    b = -1;
    for (int e = 0; e < g.groups; ++e) {
      const int s0 = g.seg_start[e], n = g.seg_start[e + 1] - s0, tiles = (n + GP_TM - 1) / GP_TM;
      if (t < tiles) {
        b = e, row0 = s0 + t * GP_TM, row_end = s0 + n;
        break;
      }
      t -= tiles;
    }
    if (b < 0) return;
  } else {
    row0 = blockIdx.x * GP_TM, row_end = g.M;
    if (row0 >= row_end) return;
  }
  const int n0 = (blockIdx.y * 4 + wave) * 16 * NB;
  if (n0 >= g.N) return;
  const bf16* A = (const bf16*)g.a + (size_t)b * g.a_group;
  const bf16* W = (const bf16*)g.w + (size_t)b * g.w_group;
  // rows beyond the segment and outputs beyond N read row 0 (a valid address) and count as zeros
  const bf16* arow[2];
  bool a_ok[2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int r = row0 + mb * 16 + i;
    a_ok[mb] = r < row_end;
    const int src = a_ok[mb] ? (g.a_rows ? g.a_rows[r] : r) : (g.a_rows ? g.a_rows[row0] : row0);
    arow[mb] = A + (size_t)src * g.lda + q * 8;
  }
  const bf16* wrow[NB];
  bool w_ok[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int n = n0 + nb * 16 + i;
    w_ok[nb] = n < g.N;
    // (in fragment order a wave's load of a k-step is 1 KB of consecutive bytes, and the next k-step lies 1 KB on)
    wrow[nb] = g.w_packed ? W + (size_t)((w_ok[nb] ? n : 0) >> 4) * (g.K / 32) * 512 + lane * 8
                          : W + (size_t)(w_ok[nb] ? n : 0) * g.ldw + q * 8;
  }
  const int w_step = g.w_packed ? 512 : 32;          // elements from one k-step of 32 to the next
  f32x4 acc[2][NB];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  // several k-steps at a time: their loads (24) are asked for together (a group's matrix is read once, as a stream), then
  // multiplied; the k-steps that are left over follow one by one
  constexpr int AHEAD = NB == 1 ? 8 : 4;
  int k0 = 0;
  for (; k0 + 32 * AHEAD <= g.K; k0 += 32 * AHEAD) {
    bf16x8 xa[AHEAD][2], xw[AHEAD][NB];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) xa[u][mb] = *(const bf16x8*)(arow[mb] + k0 + 32 * u);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) xw[u][nb] = __builtin_nontemporal_load((const bf16x8*)(wrow[nb] + (size_t)(k0 / 32 + u) * w_step));
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
#pragma unroll
      for (int mb = 0; mb < 2; ++mb) xa[u][mb] = a_ok[mb] ? xa[u][mb] : zero;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) xw[u][nb] = w_ok[nb] ? xw[u][nb] : zero;
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xw[u][nb], xa[u][mb], acc[mb][nb], 0, 0, 0);
    }
  }
  for (; k0 < g.K; k0 += 32) {
    bf16x8 xa[2], xw[NB];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) xa[mb] = a_ok[mb] ? *(const bf16x8*)(arow[mb] + k0) : zero;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) xw[nb] = w_ok[nb] ? *(const bf16x8*)(wrow[nb] + (size_t)(k0 / 32) * w_step) : zero;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xw[nb], xa[mb], acc[mb][nb], 0, 0, 0);
  }
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int r = row0 + mb * 16 + i;
    if (r >= row_end) continue;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = n0 + nb * 16 + q * 4 + e;
        if (g.pair) {      // (a lane holds four consecutive outputs: two pairs)
          if (e % 2 == 0 && n < g.N) grouped_store(g, r, b, n / 2, grouped_pair(g, acc[mb][nb][e], acc[mb][nb][e + (e % 2 == 0)], r));
        } else if (n < g.N) {
          grouped_store(g, r, b, n, grouped_epilogue(g, acc[mb][nb][e], r, b, n));
        }
      }
  }
}

// ---------------------------------------------------------------- bf16 on the matrix cores, many rows a group
// Tiles of 128 rows x 128 outputs x 64 k through LDS (double-buffered: while one k-tile is multiplied the next is on
// its way from memory into registers), four waves of 64 x 64 each, MFMA 32x32x16: A = rows of x, B = rows of W,
// D[m = 8 (e / 4) + 4 (lane / 32) + e % 4][n = lane % 32].  Rows of x are gathered through a_rows on their way into
// LDS.  K is a multiple of 8 (a 16-byte chunk lies inside or outside as a whole).
#define GT_BM 128
#define GT_BN 128
#define GT_BK 64
#define GT_LD (GT_BK + 8)
template <bool PAIR>
__global__ void __launch_bounds__(256) grouped_product_tiled_kernel(GroupedArgs g) {
  extern __shared__ __attribute__((aligned(16))) bf16 smem[];      // [2][(GT_BM + GT_BN) * GT_LD]
  const int tid = threadIdx.x, wave = tid / SYN_WAVE, lane = tid % SYN_WAVE;
  // Workgroups go to the eight XCDs in turns, each with an L2 of its own: workgroup w takes place
  // (w % 8) * (places / 8) + w / 8 of the order (row tile, column tile), so that one XCD walks the column tiles of a
  // few row tiles: it reads those rows of x once, and a group's matrix for the group's few row tiles in a row.
  const int col_tiles = (g.N + GT_BN - 1) / GT_BN;
  const int places = gridDim.x;                       // a multiple of 8
  const int place = (blockIdx.x % 8) * (places / 8) + blockIdx.x / 8;
  int b = blockIdx.z, row0, row_end;
  if (g.seg_start) {
    int t = place / col_tiles;
    b = -1;
    for (int e = 0; e < g.groups; ++e) {
      const int s0 = g.seg_start[e], n = g.seg_start[e + 1] - s0, tiles = (n + GT_BM - 1) / GT_BM;
      if (t < tiles) {
        b = e, row0 = s0 + t * GT_BM, row_end = s0 + n;
        break;
      }
      t -= tiles;
    }
    if (b < 0) return;                      // (the whole workgroup, before any barrier)
  } else {
    row0 = (place / col_tiles) * GT_BM, row_end = g.M;
    if (row0 >= row_end) return;
  }
  const int n0 = (place % col_tiles) * GT_BN;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;
  constexpr int CPR = GT_BK / 8, RPP = 256 / CPR, XL = GT_BM / RPP, WL = GT_BN / RPP;
  const int lrow = tid / CPR, lchunk = (tid % CPR) * 8;
  const bf16* A = (const bf16*)g.a + (size_t)b * g.a_group;
  const bf16* W = (const bf16*)g.w + (size_t)b * g.w_group;
  const bf16* xg[XL];
  const bf16* wg[WL];
  bool xin[XL], win[WL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int r = row0 + lrow + RPP * i;
    xin[i] = r < row_end;
    const int src = xin[i] ? (g.a_rows ? g.a_rows[r] : r) : 0;
    xg[i] = A + (size_t)src * g.lda + lchunk;
  }
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int n = n0 + lrow + RPP * i;
    win[i] = n < g.N;
    const int nn = win[i] ? n : 0;
    wg[i] = g.w_packed ? W + (size_t)(nn >> 4) * (g.K / 32) * 512 + ((nn & 15) << 3) + ((lchunk >> 5) << 9) + (((lchunk & 31) >> 3) << 7)
                       : W + (size_t)nn * g.ldw + lchunk;
  }
  const int w_tile = g.w_packed ? (GT_BK / 32) * 512 : GT_BK;      // elements from one k-tile to the next
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int nk = (g.K + GT_BK - 1) / GT_BK;
  bf16x8 rx[XL], rw[WL];
  auto fetch = [&](int kt) {
    const int k = kt * GT_BK;
    const bool kin = k + lchunk < g.K;
#pragma unroll
    for (int i = 0; i < XL; ++i) rx[i] = (kin && xin[i]) ? *(const bf16x8*)(xg[i] + k) : zero;
#pragma unroll
    for (int i = 0; i < WL; ++i) rw[i] = (kin && win[i]) ? *(const bf16x8*)(wg[i] + (size_t)kt * w_tile) : zero;
  };
  auto stash = [&](int buf) {
    bf16* xs = smem + buf * (GT_BM + GT_BN) * GT_LD;
    bf16* ws = xs + GT_BM * GT_LD;
#pragma unroll
    for (int i = 0; i < XL; ++i) *(bf16x8*)(xs + (lrow + RPP * i) * GT_LD + lchunk) = rx[i];
#pragma unroll
    for (int i = 0; i < WL; ++i) *(bf16x8*)(ws + (lrow + RPP * i) * GT_LD + lchunk) = rw[i];
  };
  fetch(0);
  stash(0);
  __syncthreads();
  const int fr = lane % 32, fk = (lane / 32) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) fetch(kt + 1);
    const bf16* xs = smem + buf * (GT_BM + GT_BN) * GT_LD;
    const bf16* ws = xs + GT_BM * GT_LD;
#pragma unroll
    for (int ks = 0; ks < GT_BK; ks += 16) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = *(const bf16x8*)(xs + (wm + i * 32 + fr) * GT_LD + ks + fk);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = *(const bf16x8*)(ws + (wn + j * 32 + fr) * GT_LD + ks + fk);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) stash(buf ^ 1);      // the other buffer was last read before the previous barrier
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int r = row0 + wm + i * 32 + 8 * (e / 4) + 4 * (lane / 32) + e % 4;
        const int n = n0 + wn + j * 32 + lane % 32;
        if constexpr (PAIR) {      // (neighbouring lanes hold neighbouring outputs: the even lane takes its neighbour's up sum)
          const float up = __shfl_xor(acc[i][j][e], 1, SYN_WAVE);
          if (lane % 2 == 0 && r < row_end && n < g.N) grouped_store(g, r, b, n / 2, grouped_pair(g, acc[i][j][e], up, r));
        } else if (r < row_end && n < g.N) {
          grouped_store(g, r, b, n, grouped_epilogue(g, acc[i][j][e], r, b, n));
        }
      }
}

// rows_bound: with segments, the number of rows in all segments together (what the index lists hold)
SYN_EXPORT int syn_grouped_product(const void* a, long lda, long a_group, const void* w, long w_group, long ldw, void* out,
                                   long ldo, long o_group, int in_is_f32, int out_is_f32, const int* seg_start,
                                   const int* a_rows, const int* o_rows, const float* row_weight, const float* gate,
                                   long gate_ld, long gate_group, int gate_col, int act, int M, int N, int K, int groups,
                                   int rows_bound, int force_simt, int w_packed, int pair, float limit,
                                   hipStream_t stream) {
  SYN_CHECK(M > 0 && N > 0 && K > 0 && groups > 0, "grouped_product: empty input (%d rows, %d x %d, %d groups)", M, N, K, groups);
  SYN_CHECK(act == 0 || act == 1, "grouped_product: unknown activation code %d", act);
  SYN_CHECK(pair >= 0 && pair <= SYN_ACT_COUNT && (pair == 0 || (N % 2 == 0 && act == 0 && gate == nullptr)),
            "grouped_product: a gated activation (code %d) over %d rows of W in pairs, with no other activation", pair - 1, N);
  SYN_CHECK(seg_start != nullptr || (a_rows == nullptr && o_rows == nullptr && row_weight == nullptr),
            "grouped_product: index lists and row weights come with segments");
  SYN_CHECK(seg_start == nullptr || rows_bound > 0, "grouped_product: segments over %d rows", rows_bound);
  SYN_CHECK(seg_start == nullptr || gate == nullptr, "grouped_product: a gate is read by row and group, not through segments");
  SYN_CHECK(!w_packed || (!in_is_f32 && N % 16 == 0 && K % 32 == 0),
            "grouped_product: matrices in fragment order are bf16 of %d x %d (multiples of 16 and 32)?", N, K);
  const GroupedArgs g = {a, lda, a_group, w, w_group, ldw, out, ldo, o_group, out_is_f32, seg_start, a_rows, o_rows,
                         row_weight, gate, gate_ld, gate_group, gate_col, act, pair, limit, M, N, K, groups, w_packed};
  const bool aligned = K % 32 == 0 && lda % 8 == 0 && a_group % 8 == 0 && ldw % 8 == 0 && w_group % 8 == 0 &&
                       (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
  // many rows a group (on average, where the host does not know the segments): the tiles through LDS
  const long rows_a_group = seg_start ? rows_bound / groups : M;
  const bool chunks = K % 8 == 0 && lda % 8 == 0 && a_group % 8 == 0 && ldw % 8 == 0 && w_group % 8 == 0 &&
                      (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
  if (!in_is_f32 && chunks && force_simt == 0 && rows_a_group >= 48) {
    const int row_tiles = seg_start ? (rows_bound + GT_BM - 1) / GT_BM + groups : (M + GT_BM - 1) / GT_BM;
    const int places = (row_tiles * ((N + GT_BN - 1) / GT_BN) + 7) / 8 * 8;
    const dim3 grid(places, 1, seg_start ? 1 : groups);
    const size_t lds = (size_t)2 * (GT_BM + GT_BN) * GT_LD * sizeof(bf16);
    static OncePerDevice raised;
    const hipError_t e = once_per_device(raised, [&] {
      const hipError_t r = hipFuncSetAttribute((const void*)grouped_product_tiled_kernel<false>,
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      return r != hipSuccess ? r : hipFuncSetAttribute((const void*)grouped_product_tiled_kernel<true>,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    SYN_CHECK(e == hipSuccess, "grouped_product: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
    if (pair) grouped_product_tiled_kernel<true><<<grid, 256, lds, stream>>>(g);
    else grouped_product_tiled_kernel<false><<<grid, 256, lds, stream>>>(g);
  } else if (!in_is_f32 && aligned && force_simt != 1) {
    const int row_tiles = seg_start ? (rows_bound + GP_TM - 1) / GP_TM + groups : (M + GP_TM - 1) / GP_TM;
    const long wide = (long)row_tiles * ((N + 255) / 256) * (seg_start ? 1 : groups);
    // (force_simt 3: the wide waves whatever the sizes, for tests)
    if (wide >= 8L * syn_compute_units() || force_simt == 3) {
      const dim3 grid(row_tiles, (N + 255) / 256, seg_start ? 1 : groups);
      grouped_product_mfma_kernel<4><<<grid, 256, 0, stream>>>(g);
    } else {
      const dim3 grid(row_tiles, (N + 63) / 64, seg_start ? 1 : groups);
      grouped_product_mfma_kernel<1><<<grid, 256, 0, stream>>>(g);
    }
  } else {
    const dim3 grid(seg_start ? rows_bound : M, (N + 31) / 32, seg_start ? 1 : groups);
    if (in_is_f32) grouped_product_simt_kernel<float><<<grid, 256, 0, stream>>>(g);
    else grouped_product_simt_kernel<bf16><<<grid, 256, 0, stream>>>(g);
  }
  SYN_LAUNCH_CHECK("grouped_product");
  return 0;
}

// ---------------------------------------------------------------- router: the largest `top` logits, their softmax
// One wave a token over its row of logits z [E] (32-bit sums of a product that ran before) + bias; of equal logits
// the lower index comes first.
#define ROUTE_MAX_EXPERTS 1024
#define ROUTE_MAX_TOP 64
__global__ void __launch_bounds__(256) route_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                         int* __restrict__ ids, float* __restrict__ weights,
                                                         int n_tokens, int E, int top) {
  __shared__ float zs[4][ROUTE_MAX_EXPERTS];
  __shared__ float chosen_s[4][ROUTE_MAX_TOP];
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, tok = blockIdx.x * 4 + wave;
  if (tok >= n_tokens) return;             // (waves work alone: no barrier of the workgroup below)
  float* z = zs[wave];
  float* chosen = chosen_s[wave];
  for (int e = lane; e < E; e += SYN_WAVE) z[e] = logits[(size_t)tok * E + e] + (bias ? bias[e] : 0.f);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (int t = 0; t < top; ++t) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += SYN_WAVE) {
      const float v = z[e];
      if (v > best) best = v, at = e;      // (a lane meets its experts in rising order)
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, SYN_WAVE);
      const int oa = __shfl_xor(at, off, SYN_WAVE);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    if (lane == 0) {
      if (at >= E) at = t;          // every logit left is NaN or -inf: any expert, and no access beyond the table
      ids[(size_t)tok * top + t] = at;
      chosen[t] = best;
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (lane == 0) {
    const float m = chosen[0];      // the first chosen is the largest
    float sum = 0.f;
    for (int t = 0; t < top; ++t) sum += expf(chosen[t] - m);
    for (int t = 0; t < top; ++t) weights[(size_t)tok * top + t] = expf(chosen[t] - m) / sum;
  }
}

SYN_EXPORT int syn_route_topk(const float* logits, const float* bias, int* ids, float* weights, int n_tokens, int E,
                              int top, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0, "route_topk: empty input");
  SYN_CHECK(E > 0 && E <= ROUTE_MAX_EXPERTS, "route_topk: %d experts (at most %d)", E, ROUTE_MAX_EXPERTS);
  SYN_CHECK(top > 0 && top <= E && top <= ROUTE_MAX_TOP, "route_topk: the %d largest of %d (at most %d)", top, E, ROUTE_MAX_TOP);
  route_topk_kernel<<<(n_tokens + 3) / 4, 256, 0, stream>>>(logits, bias, ids, weights, n_tokens, E, top);
  SYN_LAUNCH_CHECK("route_topk");
  return 0;
}

// ---------------------------------------------------------------- a router that scores all experts
// s = softmax(logits) over all E outputs (32-bit).  The choice is made on s + correction: the E outputs form n_groups
// equal groups of neighbours, a group's score is its largest choice score, only members of the keep_groups best groups
// can be chosen (the others count as minus infinity), and of those the `top` largest are taken (the lower index of
// equal ones, for groups and for experts).  weights: the chosen experts' s itself, without the correction; renorm:
// divided by their sum.  One wave a token.
__global__ void __launch_bounds__(256) route_scores_kernel(const float* __restrict__ logits, const float* __restrict__ correction,
                                                           int* __restrict__ ids, float* __restrict__ weights, int n_tokens,
                                                           int E, int ld, int top, int n_groups, int keep_groups, int renorm,
                                                           float scale) {
  __shared__ float ss[4][ROUTE_MAX_EXPERTS];       // the scores
  __shared__ float cs[4][ROUTE_MAX_EXPERTS];       // the choice scores
  __shared__ float gs[4][ROUTE_MAX_EXPERTS];       // the groups' scores
  __shared__ float chosen_s[4][ROUTE_MAX_TOP];
  const int wave = threadIdx.x / SYN_WAVE, lane = threadIdx.x % SYN_WAVE, tok = blockIdx.x * 4 + wave;
  if (tok >= n_tokens) return;             // (waves work alone: no barrier of the workgroup below)
  float* sc = ss[wave];
  float* c = cs[wave];
  float* grp = gs[wave];
  float* chosen = chosen_s[wave];
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  float mx = -INFINITY;
  for (int e = lane; e < E; e += SYN_WAVE) mx = fmaxf(mx, logits[(size_t)tok * ld + e]);
  mx = wave_max(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += SYN_WAVE) {
    const float p = expf(logits[(size_t)tok * ld + e] - mx);
    sc[e] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  const int per = E / n_groups;
  for (int e = lane; e < E; e += SYN_WAVE) {
    sc[e] = sc[e] / sum;
    c[e] = sc[e] + (correction ? correction[e] : 0.f);
  }
  wave_sync();
  if (keep_groups < n_groups) {
    for (int g = lane; g < n_groups; g += SYN_WAVE) {
      float best = -INFINITY;
      for (int j = 0; j < per; ++j) best = fmaxf(best, c[g * per + j]);
      grp[g] = best;
    }
    wave_sync();
    // a group stays if fewer than keep_groups others come before it (a larger score, or an equal one at a lower index)
    for (int g = lane; g < n_groups; g += SYN_WAVE) {
      int before = 0;
      for (int o = 0; o < n_groups; ++o) before += (grp[o] > grp[g] || (grp[o] == grp[g] && o < g)) ? 1 : 0;
      if (before >= keep_groups)
        for (int j = 0; j < per; ++j) c[g * per + j] = -INFINITY;
    }
    wave_sync();
  }
  for (int t = 0; t < top; ++t) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < E; e += SYN_WAVE) {
      const float v = c[e];
      if (v > best) best = v, at = e;      // (a lane meets its experts in rising order)
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, SYN_WAVE);
      const int oa = __shfl_xor(at, off, SYN_WAVE);
      if (ob > best || (ob == best && oa < at)) best = ob, at = oa;
    }
    if (lane == 0) {
      if (at >= E) at = t;          // nothing left to choose from: any expert, and no access beyond the table
      ids[(size_t)tok * top + t] = at;
      chosen[t] = sc[at];
      c[at] = -INFINITY;
    }
    wave_sync();
  }
  if (lane == 0) {
    float total = 1.f;
    if (renorm) {
      total = 0.f;
      for (int t = 0; t < top; ++t) total += chosen[t];
    }
    for (int t = 0; t < top; ++t) weights[(size_t)tok * top + t] = chosen[t] / total * scale;
  }
}

// logits: rows of `ld` values whose first E are the router's outputs; weights: the chosen scores (over their sum with
// renorm) times `scale`
SYN_EXPORT int syn_route_scores(const float* logits, const float* correction, int* ids, float* weights, int n_tokens, int E,
                                int ld, int top, int n_groups, int keep_groups, int renorm, float scale, hipStream_t stream) {
  SYN_CHECK(ld >= E, "route_scores: rows of %d values for %d experts", ld, E);
  SYN_CHECK(n_tokens > 0, "route_scores: empty input");
  SYN_CHECK(E > 0 && E <= ROUTE_MAX_EXPERTS, "route_scores: %d experts (at most %d)", E, ROUTE_MAX_EXPERTS);
  SYN_CHECK(n_groups > 0 && E % n_groups == 0 && keep_groups > 0 && keep_groups <= n_groups,
            "route_scores: %d experts in %d groups of which %d stay", E, n_groups, keep_groups);
  SYN_CHECK(top > 0 && top <= ROUTE_MAX_TOP && top <= keep_groups * (E / n_groups),
            "route_scores: the %d largest of %d groups of %d (at most %d)", top, keep_groups, E / n_groups, ROUTE_MAX_TOP);
  route_scores_kernel<<<(n_tokens + 3) / 4, 256, 0, stream>>>(logits, correction, ids, weights, n_tokens, E, ld, top, n_groups,
                                                             keep_groups, renorm, scale);
  SYN_LAUNCH_CHECK("route_scores");
  return 0;
}

// Experts that are the identity: for the places r of seg_start[first] .. seg_start[last] (the segments of the experts
// first .. last - 1 after the sort), out[o_rows[r]] = weight_of[r] * x[a_rows[r]].  x [*, H] in the engine's type, out
// [*, H] float.  One workgroup a place of the list; those outside the range leave at once.
template <typename T>
__global__ void __launch_bounds__(256) route_identity_kernel(const T* __restrict__ x, float* __restrict__ out,
                                                             const int* __restrict__ seg_start, int first, int last,
                                                             const int* __restrict__ a_rows, const int* __restrict__ o_rows,
                                                             const float* __restrict__ weight_of, int H) {
  const int r = blockIdx.x;
  if (r < seg_start[first] || r >= seg_start[last]) return;
  const T* src = x + (size_t)a_rows[r] * H;
  float* dst = out + (size_t)o_rows[r] * H;
  const float w = weight_of[r];
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = w * to_f32<T>(src[i]);
}

SYN_EXPORT int syn_route_identity(const void* x, int is_f32, float* out, const int* seg_start, int first, int last,
                                  const int* a_rows, const int* o_rows, const float* weight_of, int places, int H,
                                  hipStream_t stream) {
  SYN_CHECK(places > 0 && H > 0 && first >= 0 && last >= first, "route_identity: empty input");
  if (last == first) return 0;
  if (is_f32)
    route_identity_kernel<float><<<places, 256, 0, stream>>>((const float*)x, out, seg_start, first, last, a_rows, o_rows,
                                                             weight_of, H);
  else
    route_identity_kernel<bf16><<<places, 256, 0, stream>>>((const bf16*)x, out, seg_start, first, last, a_rows, o_rows,
                                                            weight_of, H);
  SYN_LAUNCH_CHECK("route_identity");
  return 0;
}

// ---------------------------------------------------------------- the router's choices as segments
// P = n_tokens * top pairs (token n, its t-th expert), pair p = n * top + t.  Sorted by expert:
//   seg_start[e] .. seg_start[e + 1]: the places of expert e;  for a place r:
//   tok_of[r] = n, pair_of[r] = p, part_of[r] = t * n_tokens + n (the pair's row in partial sums [top, n_tokens]),
//   weight_of[r] = weights[p].
// One workgroup.  The order inside a segment is the order of arrival; no result depends on it (a row's sums do not
// depend on its place in a tile).
__global__ void __launch_bounds__(1024) route_sort_kernel(const int* __restrict__ ids, const float* __restrict__ weights,
                                                          int* __restrict__ seg_start, int* __restrict__ tok_of,
                                                          int* __restrict__ pair_of, int* __restrict__ part_of,
                                                          float* __restrict__ weight_of, int n_tokens, int top, int E) {
  __shared__ int count[ROUTE_MAX_EXPERTS];
  __shared__ int cursor[ROUTE_MAX_EXPERTS];
  const int P = n_tokens * top;
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&count[min(max(ids[p], 0), E - 1)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      cursor[e] = at;
      seg_start[e] = at;
      at += count[e];
    }
    seg_start[E] = at;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int r = atomicAdd(&cursor[min(max(ids[p], 0), E - 1)], 1);
    const int n = p / top, t = p % top;
    tok_of[r] = n;
    pair_of[r] = p;
    part_of[r] = t * n_tokens + n;
    weight_of[r] = weights[p];
  }
}

SYN_EXPORT int syn_route_sort(const int* ids, const float* weights, int* seg_start, int* tok_of, int* pair_of,
                              int* part_of, float* weight_of, int n_tokens, int top, int E, hipStream_t stream) {
  SYN_CHECK(n_tokens > 0 && top > 0, "route_sort: empty input");
  SYN_CHECK(E > 0 && E <= ROUTE_MAX_EXPERTS, "route_sort: %d experts (at most %d)", E, ROUTE_MAX_EXPERTS);
  SYN_CHECK((long)n_tokens * top < (1L << 30), "route_sort: %d tokens x %d", n_tokens, top);
  route_sort_kernel<<<1, 1024, 0, stream>>>(ids, weights, seg_start, tok_of, pair_of, part_of, weight_of, n_tokens, top, E);
  SYN_LAUNCH_CHECK("route_sort");
  return 0;
}
