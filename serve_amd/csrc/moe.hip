// Routed experts: every token takes the `top` experts with the largest router logits, weighted by the
// softmax over those logits alone (or: by their shares of the softmax over all experts, divided by the sum
// of the chosen shares + 1e-20; or: by the sigmoid of each chosen logit as it is; each times a constant); an expert
// is down(gate(gate x, up x)) with one of the gates of common.h (silu(g) u and others).  The weight multiplies the
// expert's output (in `combine`), or, where a design says so, its input: gate and up are linear in x, so
// expert(w x) = down(gate(w gate x, w up x)), and the weight enters where the gate is applied.
//
// Nothing is read back to the host: the tokens are grouped by expert on the device, and the
// products run over a list of (expert, rows) tiles that is built there, from a grid sized for
// the worst case whose surplus workgroups leave at once.
//
//   route     logits fp32 [T, ldz] -> ids int32 [T, top], weights fp32 [T, top]
//   group     ids -> offsets[E + 1], perm[T top] (row of the grouped order -> t * top + k),
//             tile_expert[], tile_row0[], num_tiles
//   gate_up   act[row, :] = silu(Wg_e x) * (Wu_e x),  x = h[perm[row] / top]
//   down      yk[perm[row], :] = Wd_e act[row, :]          (fp32)
//   combine   y[t, :] = sum_k weights[t, k] yk[t top + k, :]  (+ sigmoid(sg[t]) * shared[t, :])
//
// Products: bf16 on the matrix cores (moe_mfma_kernel); float32, and bf16 at sizes those do not take, as fp32
// sums on the vector ALU over LDS tiles (storage types templated).
#include "common.h"

#define MOE_TM 32
#define MOE_TN 64
#define MOE_TK 32

// ---------------------------------------------------------------------------------------------
// route: a wave per token.  Ties go to the lower index.
// ---------------------------------------------------------------------------------------------
// mode 1: the weights are shares of the softmax over all E logits, renormalised over the chosen ones
// (p_k / S) / (sum_chosen p / S + 1e-20) with S the sum over all; mode 0: p_k / sum_chosen p; mode 2: the sigmoid of
// every chosen logit, not normalised.  All times wscale.
__device__ __forceinline__ void route_token(const float* __restrict__ z, int* __restrict__ ids, float* __restrict__ wts,
                                            int E, int top, int lane, int mode, float wscale);

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int ldz, int* __restrict__ ids,
                                                        float* __restrict__ wts, int T, int E, int top, int over_all,
                                                        float wscale) {
  const int t = blockIdx.x * (blockDim.x / SA_WAVE) + threadIdx.x / SA_WAVE;
  if (t >= T) return;
  route_token(logits + (size_t)t * ldz, ids + (size_t)t * top, wts + (size_t)t * top, E, top,
              threadIdx.x & (SA_WAVE - 1), over_all, wscale);
}

__device__ __forceinline__ void route_token(const float* __restrict__ z, int* __restrict__ ids, float* __restrict__ wts,
                                            int E, int top, int lane, int mode, float wscale) {
  const int over_all = mode == 1;
  float prev_v = INFINITY;
  int prev_i = -1;
  float first = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    // the largest logit that comes after (prev_v, prev_i) in the order (value descending, index ascending)
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += SA_WAVE) {
      const float v = z[e];
      const bool after = v < prev_v || (v == prev_v && e > prev_i);
      if (after && (v > bv || (v == bv && e < bi))) { bv = v; bi = e; }
    }
#pragma unroll
    for (int o = SA_WAVE / 2; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, SA_WAVE);
      const int oi = __shfl_xor(bi, o, SA_WAVE);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (k == 0) first = bv;
    const float p = mode == 2 ? 1.f / (1.f + expf(-bv)) : expf(bv - first);
    sum += p;
    if (lane == 0) {
      ids[k] = bi;
      wts[k] = p;
    }
    prev_v = bv;
    prev_i = bi;
  }
  float all = 1.f;
  if (over_all) {
    // the softmax's denominator over every expert, with the largest logit taken off
    float part = 0.f;
    for (int e = lane; e < E; e += SA_WAVE) part += expf(z[e] - first);
    all = wave_sum(part);
  }
  if (lane == 0 && mode == 2) {
    for (int k = 0; k < top; ++k) wts[k] *= wscale;
  } else if (lane == 0) {
    const float denom = over_all ? sum / all + 1e-20f : sum;
    for (int k = 0; k < top; ++k) wts[k] = ((over_all ? wts[k] / all : wts[k]) / denom) * wscale;
  }
}

// ---------------------------------------------------------------------------------------------
// group: one workgroup.  Counts per expert, their running sum, the tiles, then every (token, k)
// takes the next free row of its expert (the order inside an expert does not matter: a row's sums
// do not depend on its place).  Up to MOE_LDS_EXPERTS experts the counters live in LDS, whose atomics
// on a few dozen addresses are far cheaper than the same through memory (thousands of rows of a prompt
// step on 32 experts: 64 us with the counters in memory).
// ---------------------------------------------------------------------------------------------
#define MOE_LDS_EXPERTS 1024
// counts, running sums and tiles, then the rows' places; `cursor`: E counters, in LDS or in memory
__device__ __forceinline__ void group_rows(const int* ids, int n, int E, int tile_rows, int* __restrict__ offsets,
                                           int* cursor, int* __restrict__ perm, int* __restrict__ tile_expert,
                                           int* __restrict__ tile_row0, int* __restrict__ num_tiles) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) atomicAdd(&cursor[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cursor[e];
      offsets[e] = run;
      for (int r0 = 0; r0 < c; r0 += tile_rows) {
        tile_expert[tiles] = e;
        tile_row0[tiles] = run + r0;
        ++tiles;
      }
      cursor[e] = run;
      run += c;
    }
    offsets[E] = run;
    *num_tiles = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) perm[atomicAdd(&cursor[ids[i]], 1)] = i;
}

__global__ __launch_bounds__(1024) void moe_group_kernel(const int* ids, int n, int E, int tile_rows,
                                                         int* __restrict__ offsets, int* __restrict__ cursor,
                                                         int* __restrict__ perm, int* __restrict__ tile_expert,
                                                         int* __restrict__ tile_row0, int* __restrict__ num_tiles,
                                                         const float* __restrict__ logits, int ldz, int* ids_out,
                                                         float* __restrict__ wts, int top, int over_all, float wscale) {
  __shared__ int lds_cursor[MOE_LDS_EXPERTS];
  const bool in_lds = E <= MOE_LDS_EXPERTS;              // (the counters are scratch: nobody reads them afterwards)
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    if (in_lds) lds_cursor[e] = 0;
    else cursor[e] = 0;
  }
  if (logits) {
    // a step of few tokens: the routing is done here, a wave a token in turn, and saves a kernel
    const int waves = blockDim.x / SA_WAVE, T = n / top;
    for (int t = threadIdx.x / SA_WAVE; t < T; t += waves)
      route_token(logits + (size_t)t * ldz, ids_out + (size_t)t * top, wts + (size_t)t * top, E, top,
                  threadIdx.x & (SA_WAVE - 1), over_all, wscale);
  }
  __syncthreads();
  if (in_lds) group_rows(ids, n, E, tile_rows, offsets, lds_cursor, perm, tile_expert, tile_row0, num_tiles);
  else group_rows(ids, n, E, tile_rows, offsets, cursor, perm, tile_expert, tile_row0, num_tiles);
}

// ---------------------------------------------------------------------------------------------
// The tile product: C[TM x TN] = A[TM x K] . W[TN x K]^T, both contiguous along K.  256 threads,
// thread (ty, tx) = (tid / 16, tid % 16) owns rows ty, ty + 16 and columns tx + 16 c, c < 4.
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TW, bool DUAL>
__device__ __forceinline__ void tile_product(const TA* __restrict__ A, const int* a_row_index,
                                             int a_stride, int rows, const TW* __restrict__ W0,
                                             const TW* __restrict__ W1, int n0, int N, int K, float acc0[2][4],
                                             float acc1[2][4], float (*sa)[MOE_TM + 1], float (*sw0)[MOE_TN + 1],
                                             float (*sw1)[MOE_TN + 1]) {
  const int tid = threadIdx.x;
  const int ty = tid >> 4, tx = tid & 15;
  for (int k0 = 0; k0 < K; k0 += MOE_TK) {
    __syncthreads();
    for (int idx = tid; idx < MOE_TM * MOE_TK; idx += 256) {
      const int r = idx / MOE_TK, k = idx - r * MOE_TK;
      float v = 0.f;
      if (r < rows && k0 + k < K) v = to_float(A[(size_t)a_row_index[r] * a_stride + k0 + k]);
      sa[k][r] = v;
    }
    for (int idx = tid; idx < MOE_TN * MOE_TK; idx += 256) {
      const int c = idx / MOE_TK, k = idx - c * MOE_TK;
      const bool in = n0 + c < N && k0 + k < K;
      sw0[k][c] = in ? to_float(W0[(size_t)(n0 + c) * K + k0 + k]) : 0.f;
      if (DUAL) sw1[k][c] = in ? to_float(W1[(size_t)(n0 + c) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < MOE_TK; ++k) {
      const float a0 = sa[k][ty], a1 = sa[k][ty + 16];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float w0 = sw0[k][tx + 16 * c];
        acc0[0][c] += a0 * w0;
        acc0[1][c] += a1 * w0;
        if (DUAL) {
          const float w1 = sw1[k][tx + 16 * c];
          acc1[0][c] += a0 * w1;
          acc1[1][c] += a1 * w1;
        }
      }
    }
  }
}

// gate_up: grid (max tiles, ceil(F / TN)).  Wg, Wu [E, F, d]; h [T, d]; act [T top, F] in grouped order.
template <typename TA>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const TA* __restrict__ h, const TA* __restrict__ Wg,
                                                          const TA* __restrict__ Wu, const int* __restrict__ offsets,
                                                          const int* __restrict__ perm, const int* __restrict__ tile_expert,
                                                          const int* __restrict__ tile_row0, const int* __restrict__ num_tiles,
                                                          TA* __restrict__ act, int top, int d, int F, int gate_kind,
                                                          float gate_limit, const float* __restrict__ in_wts) {
  __shared__ float sa[MOE_TK][MOE_TM + 1];
  __shared__ float sw0[MOE_TK][MOE_TN + 1];
  __shared__ float sw1[MOE_TK][MOE_TN + 1];
  __shared__ int rowidx[MOE_TM];
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile];
  const int rows = min(MOE_TM, offsets[e + 1] - row0);
  if (threadIdx.x < MOE_TM) rowidx[threadIdx.x] = threadIdx.x < rows ? perm[row0 + threadIdx.x] / top : 0;
  const int n0 = blockIdx.y * MOE_TN;
  float g[2][4] = {}, u[2][4] = {};
  tile_product<TA, TA, true>(h, rowidx, d, rows, Wg + (size_t)e * F * d, Wu + (size_t)e * F * d, n0, F, d, g, u,
                             sa, sw0, sw1);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int r = ty + 16 * rr;
    if (r >= rows) continue;
    const float w = in_wts ? in_wts[perm[row0 + r]] : 1.f;          // (the weight on the expert's input)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int n = n0 + tx + 16 * c;
      if (n < F) {
        act[(size_t)(row0 + r) * F + n] = from_float<TA>(gate_mul(g[rr][c] * w, u[rr][c] * w, gate_kind, gate_limit));
      }
    }
  }
}

// down: grid (max tiles, ceil(d / TN)).  Wd [E, d, F]; act [T top, F] grouped; yk fp32 [T top, d] by (t, k).
template <typename TA>
__global__ __launch_bounds__(256) void moe_down_kernel(const TA* __restrict__ act, const TA* __restrict__ Wd,
                                                       const int* __restrict__ offsets, const int* __restrict__ perm,
                                                       const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
                                                       const int* __restrict__ num_tiles, float* __restrict__ yk, int d,
                                                       int F) {
  __shared__ float sa[MOE_TK][MOE_TM + 1];
  __shared__ float sw0[MOE_TK][MOE_TN + 1];
  __shared__ int rowidx[MOE_TM];
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile];
  const int rows = min(MOE_TM, offsets[e + 1] - row0);
  if (threadIdx.x < MOE_TM) rowidx[threadIdx.x] = threadIdx.x < rows ? row0 + threadIdx.x : 0;
  const int n0 = blockIdx.y * MOE_TN;
  float acc[2][4] = {}, none[2][4];
  tile_product<TA, TA, false>(act, rowidx, F, rows, Wd + (size_t)e * d * F, nullptr, n0, d, F, acc, none, sa,
                              sw0, nullptr);
  const int ty = threadIdx.x >> 4, tx = threadIdx.x & 15;
#pragma unroll
  for (int rr = 0; rr < 2; ++rr) {
    const int r = ty + 16 * rr;
    if (r >= rows) continue;
    const size_t dst = (size_t)perm[row0 + r] * d;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int n = n0 + tx + 16 * c;
      if (n < d) yk[dst + n] = acc[rr][c];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same two products on the matrix cores (bf16, K % 8 == 0): v_mfma_f32_16x16x32_bf16 computes the
// transposed tile, operand "A" = 16 rows of the expert's matrix (lane l: row l % 16, k-slots 8 (l / 16) .. + 7),
// operand "B" = 16 rows of activations, and lane l gets outputs n = 4 (l / 16) .. + 3 of activation row l % 16.
// Weights and activations go from memory straight into registers, two steps of 32 along K ahead.
//   KS == 1: tiles of up to 16 MT rows; the four waves of a workgroup own four groups of 16 weight rows
//            and walk all of K (prompt portions: an expert's matrix is read once per 16 MT rows).
//   KS == 4: tiles of up to 16 rows (MT 1); the four waves cut K between them and add through LDS in a
//            fixed order (decode steps: few rows per expert, the chip is filled by cutting K and N).
// GATE_UP: rows come from h by perm[row] / top, two matrices, act = gate(gate, up) in bf16.
// else:    rows are act's own, one matrix, fp32 sums go to yk[perm[row]].
// ---------------------------------------------------------------------------------------------
typedef __bf16 moe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float moe_floatx4_t __attribute__((ext_vector_type(4)));
typedef unsigned int moe_u32x4_t __attribute__((ext_vector_type(4)));
union MoeFrag {
  moe_u32x4_t r;
  moe_bf16x8_t v;
};

template <int MT, int KS, bool GATE_UP, int WR = 1, int KU = 2>
__global__ __launch_bounds__(256) void moe_mfma_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W0,
                                                       const bf16_t* __restrict__ W1, const int* __restrict__ offsets,
                                                       const int* __restrict__ perm, const int* __restrict__ tile_expert,
                                                       const int* __restrict__ tile_row0, const int* __restrict__ num_tiles,
                                                       bf16_t* __restrict__ act, float* __restrict__ yk, int top, int N,
                                                       int K, int gate_kind, float gate_limit,
                                                       const float* __restrict__ in_wts) {
  // WR: groups of 16 weight rows a wave owns (per matrix); KU: steps of 32 along K whose loads are in flight together
  constexpr int NM = GATE_UP ? 2 : 1;
  constexpr int RT = NM * WR;
  static_assert(KS == 1 || WR == 1, "a cut K goes with one group of weight rows");
  __shared__ float red[KS > 1 ? KS : 1][KS > 1 ? RT * MT * 4 : 1][64];
  const int tile = blockIdx.x;
  if (tile >= *num_tiles) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile];
  const int rows = min(16 * MT, offsets[e + 1] - row0);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, c = lane & 15;
  const int n0 = (KS > 1 ? blockIdx.y : blockIdx.y * 4 + wave) * 16 * WR;
  if (KS == 1 && n0 >= N) return;
  const bf16_t* wp[RT];
#pragma unroll
  for (int wr = 0; wr < WR; ++wr) {
    const int nrow = min(n0 + wr * 16 + c, N - 1);
    wp[wr] = W0 + ((size_t)e * N + nrow) * K;
    if (GATE_UP) wp[WR + wr] = W1 + ((size_t)e * N + nrow) * K;
  }
  const bf16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int r = mt * 16 + c;
    const int src = row0 + (r < rows ? r : 0);
    arow[mt] = A + (size_t)(GATE_UP ? perm[src] / top : src) * K;
  }
  const int nchunks = (K + 31) >> 5;
  const int per = (nchunks + KS - 1) / KS;
  const int ch_begin = KS > 1 ? wave * per : 0;
  const int ch_end = KS > 1 ? min(nchunks, ch_begin + per) : nchunks;
  moe_floatx4_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (moe_floatx4_t){0.f, 0.f, 0.f, 0.f};
  const moe_u32x4_t zero = {0u, 0u, 0u, 0u};
  for (int ch = ch_begin; ch < ch_end; ch += KU) {
    MoeFrag wf[RT][KU], af[MT][KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int k = min((ch + u) * 32 + g * 8, K - 8);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wf[rt][u].r = *reinterpret_cast<const moe_u32x4_t*>(wp[rt] + k);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) af[mt][u].r = *reinterpret_cast<const moe_u32x4_t*>(arow[mt] + k);
    }
    if (ch + KU > ch_end || (ch + KU) * 32 > K) {          // the last, partial round of the slice
#pragma unroll
      for (int u = 0; u < KU; ++u) {
        const bool kin = (ch + u) < ch_end && (ch + u) * 32 + g * 8 < K;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) af[mt][u].r = kin ? af[mt][u].r : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < KU; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][u].v, af[mt][u].v, acc[rt][mt], 0, 0, 0);
  }
  if (KS > 1) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][(rt * MT + mt) * 4 + r][lane] = acc[rt][mt][r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float sum = acc[rt][mt][r];
          for (int w = 1; w < KS; ++w) sum += red[w][(rt * MT + mt) * 4 + r][lane];
          acc[rt][mt][r] = sum;
        }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + c;
    if (m >= rows) continue;
    const float w = GATE_UP && in_wts ? in_wts[perm[row0 + m]] : 1.f;          // (the weight on the expert's input)
#pragma unroll
    for (int wr = 0; wr < WR; ++wr) {
      const int n = n0 + wr * 16 + 4 * g;
      if (GATE_UP) {
        bf16_t* dst = act + (size_t)(row0 + m) * N + n;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N)
            dst[r] = from_float<bf16_t>(gate_mul(acc[wr][mt][r] * w, acc[RT - WR + wr][mt][r] * w, gate_kind, gate_limit));
      } else {
        float* dst = yk + (size_t)perm[row0 + m] * N + n;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) dst[r] = acc[wr][mt][r];
      }
    }
  }
}

// combine: grid (T, parts of a row).  shared: [parts, T, d] (TS), or null; sg: logits fp32, row stride ldz (null: no gate);
// wts null: the rows are added as they are (their weights went into the experts' inputs).
// TOPMAX / PMAX: upper bounds of `top` / `parts` (0: any number, in a loop): with bounds, all loads of an output
// are issued before anything is added (rows beyond the bounds are read from a clamped place and dropped).
template <typename TS, int TOPMAX, int PMAX>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ yk, const float* __restrict__ wts,
                                                          const TS* __restrict__ shared, int parts, size_t part_stride,
                                                          const float* __restrict__ sg, int ldz, float* __restrict__ y,
                                                          int top, int d) {
  const int t = blockIdx.x;
  float gate = 1.f;
  if (shared && sg) gate = 1.f / (1.f + expf(-sg[(size_t)t * ldz]));
  if (TOPMAX > 0) {
    float wk[TOPMAX > 0 ? TOPMAX : 1];
#pragma unroll
    for (int k = 0; k < TOPMAX; ++k) wk[k] = k < top ? (wts ? wts[(size_t)t * top + k] : 1.f) : 0.f;
    for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
      float a[TOPMAX > 0 ? TOPMAX : 1], sp[PMAX];
#pragma unroll
      for (int k = 0; k < TOPMAX; ++k) a[k] = yk[((size_t)t * top + min(k, top - 1)) * d + i];
#pragma unroll
      for (int p = 0; p < PMAX; ++p) sp[p] = shared ? to_float(shared[min(p, parts - 1) * part_stride + (size_t)t * d + i]) : 0.f;
      float v = 0.f;
#pragma unroll
      for (int k = 0; k < TOPMAX; ++k) v += wk[k] * a[k];
      float sh = 0.f;
#pragma unroll
      for (int p = 0; p < PMAX; ++p) sh += p < parts ? sp[p] : 0.f;
      y[(size_t)t * d + i] = shared ? v + gate * sh : v;
    }
    return;
  }
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
    float v = 0.f;
    for (int k = 0; k < top; ++k) v += (wts ? wts[(size_t)t * top + k] : 1.f) * yk[((size_t)t * top + k) * d + i];
    if (shared) {
      float sh = 0.f;
      for (int p = 0; p < parts; ++p) sh += to_float(shared[p * part_stride + (size_t)t * d + i]);
      v += gate * sh;
    }
    y[(size_t)t * d + i] = v;
  }
}

// the most tiles a step can have, at the smallest tile (16 rows): what the scratch arrays are sized for
extern "C" int sa_moe_max_tiles(int rows, int E) { return (rows + 15) / 16 + E; }

extern "C" int sa_moe_route(const float* logits, int ldz, int* ids, float* wts, int T, int E, int top,
                            int over_all, float wscale, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E <= 0 || top <= 0 || top > E || ldz < E) return SA_ERR_ARG;
  dim3 grid((T + 3) / 4), block(256);
  hipLaunchKernelGGL(moe_route_kernel, grid, block, 0, stream, logits, ldz, ids, wts, T, E, top, over_all, wscale);
  SA_LAUNCH_CHECK();
  return 0;
}

// ints: scratch of (E + 1) + E + n + 2 max_tiles + 1 int32 (offsets, cursor, perm, tile_expert, tile_row0, num_tiles)
// with max_tiles = sa_moe_max_tiles(n, E).  bf16 with d and F multiples of 8 takes the matrix cores: up to
// MOE_SMALL_ROWS rows (T top) in tiles of 16 with K cut over the waves, more in tiles of 64.
#define MOE_SMALL_ROWS 1024

// logits != nullptr (and T <= MOE_ROUTE_INSIDE): ids and wts are made here from the router's logits fp32 [T, ldz]
// (over_all: the mode of route_token, 0 to 2).  in_wts (fp32 [T top], may be wts itself): the weights multiply the experts' inputs
#define MOE_ROUTE_INSIDE 16

extern "C" int sa_moe_route_inside_limit() { return MOE_ROUTE_INSIDE; }

extern "C" int sa_moe_experts(const void* h, int act_dtype, int* ids, const void* Wg, const void* Wu,
                              const void* Wd, int* ints, void* act, float* yk, int T, int top, int E, int d, int F,
                              const float* logits, int ldz, float* wts, int over_all, float wscale, int gate_kind,
                              float gate_limit, const float* in_wts, hipStream_t stream) {
  if (T <= 0) return 0;
  const long long n = (long long)T * top;
  if (E <= 0 || top <= 0 || d <= 0 || F <= 0 || n > 0x3fffffffLL) return SA_ERR_ARG;
  if (gate_kind < 0 || gate_kind >= SA_GATE_KINDS) return SA_ERR_ARG;
  const int max_tiles = sa_moe_max_tiles((int)n, E);
  int* offsets = ints;
  int* cursor = offsets + E + 1;
  int* perm = cursor + E;
  int* tile_expert = perm + n;
  int* tile_row0 = tile_expert + max_tiles;
  int* num_tiles = tile_row0 + max_tiles;
  const bool mfma = act_dtype == SA_BF16 && (d & 7) == 0 && (F & 7) == 0;
  const bool small = n <= MOE_SMALL_ROWS;
  const int tile_rows = mfma ? (small ? 16 : 64) : MOE_TM;
  const int tiles = (int)((n + tile_rows - 1) / tile_rows) + E;
  if (logits && (T > MOE_ROUTE_INSIDE || !wts || ldz < E || top > E)) return SA_ERR_ARG;
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, stream, ids, (int)n, E, tile_rows, offsets, cursor, perm,
                     tile_expert, tile_row0, num_tiles, logits, ldz, ids, wts, top, over_all, wscale);
  SA_LAUNCH_CHECK();
  dim3 block(256);
  if (mfma) {
    // (tiles of 64 rows: a wave owns four groups of 16 weight rows per matrix, 256 a workgroup: 542 us against 604
    // with two groups and 874 with one, for 2,048 tokens, 32 experts of width 1,024, top 4, model width 2,048;
    // tiles of 128 rows were no faster)
    const int per = small ? 16 : 256;          // weight rows a workgroup owns
    dim3 g1(tiles, (F + per - 1) / per), g2(tiles, (d + per - 1) / per);
    if (g1.y > 65535 || g2.y > 65535) return SA_ERR_ARG;
#define GO(MT, KS, WR, KU)                                                                                                   \
  do {                                                                                                                 \
    hipLaunchKernelGGL((moe_mfma_kernel<MT, KS, true, WR, KU>), g1, block, 0, stream, (const bf16_t*)h, (const bf16_t*)Wg,     \
                       (const bf16_t*)Wu, offsets, perm, tile_expert, tile_row0, num_tiles, (bf16_t*)act, nullptr,     \
                       top, F, d, gate_kind, gate_limit, in_wts);                                                      \
    SA_LAUNCH_CHECK();                                                                                                 \
    hipLaunchKernelGGL((moe_mfma_kernel<MT, KS, false, WR, KU>), g2, block, 0, stream, (const bf16_t*)act, (const bf16_t*)Wd,  \
                       nullptr, offsets, perm, tile_expert, tile_row0, num_tiles, nullptr, yk, top, d, F, 0, 0.f,      \
                       nullptr);                                                                                       \
  } while (0)
    if (small) GO(1, 4, 1, 2);
    else GO(4, 1, 4, 2);
#undef GO
    SA_LAUNCH_CHECK();
    return 0;
  }
  dim3 g1(tiles, (F + MOE_TN - 1) / MOE_TN), g2(tiles, (d + MOE_TN - 1) / MOE_TN);
  if (g1.y > 65535 || g2.y > 65535) return SA_ERR_ARG;
  if (act_dtype == SA_F32) {
    hipLaunchKernelGGL(moe_gate_up_kernel<float>, g1, block, 0, stream, (const float*)h, (const float*)Wg,
                       (const float*)Wu, offsets, perm, tile_expert, tile_row0, num_tiles, (float*)act, top, d, F,
                       gate_kind, gate_limit, in_wts);
    SA_LAUNCH_CHECK();
    hipLaunchKernelGGL(moe_down_kernel<float>, g2, block, 0, stream, (const float*)act, (const float*)Wd, offsets, perm,
                       tile_expert, tile_row0, num_tiles, yk, d, F);
  } else if (act_dtype == SA_BF16) {
    hipLaunchKernelGGL(moe_gate_up_kernel<bf16_t>, g1, block, 0, stream, (const bf16_t*)h, (const bf16_t*)Wg,
                       (const bf16_t*)Wu, offsets, perm, tile_expert, tile_row0, num_tiles, (bf16_t*)act, top, d, F,
                       gate_kind, gate_limit, in_wts);
    SA_LAUNCH_CHECK();
    hipLaunchKernelGGL(moe_down_kernel<bf16_t>, g2, block, 0, stream, (const bf16_t*)act, (const bf16_t*)Wd, offsets,
                       perm, tile_expert, tile_row0, num_tiles, yk, d, F);
  } else {
    return SA_ERR_UNSUPPORTED;
  }
  SA_LAUNCH_CHECK();
  return 0;
}

// Only the grouping (and, with logits, the routing): the lists for products that another library runs over tiles of
// `tile_rows` grouped rows.  ints: as for sa_moe_experts, with max_tiles = sa_moe_max_tiles(T top, E).
extern "C" int sa_moe_group(int* ids, int* ints, int T, int top, int E, int tile_rows, const float* logits, int ldz,
                            float* wts, int over_all, float wscale, hipStream_t stream) {
  if (T <= 0) return 0;
  const long long n = (long long)T * top;
  if (E <= 0 || top <= 0 || tile_rows < 16 || n > 0x3fffffffLL) return SA_ERR_ARG;
  if (logits && (T > MOE_ROUTE_INSIDE || !wts || ldz < E || top > E)) return SA_ERR_ARG;
  const int max_tiles = sa_moe_max_tiles((int)n, E);
  int* offsets = ints;
  int* cursor = offsets + E + 1;
  int* perm = cursor + E;
  int* tile_expert = perm + n;
  int* tile_row0 = tile_expert + max_tiles;
  int* num_tiles = tile_row0 + max_tiles;
  hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 0, stream, ids, (int)n, E, tile_rows, offsets, cursor, perm,
                     tile_expert, tile_row0, num_tiles, logits, ldz, ids, wts, top, over_all, wscale);
  SA_LAUNCH_CHECK();
  return 0;
}

extern "C" int sa_moe_combine(const float* yk, const float* wts, const void* shared, int shared_dtype, int parts,
                              const float* sg, int ldz, float* y, int T, int top, int d, hipStream_t stream) {
  if (T <= 0) return 0;
  if (top <= 0 || d <= 0 || parts < 1) return SA_ERR_ARG;
  const size_t part_stride = (size_t)T * d;
  // a step of few rows: a value a thread, so that a row's loads are not a chain in one workgroup
  const int threads = d >= 256 ? 256 : 64;
  dim3 grid(T, T <= 64 ? (unsigned)((d + threads - 1) / threads) : 1u), block(threads);
#define GO(TS, TOPMAX, PMAX)                                                                                       \
  hipLaunchKernelGGL((moe_combine_kernel<TS, TOPMAX, PMAX>), grid, block, 0, stream, yk, wts, (const TS*)shared,     \
                     parts, part_stride, sg, ldz, y, top, d)
  const bool bounded = top <= 8 && parts <= 8;
  if (!shared || shared_dtype == SA_F32) {
    if (bounded) GO(float, 8, 8);
    else GO(float, 0, 1);
  } else if (shared_dtype == SA_BF16 && parts == 1) {
    if (bounded) GO(bf16_t, 8, 1);
    else GO(bf16_t, 0, 1);
  }
#undef GO
  else return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
