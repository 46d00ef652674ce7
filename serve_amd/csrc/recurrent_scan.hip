// Mixers whose memory is one fp32 matrix S [dk, dv] per head and request that decays and takes an outer product a token:
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t          a_t: a vector over dk, or one number a head
//
// A gated linear attention is this with a decay per key channel; a selective state-space mixer with S [state, head dim],
// k = B_t, q = C_t, v = dt_t x_t and the one decay exp(-exp(A_log) dt_t) a head.  What differs between such mixers lies
// in front of the recurrence (how q, k, v and the decays are made) and behind it (norm and gate of the read-out), so the
// file has the recurrence itself (`decay_scan`: token by token for single tokens and short portions, sixteen tokens a
// pass on the matrix cores for prompts), the two preparations (`gla_decay`; `ssm_prepare` with the causal convolution,
// and `conv_state_update` for the convolution's last inputs) and one kernel for what follows (`gated_group_norm`).
// The decays travel as their logarithms (<= 0), which is how both preparations get them and what a pass over several
// tokens sums.  All arithmetic is fp32, also on the matrix cores (v_mfma_f32_16x16x4_f32); template types are the
// storage of projections and outputs.
#include "common.h"

#define RS_MAX_TAPS 16

// e^x in a few instructions (a result below the normal range may come out as 0, one above it as infinity): 2^t with t = x log2(e) rounded, corrected by what the rounding of t lost, r = x log2(e) - t, as
// 2^t (1 + r ln 2).  A few instructions, and within two units in the last place.
__device__ __forceinline__ float rs_exp(float x) {
  const float L2E = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-8f;
  const float t = x * L2E;
  float r = fmaf(x, L2E, -t);
  r = fmaf(x, L2E_LO, r);
  const float e = __builtin_amdgcn_exp2f(t);
  return fmaf(e, r * 0.693147182464599609375f, e);
}

// z sigmoid(z) with that exponential and the hardware's reciprocal: within a few units in the last place
// (the exponent is kept below the overflow: beyond 80 the result is z e^z, which is nothing, either way)
__device__ __forceinline__ float rs_silu(float z) { return z * __builtin_amdgcn_rcpf(1.f + rs_exp(fminf(-z, 80.f))); }
__device__ __forceinline__ float rs_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
// ln(sigmoid(z)) without overflow on either side
__device__ __forceinline__ float rs_logsigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <int CTRL>
__device__ __forceinline__ float rs_dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// the sum over a row of 16 neighbouring lanes, in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
  v += rs_dpp<0xB1>(v);           // quad_perm [1, 0, 3, 2]
  v += rs_dpp<0x4E>(v);           // quad_perm [2, 3, 0, 1]
  v += rs_dpp<0x141>(v);          // row_half_mirror
  v += rs_dpp<0x140>(v);          // row_mirror
  return v;
}

// ---------------------------------------------------------------------------------------------
// The recurrence.  grid (column tiles, H, B), 256 threads = 16 groups of columns x 16 parts of the rows: thread
// (cl, r) keeps rows r RPT .. r RPT + RPT - 1 of columns (tile 16 + cl) CPT .. + CPT - 1 in registers for the whole
// segment; a token is RPT CPT decays and outer-product terms, the same number of read-out terms, and one sum over the
// 16 lanes of a row for each of the CPT columns.  The tokens of a segment come through LDS in chunks.  A token's
// arithmetic does not depend on where the segment was cut, so prompts, portions and single tokens give the same bits.
//
// The state of a request lives in the layout of these registers: [H][tile][RPT][256 threads][CPT] floats, so that a
// segment's first and last act are whole-wave contiguous loads and stores (rows beyond dk and columns beyond dv are
// padding that stays zero).
// ---------------------------------------------------------------------------------------------
template <typename TQ, int RPT, int CPT, int CH>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    const TQ* __restrict__ q, const TQ* __restrict__ k, const TQ* __restrict__ v, long long q_stride,
    long long k_stride, long long v_stride, const float* __restrict__ log_decay, int per_channel, float q_scale,
    float* __restrict__ state, long long state_stride, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, float* __restrict__ o, int H, int Hk, int dk, int dv) {
  constexpr int ROWS = 16 * RPT;
  constexpr int PAD = RPT == 1 ? 1 : RPT + 1;      // an odd stride between the parts of a row: different banks
  constexpr int ROW = 16 * PAD;
  __shared__ float sq[CH][ROW];
  __shared__ float sk[CH][ROW];
  __shared__ float sa[CH][ROW];
  __shared__ float sv[CH][16 * CPT];
  const int cl = threadIdx.x >> 4, r = threadIdx.x & 15;
  const int tile = blockIdx.x, h = blockIdx.y, seg = blockIdx.z;
  const int hk = h / (H / Hk);
  const int j0 = (tile * 16 + cl) * CPT;
  const int slot = state_slots[seg];
  const int t0 = cu_q[seg], n = cu_q[seg + 1] - t0;
  float* st = slot >= 0 ? state + (size_t)slot * state_stride +
                              ((size_t)h * gridDim.x + tile) * (size_t)(RPT * 256 * CPT) + (size_t)threadIdx.x * CPT
                        : nullptr;
  float S[RPT][CPT];
#pragma unroll
  for (int ii = 0; ii < RPT; ++ii)
#pragma unroll
    for (int cc = 0; cc < CPT; ++cc) S[ii][cc] = st ? st[(size_t)ii * 256 * CPT + cc] : 0.f;
  for (int c0 = 0; c0 < n; c0 += CH) {
    const int m = min(CH, n - c0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < m * ROWS; idx += 256) {
      const int tt = idx / ROWS, i = idx - tt * ROWS;
      const int pos = (i / RPT) * PAD + (i % RPT);
      const bool in = i < dk;
      const size_t tok = (size_t)(t0 + c0 + tt);
      const int ic = in ? i : 0;
      const float qv = to_float(q[tok * q_stride + (size_t)hk * dk + ic]) * q_scale;
      const float kv = to_float(k[tok * k_stride + (size_t)hk * dk + ic]);
      const float av = expf(per_channel ? log_decay[(tok * H + h) * (size_t)dk + ic] : log_decay[tok * H + h]);
      sq[tt][pos] = in ? qv : 0.f;
      sk[tt][pos] = in ? kv : 0.f;
      sa[tt][pos] = in ? av : 1.f;
    }
    for (int idx = threadIdx.x; idx < m * 16 * CPT; idx += 256) {
      const int tt = idx / (16 * CPT), c = idx - tt * (16 * CPT);
      const int jj = tile * 16 * CPT + c;
      sv[tt][c] = jj < dv ? to_float(v[(size_t)(t0 + c0 + tt) * v_stride + (size_t)h * dv + jj]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < m; ++tt) {
      float vv[CPT], acc[CPT];
#pragma unroll
      for (int cc = 0; cc < CPT; ++cc) {
        vv[cc] = sv[tt][cl * CPT + cc];
        acc[cc] = 0.f;
      }
#pragma unroll
      for (int ii = 0; ii < RPT; ++ii) {
        const float a = sa[tt][r * PAD + ii], kk = sk[tt][r * PAD + ii], qq = sq[tt][r * PAD + ii];
#pragma unroll
        for (int cc = 0; cc < CPT; ++cc) {
          S[ii][cc] = fmaf(a, S[ii][cc], kk * vv[cc]);
          acc[cc] = fmaf(S[ii][cc], qq, acc[cc]);
        }
      }
#pragma unroll
      for (int cc = 0; cc < CPT; ++cc) acc[cc] = row16_sum(acc[cc]);
      if (r == 0) {
        float* dst = o + ((size_t)(t0 + c0 + tt) * H + h) * dv;
#pragma unroll
        for (int cc = 0; cc < CPT; ++cc)
          if (j0 + cc < dv) dst[j0 + cc] = acc[cc];
      }
    }
  }
  if (st) {
#pragma unroll
    for (int ii = 0; ii < RPT; ++ii)
#pragma unroll
      for (int cc = 0; cc < CPT; ++cc) st[(size_t)ii * 256 * CPT + cc] = S[ii][cc];
  }
}

static int scan_rpt(int dk) {
  int rpt = 1;
  while (16 * rpt < dk) rpt *= 2;
  return rpt;
}
static int scan_cpt(int dv) { return dv >= 64 ? 4 : (dv >= 32 ? 2 : 1); }

// floats of a request's state that the recurrence of H heads of [dk, dv] keeps (its own padded layout)
extern "C" long long sa_decay_scan_state_floats(int H, int dk, int dv) {
  if (H <= 0 || dk <= 0 || dv <= 0 || dk > 256) return -1;
  const int rpt = scan_rpt(dk), cpt = scan_cpt(dv);
  const int tiles = (dv + 16 * cpt - 1) / (16 * cpt);
  return (long long)H * tiles * rpt * 256 * cpt;
}

template <typename TQ, int RPT, int CPT>
static void launch_scan(const void* q, const void* k, const void* v, long long qs, long long ks, long long vs,
                        const float* decay, int per_channel, float q_scale, float* state, long long state_stride,
                        const int* cu_q, const int* slots, float* o, int B, int H, int Hk, int dk, int dv,
                        hipStream_t stream) {
  constexpr int CH = RPT >= 16 ? 8 : 16;
  const int tiles = (dv + 16 * CPT - 1) / (16 * CPT);
  dim3 grid(tiles, H, B), block(256);
  hipLaunchKernelGGL((decay_scan_kernel<TQ, RPT, CPT, CH>), grid, block, 0, stream, (const TQ*)q, (const TQ*)k,
                     (const TQ*)v, qs, ks, vs, decay, per_channel, q_scale, state, state_stride, cu_q, slots, o, H, Hk,
                     dk, dv);
}

template <typename TQ, int RPT>
static void launch_scan_c(int cpt, const void* q, const void* k, const void* v, long long qs, long long ks,
                          long long vs, const float* decay, int per_channel, float q_scale, float* state,
                          long long state_stride, const int* cu_q, const int* slots, float* o, int B, int H, int Hk,
                          int dk, int dv, hipStream_t stream) {
#define GO(C) launch_scan<TQ, RPT, C>(q, k, v, qs, ks, vs, decay, per_channel, q_scale, state, state_stride, cu_q, slots, o, B, H, Hk, dk, dv, stream)
  if (cpt == 4) GO(4);
  else if (cpt == 2) GO(2);
  else GO(1);
#undef GO
}

template <typename TQ>
static void launch_scan_r(int rpt, int cpt, const void* q, const void* k, const void* v, long long qs, long long ks,
                          long long vs, const float* decay, int per_channel, float q_scale, float* state,
                          long long state_stride, const int* cu_q, const int* slots, float* o, int B, int H, int Hk,
                          int dk, int dv, hipStream_t stream) {
#define GO(R) launch_scan_c<TQ, R>(cpt, q, k, v, qs, ks, vs, decay, per_channel, q_scale, state, state_stride, cu_q, slots, o, B, H, Hk, dk, dv, stream)
  switch (rpt) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 4: GO(4); break;
    case 8: GO(8); break;
    default: GO(16); break;
  }
#undef GO
}

// ---------------------------------------------------------------------------------------------
// The recurrence for prompts: sixteen tokens a pass.  With b_t the sum of the logarithms of the decays of tokens
// 0..t of the pass (a vector over the key channels, <= 0 and falling) and S0 the state before it:
//
//   o_t = S0^T (q_t e^(b_t))  +  sum_(s<=t) A[t, s] v_s          A[t, s] = sum_c q_t[c] k_s[c] e^(b_t[c] - b_s[c])
//   S   = diag(e^(b_15)) S0   +  sum_s (k_s e^(b_15 - b_s)) v_s^T
//
// Both lines are matrix products of fp32 operands (v_mfma_f32_16x16x4_f32, fp32 in and out), and every factor
// e^(..) in them is at most 1.  A too is a product, (q_t e^(b_t - b_7)) . (k_s e^(b_7 - b_s)), as long as no channel
// decays by more than e^-80 within either half of the pass, so that neither factor leaves the range of fp32; a pass
// where one does sums the channels of each of its 136 entries one by one, with the exponent of the difference
// itself.  A pass that the segment's end cuts short is filled with tokens that change nothing (q = k = v = 0,
// decay 1).
//
// grid (ceil(dv / 64), H, B x pieces), 256 threads: wave w owns 16 columns and keeps their S in the registers of the matrix
// cores' result layout (lane (g, j): rows 16 m + 4 g + r, column j), which serves as the second operand of
// S0^T q directly when the contraction runs over the rows in that same order.  All waves share the scaled q and k
// of the pass in LDS; the next pass's inputs are loaded into registers while this one's products run.  A request's
// state is read and written in the token-by-token kernel's layout (RPT, CPT: its row and column split), since a
// request changes between the two with every step.
// ---------------------------------------------------------------------------------------------
typedef float rs_f4 __attribute__((ext_vector_type(4)));
#define RS_RANGE 80.f
// what a launch of the kernel does: whole segments from the requests' states; or, where long segments are cut into
// pieces that run side by side, first every piece from zeros for the state that its tokens add, then (after the chain
// through the pieces) every piece from the state it truly starts from
enum { RS_WHOLE = 0, RS_PIECE_STATES = 1, RS_PIECE_OUTPUTS = 2 };

template <typename TQ, int NT>
__global__ __launch_bounds__(256) void decay_scan_block_kernel(
    const TQ* __restrict__ q, const TQ* __restrict__ k, const TQ* __restrict__ v, long long q_stride,
    long long k_stride, long long v_stride, const float* __restrict__ log_decay, int per_channel, float q_scale,
    float* __restrict__ state, long long state_stride, const int* __restrict__ cu_q,
    const int* __restrict__ state_slots, float* __restrict__ o, int H, int Hk, int dk, int dv, int RPT, int CPT,
    int mode, int piece, int pieces, float* __restrict__ scratch, long long scratch_stride, long long scratch_decays) {
  constexpr int DKP = 16 * NT;                   // the key channels, padded
  constexpr int ST = DKP + 4;                    // row stride in LDS: 4 (or 20) mod 32 banks, and rows stay 16-byte aligned
  constexpr int NE = NT;                         // q / k elements of a pass per thread: 16 DKP / 256
  __shared__ __attribute__((aligned(16))) float sb[16][ST];     // b_t
  __shared__ __attribute__((aligned(16))) float sqh[16][ST];    // q e^(b_t)
  __shared__ __attribute__((aligned(16))) float skt[16][ST];    // k e^(b_15 - b_t)
  __shared__ __attribute__((aligned(16))) float sqp[16][ST];    // q e^(b_t - b_7), or q itself
  __shared__ __attribute__((aligned(16))) float skp[16][ST];    // k e^(b_7 - b_t), or k itself
  __shared__ __attribute__((aligned(16))) float sdec[DKP];      // e^(b_15)
  __shared__ float sv[16][68];
  __shared__ float sap[4][16][17];
  __shared__ float sam[16][20];
  const int tid = threadIdx.x, w = tid >> 6, lane = tid & 63, g = lane >> 4, j = lane & 15;
  const int tile = blockIdx.x, h = blockIdx.y, seg = blockIdx.z / pieces, pj = blockIdx.z - seg * pieces;
  const int hk = h / (H / Hk);
  const int slot = state_slots[seg];
  const int whole = cu_q[seg + 1] - cu_q[seg];   // the segment; this workgroup's piece of it: n tokens from t0
  const int t0 = cu_q[seg] + pj * piece, n = min(piece, cu_q[seg + 1] - t0);
  if (n <= 0) return;
  const bool split = whole > piece;              // the segment has several pieces: their states go through `scratch`
  if (mode == RS_PIECE_STATES && !split) return;
  const int col = tile * 64 + w * 16 + j;        // this lane's column of S and o
  const int seq_tiles = (dv + 16 * CPT - 1) / (16 * CPT);
  // where the token-by-token kernel keeps (row, col) of head h
  auto state_at = [&](int row) -> size_t {
    return (((size_t)h * seq_tiles + col / (16 * CPT)) * RPT + row % RPT) * (size_t)(256 * CPT) +
           (size_t)(((col / CPT) % 16) * 16 + row / RPT) * CPT + col % CPT;
  };
  // this piece's row of the scratch: the segments that are cut have `pieces` rows each, in their order
  int cut_before = 0;
  if (split)
    for (int s2 = 0; s2 < seg; ++s2) cut_before += (cu_q[s2 + 1] - cu_q[s2] > piece) ? 1 : 0;
  float* const mine = scratch + (size_t)(cut_before * pieces + pj) * scratch_stride;
  float* st = col >= dv ? nullptr : (split ? mine : (slot >= 0 ? state + (size_t)slot * state_stride : nullptr));
  rs_f4 S[NT];
#pragma unroll
  for (int m = 0; m < NT; ++m)
#pragma unroll
    for (int r = 0; r < 4; ++r) S[m][r] = (st && mode != RS_PIECE_STATES) ? st[state_at(16 * m + 4 * g + r)] : 0.f;
  float btotal = 0.f;                            // (threads below DKP) the piece's sum of a channel's log decays

  // the inputs of a pass, in registers as they were loaded (nothing is computed on them before their pass, so the
  // loads of the next pass stay in flight under this one's products): log decays (threads below DKP: one channel
  // each), q, k, v.  Places outside the segment or the head load a neighbour's value and are masked at use.
  float rla[16];
  TQ rq[NE], rk[NE], rv[4];
  // where a thread's loads lie from the first token of a pass on: 32-bit offsets that change only for a last,
  // shorter pass (beside a base that is the same for the whole workgroup, a load is then one instruction)
  unsigned lo[16], qo[NE], ko[NE], vo[4];
  auto place = [&](int last) {
    const unsigned c = (unsigned)min(tid, dk - 1);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      const unsigned tt = (unsigned)min(t, last);
      lo[t] = per_channel ? (tt * H) * (unsigned)dk + c : tt * H;
    }
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int idx = tid + 256 * e;
      const unsigned tt = (unsigned)min(idx / DKP, last), cc = (unsigned)min(idx % DKP, dk - 1);
      qo[e] = tt * (unsigned)q_stride + cc;
      ko[e] = tt * (unsigned)k_stride + cc;
    }
    const unsigned vcol = (unsigned)min(tile * 64 + (tid & 63), dv - 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) vo[e] = (unsigned)min((tid + 256 * e) >> 6, last) * (unsigned)v_stride + vcol;
  };
  auto fetch = [&](int c0) {
    const size_t tok = (size_t)(t0 + c0);
    const float* lb = log_decay + (per_channel ? (tok * H + h) * (size_t)dk : tok * H + h);
    const TQ* qb = q + tok * q_stride + (size_t)hk * dk;
    const TQ* kb = k + tok * k_stride + (size_t)hk * dk;
    const TQ* vb = v + tok * v_stride + (size_t)h * dv;
    if (tid < DKP) {
#pragma unroll
      for (int t = 0; t < 16; ++t) rla[t] = lb[lo[t]];
    }
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      rq[e] = qb[qo[e]];
      rk[e] = kb[ko[e]];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) rv[e] = vb[vo[e]];
  };
  place(min(16, n) - 1);
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += 16) {
    const int m = min(16, n - c0);
    __syncthreads();                             // the pass before has read its LDS
    int far = 0;
    if (tid < DKP) {
      float run = 0.f, b7 = 0.f;
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        run += (t < m && tid < dk) ? rla[t] : 0.f;
        sb[t][tid] = run;
        if (t == 7) b7 = run;
      }
      sdec[tid] = rs_exp(run);
      btotal += run;
      far = (b7 < -RS_RANGE) || (run - b7 < -RS_RANGE);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int idx = tid + 256 * e;
      sv[idx >> 6][idx & 63] = ((idx >> 6) < m && tile * 64 + (idx & 63) < dv) ? to_float(rv[e]) : 0.f;
    }
    const int wide = __syncthreads_or(far);
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int idx = tid + 256 * e, t = idx / DKP, c = idx % DKP;
      const bool in = t < m && c < dk;
      const float qv = in ? to_float(rq[e]) * q_scale : 0.f, kv = in ? to_float(rk[e]) : 0.f;
      const float bt = sb[t][c], b7 = sb[7][c], b15 = sb[15][c];
      skt[t][c] = kv * rs_exp(b15 - bt);
      if (mode != RS_PIECE_STATES) {
        sqh[t][c] = qv * rs_exp(bt);
        sqp[t][c] = wide ? qv : qv * rs_exp(bt - b7);
        skp[t][c] = wide ? kv : kv * rs_exp(b7 - bt);
      }
    }
    if (c0 + 16 < n) {                           // in flight while the products run
      if (n - (c0 + 16) < 16) place(n - (c0 + 16) - 1);
      fetch(c0 + 16);
    }
    __syncthreads();
    // A, the weights of the pass's own tokens
    if (mode == RS_PIECE_STATES) {
    } else if (!wide) {
      rs_f4 acc = {0.f, 0.f, 0.f, 0.f};
      const int cb = w * 4 * NT;                 // each wave a quarter of the channels
#pragma unroll
      for (int s4 = 0; s4 < NT; ++s4)
        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(sqp[j][cb + 4 * s4 + g], skp[j][cb + 4 * s4 + g], acc, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) sap[w][4 * g + r][j] = acc[r];
      __syncthreads();
      const int t = tid >> 4, s = tid & 15;
      sam[t][s] = s <= t ? (sap[0][t][s] + sap[1][t][s]) + (sap[2][t][s] + sap[3][t][s]) : 0.f;
    } else {
      const int t = tid >> 4, s = tid & 15;
      float a = 0.f;
      if (s <= t)
        for (int c = 0; c < DKP; ++c) a = fmaf(sqp[t][c] * skp[s][c], rs_exp(sb[t][c] - sb[s][c]), a);
      sam[t][s] = a;
    }
    __syncthreads();
    // this wave's 16 columns: the read-out ...
    float vb[4];
#pragma unroll
    for (int s4 = 0; s4 < 4; ++s4) vb[s4] = sv[4 * s4 + g][w * 16 + j];
    if (mode != RS_PIECE_STATES) {
      rs_f4 oc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int mt = 0; mt < NT; ++mt) {
        const rs_f4 a4 = *reinterpret_cast<const rs_f4*>(&sqh[j][16 * mt + 4 * g]);
#pragma unroll
        for (int r = 0; r < 4; ++r) oc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], S[mt][r], oc, 0, 0, 0);
      }
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) oc = __builtin_amdgcn_mfma_f32_16x16x4f32(sam[j][4 * s4 + g], vb[s4], oc, 0, 0, 0);
      if (col < dv) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (4 * g + r < m) o[((size_t)(t0 + c0 + 4 * g + r) * H + h) * dv + col] = oc[r];
      }
    }
    // ... and the state after the pass
#pragma unroll
    for (int mt = 0; mt < NT; ++mt) {
      const rs_f4 d4 = *reinterpret_cast<const rs_f4*>(&sdec[16 * mt + 4 * g]);
      rs_f4 sm = S[mt];
#pragma unroll
      for (int r = 0; r < 4; ++r) sm[r] *= d4[r];
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) sm = __builtin_amdgcn_mfma_f32_16x16x4f32(skt[4 * s4 + g][16 * mt + j], vb[s4], sm, 0, 0, 0);
      S[mt] = sm;
    }
  }
  // a whole segment leaves its state with the request; a piece leaves what its own tokens add to a state (and by how
  // much they shrink one) in its row of the scratch, and nothing after the pass that starts from the true state
  if (st && (mode == RS_PIECE_STATES || !split)) {
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) st[state_at(16 * m + 4 * g + r)] = S[m][r];
  }
  if (mode == RS_PIECE_STATES && tile == 0 && tid < DKP) mine[scratch_decays + (size_t)h * DKP + tid] = rs_exp(btotal);
}

// ---------------------------------------------------------------------------------------------
// Between the two passes over the pieces of long segments: from the request's state (or zeros) S, piece after piece,
// the piece's row takes S, the state it starts from, and S <- D S + (what the piece's tokens add), D the piece's
// decay of the row's key channel; the state after the last piece goes to the request.  A thread per float of a
// state row (the token-by-token kernel's layout: index -> row as there); grid (ceil(floats / 256), B).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void decay_scan_chain_kernel(float* __restrict__ state, long long state_stride,
                                                               const int* __restrict__ cu_q,
                                                               const int* __restrict__ state_slots,
                                                               float* __restrict__ scratch, long long scratch_stride,
                                                               long long scratch_decays, int floats, int piece,
                                                               int pieces, int RPT, int CPT, int DKP, int tiles) {
  const int seg = blockIdx.y;
  const int whole = cu_q[seg + 1] - cu_q[seg];
  const int at = blockIdx.x * 256 + threadIdx.x;
  if (whole <= piece || at >= floats) return;
  const int count = (whole + piece - 1) / piece;
  int cut_before = 0;
  for (int s2 = 0; s2 < seg; ++s2) cut_before += (cu_q[s2 + 1] - cu_q[s2] > piece) ? 1 : 0;
  // at = ((h tiles + tile) RPT + ii) 256 CPT + thread CPT + cc, thread = 16 (column group) + r: row r RPT + ii
  const int per = 256 * CPT;
  const int hi = at / per, thread = (at - hi * per) / CPT;
  const int h = hi / (tiles * RPT), row = (thread & 15) * RPT + hi % RPT;
  const int slot = state_slots[seg];
  float S = slot >= 0 ? state[(size_t)slot * state_stride + at] : 0.f;
  for (int pj = 0; pj < count; ++pj) {
    float* mine = scratch + (size_t)(cut_before * pieces + pj) * scratch_stride;
    const float add = mine[at], D = mine[scratch_decays + (size_t)h * DKP + row];
    mine[at] = S;
    S = fmaf(D, S, add);
  }
  if (slot >= 0) state[(size_t)slot * state_stride + at] = S;
}

template <typename TQ>
static int launch_scan_block(int rpt, int cpt, const void* q, const void* k, const void* v, long long qs, long long ks,
                             long long vs, const float* decay, int per_channel, float q_scale, float* state,
                             long long state_stride, const int* cu_q, const int* slots, float* o, int B, int H, int Hk,
                             int dk, int dv, int mode, int piece, int pieces, float* scratch, long long scratch_stride,
                             long long scratch_decays, hipStream_t stream) {
  dim3 grid((dv + 63) / 64, H, B * pieces), block(256);
#define GO(N) hipLaunchKernelGGL((decay_scan_block_kernel<TQ, N>), grid, block, 0, stream, (const TQ*)q, (const TQ*)k, (const TQ*)v, qs, ks, vs, decay, per_channel, q_scale, state, state_stride, cu_q, slots, o, H, Hk, dk, dv, rpt, cpt, mode, piece, pieces, scratch, scratch_stride, scratch_decays)
  switch (rpt) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 4: GO(4); break;
    case 8: GO(8); break;
    default: return SA_ERR_UNSUPPORTED;
  }
#undef GO
  return 0;
}

// the longest segment from which a launch takes sixteen tokens a pass, and the widest key it does so for
#define RS_BLOCK_MIN_TOKENS 6
#define RS_BLOCK_MAX_DK 128
extern "C" int sa_decay_scan_block_min_tokens() { return RS_BLOCK_MIN_TOKENS; }

// q, k: rows of `q_stride` / `k_stride` elements with head hk's dk values at hk dk (Hk heads; head h reads hk = h / (H / Hk));
// v: rows of `v_stride` with head h's dv values at h dv; decay: the decays' logarithms, fp32 [T, H, dk] (per_channel) or [T, H];
// o fp32 [T, H, dv]; max_q: the longest segment (what decides between the two kernels);
// state: a request's row at state + slot state_stride (the floats that sa_decay_scan_state_floats counts), slot < 0: a
// segment without a request, which starts from zeros and keeps nothing.
extern "C" int sa_decay_scan(const void* q, const void* k, const void* v, int dtype, long long q_stride,
                             long long k_stride, long long v_stride, const float* decay, int per_channel,
                             float q_scale, float* state, long long state_stride, const int* cu_q,
                             const int* state_slots, float* o, int B, int H, int Hk, int dk, int dv, int max_q,
                             int piece, float* scratch, long long scratch_stride, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H <= 0 || Hk <= 0 || H % Hk || dk <= 0 || dk > 256 || dv <= 0 || !q || !k || !v || !decay || !state || !o ||
      !cu_q || !state_slots || B > 65535 || H > 65535)
    return SA_ERR_ARG;
  const int rpt = scan_rpt(dk), cpt = scan_cpt(dv);
  const long long far_stride = 1LL << 27;         // the passes over sixteen tokens keep 32-bit offsets within a pass
  if (max_q >= RS_BLOCK_MIN_TOKENS && dk <= RS_BLOCK_MAX_DK && (dtype == SA_F32 || dtype == SA_BF16) &&
      q_stride < far_stride && k_stride < far_stride && v_stride < far_stride && (long long)H * dk < far_stride) {
    // piece > 0: segments longer than `piece` tokens (a multiple of 16) run as pieces side by side; scratch: fp32 rows
    // of scratch_stride >= state floats + H 16 rpt floats, ceil(max_q / piece) for every segment that is cut, zeroed
    const long long floats = sa_decay_scan_state_floats(H, dk, dv);
    int pieces = 1;
    if (piece > 0 && max_q > piece) {
      if (piece % 16 || !scratch || scratch_stride < floats + (long long)H * 16 * rpt) return SA_ERR_ARG;
      pieces = (max_q + piece - 1) / piece;
    } else {
      piece = 0x7fffff00;
    }
    if ((long long)B * pieces > 65535) return SA_ERR_ARG;
    const int modes[2] = {pieces > 1 ? RS_PIECE_STATES : RS_WHOLE, RS_PIECE_OUTPUTS};
    for (int pass = 0; pass < (pieces > 1 ? 2 : 1); ++pass) {
      const int rc = dtype == SA_F32
          ? launch_scan_block<float>(rpt, cpt, q, k, v, q_stride, k_stride, v_stride, decay, per_channel, q_scale, state,
                                     state_stride, cu_q, state_slots, o, B, H, Hk, dk, dv, modes[pass], piece, pieces,
                                     scratch, scratch_stride, floats, stream)
          : launch_scan_block<bf16_t>(rpt, cpt, q, k, v, q_stride, k_stride, v_stride, decay, per_channel, q_scale, state,
                                      state_stride, cu_q, state_slots, o, B, H, Hk, dk, dv, modes[pass], piece, pieces,
                                      scratch, scratch_stride, floats, stream);
      if (rc) return rc;
      SA_LAUNCH_CHECK();
      if (pieces > 1 && pass == 0) {
        const int tiles = (dv + 16 * cpt - 1) / (16 * cpt);
        hipLaunchKernelGGL(decay_scan_chain_kernel, dim3((unsigned)((floats + 255) / 256), B), dim3(256), 0, stream, state,
                           state_stride, cu_q, state_slots, scratch, scratch_stride, floats, (int)floats, piece, pieces,
                           rpt, cpt, 16 * rpt, tiles);
        SA_LAUNCH_CHECK();
      }
    }
    return 0;
  }
  if (dtype == SA_F32)
    launch_scan_r<float>(rpt, cpt, q, k, v, q_stride, k_stride, v_stride, decay, per_channel, q_scale, state,
                         state_stride, cu_q, state_slots, o, B, H, Hk, dk, dv, stream);
  else if (dtype == SA_BF16)
    launch_scan_r<bf16_t>(rpt, cpt, q, k, v, q_stride, k_stride, v_stride, decay, per_channel, q_scale, state,
                          state_stride, cu_q, state_slots, o, B, H, Hk, dk, dv, stream);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The logarithm of the decay sigmoid(z[t, c] + b[c])^(1 / tau):  ln sigmoid(z + b) / tau, c over H dk channels
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gla_decay_kernel(const float* __restrict__ z, const float* __restrict__ bias,
                                                        float inv_tau, float* __restrict__ decay, long long total,
                                                        int C) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % C);
  decay[idx] = rs_logsigmoid(z[idx] + (bias ? bias[c] : 0.f)) * inv_tau;
}

extern "C" int sa_gla_decay(const float* z, const float* bias, float tau, float* decay, int T, int C,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (!z || !decay || C <= 0 || !(tau > 0.f)) return SA_ERR_ARG;
  const long long total = (long long)T * C;
  const long long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return SA_ERR_ARG;
  hipLaunchKernelGGL(gla_decay_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, z, bias, 1.f / tau, decay, total, C);
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The state-space mixer's preparation.  zx [T, zs]: the projection's rows; columns col0 .. col0 + C - 1 are the
// convolution's channels [x: H P | B: G N | C: G N].  Per token and channel: the causal convolution over `taps` inputs
// (w [C, taps], the last column on the current token, bias b; inputs before the segment come from the request's state
// row at conv_off, [taps - 1, C] oldest first, or are zeros where the segment has no request) and silu -> xbc fp32 [T, C].
// Per token and head: dt = softplus(dtraw + dt_bias), the decay's logarithm -exp(A_log) dt -> decay [T, H]; v = dt x -> fp32 [T, H P].
// grid (T, or ceil(T / 8) from 257 tokens on; ceil((C + H) / 256)).
// ---------------------------------------------------------------------------------------------
#define RS_PREP_TOKENS 8
template <typename TA>
__global__ __launch_bounds__(256) void ssm_prepare_kernel(
    const TA* __restrict__ zx, long long zs, int col0, const float* __restrict__ conv_w,
    const float* __restrict__ conv_b, const float* __restrict__ state, long long state_stride, long long conv_off,
    const float* __restrict__ dtraw, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const int* __restrict__ seg_of_token, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
    float* __restrict__ xbc, float* __restrict__ vout, float* __restrict__ decay, int T, int H, int P, int C, int taps, int per) {
  // `per` tokens a workgroup (in a prompt a token's work for a channel is too little to pay for a workgroup's start);
  // the step sizes of the heads that the workgroup's channels belong to are made once a head and token
  __shared__ float sdt[RS_PREP_TOKENS][260];
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int c_first = blockIdx.y * 256;
  const int t_end = min(T, ((int)blockIdx.x + 1) * per);
  const int h_first = c_first / P;
  if (c_first < H * P) {
    const int nh = min(c_first + 255, H * P - 1) / P - h_first + 1;
    for (int i = threadIdx.x; i < nh * per; i += 256) {
      const int tt = i / nh, hh = i - tt * nh, t = blockIdx.x * per + tt;
      if (t < t_end) sdt[tt][hh] = rs_softplus(dtraw[(size_t)t * H + h_first + hh] + dt_bias[h_first + hh]);
    }
    __syncthreads();
  }
  if (c >= C + H) return;
  // A run of tokens inside one segment, none of them among its first taps - 1: every input comes from the step's own
  // rows.  The channel's inputs of the run and its taps are loaded once, all at a go, and each token is a window of them.
  const int t_first = blockIdx.x * per;
  if (per == RS_PREP_TOKENS && t_end - t_first == RS_PREP_TOKENS && c < C) {
    const int seg = seg_of_token[t_first];
    if (seg_of_token[t_end - 1] == seg && t_first - (taps - 1) >= cu_q[seg]) {
      float xin[RS_PREP_TOKENS + RS_MAX_TAPS - 1], w[RS_MAX_TAPS];
      const TA* src = zx + (size_t)(t_first - (taps - 1)) * zs + col0 + c;
#pragma unroll
      for (int i = 0; i < RS_PREP_TOKENS + RS_MAX_TAPS - 1; ++i)
        if (i < RS_PREP_TOKENS + taps - 1) xin[i] = to_float(src[(size_t)i * zs]);
#pragma unroll
      for (int j = 0; j < RS_MAX_TAPS; ++j)
        if (j < taps) w[j] = conv_w[(size_t)c * taps + j];
      const float bias = conv_b ? conv_b[c] : 0.f;
#pragma unroll
      for (int tt = 0; tt < RS_PREP_TOKENS; ++tt) {
        float acc = bias;
#pragma unroll
        for (int j = 0; j < RS_MAX_TAPS; ++j)
          if (j < taps) acc = fmaf(w[j], xin[tt + j], acc);
        const float y = rs_silu(acc);
        const int t = t_first + tt;
        xbc[(size_t)t * C + c] = y;
        if (c < H * P) vout[(size_t)t * H * P + c] = sdt[tt][c / P - h_first] * y;
      }
      return;
    }
  }
  for (int t = t_first; t < t_end; ++t) {
    if (c >= C) {
      const int h = c - C;
      const float dt = rs_softplus(dtraw[(size_t)t * H + h] + dt_bias[h]);
      decay[(size_t)t * H + h] = -expf(A_log[h]) * dt;
      continue;
    }
    const int seg = seg_of_token[t];
    const int t0 = cu_q[seg];
    const int slot = state_slots[seg];
    const float* cs = slot >= 0 ? state + (size_t)slot * state_stride + conv_off : nullptr;
    float acc = conv_b ? conv_b[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int tp = t - (taps - 1 - j);
      float xv;
      if (tp >= t0) xv = to_float(zx[(size_t)tp * zs + col0 + c]);
      else xv = cs ? cs[(size_t)(taps - 1 + tp - t0) * C + c] : 0.f;
      acc = fmaf(conv_w[(size_t)c * taps + j], xv, acc);
    }
    const float y = rs_silu(acc);
    xbc[(size_t)t * C + c] = y;
    if (c < H * P) vout[(size_t)t * H * P + c] = sdt[t - blockIdx.x * per][c / P - h_first] * y;
  }
}

extern "C" int sa_ssm_prepare(const void* zx, int dtype, long long zs, int col0, const float* conv_w,
                              const float* conv_b, const float* state, long long state_stride, long long conv_off,
                              const float* dtraw, const float* A_log, const float* dt_bias, const int* seg_of_token,
                              const int* cu_q, const int* state_slots, float* xbc, float* vout, float* decay, int T,
                              int H, int P, int C, int taps, hipStream_t stream) {
  if (T <= 0) return 0;
  if (!zx || !conv_w || !state || !dtraw || !A_log || !dt_bias || !xbc || !vout || !decay || H <= 0 || P <= 0 ||
      C < H * P || taps < 1 || taps > RS_MAX_TAPS || (C + H + 255) / 256 > 65535)
    return SA_ERR_ARG;
  const int per = T > 256 ? RS_PREP_TOKENS : 1;
  dim3 grid((T + per - 1) / per, (C + H + 255) / 256), block(256);
  if (dtype == SA_F32)
    hipLaunchKernelGGL(ssm_prepare_kernel<float>, grid, block, 0, stream, (const float*)zx, zs, col0, conv_w, conv_b,
                       state, state_stride, conv_off, dtraw, A_log, dt_bias, seg_of_token, cu_q, state_slots, xbc, vout,
                       decay, T, H, P, C, taps, per);
  else if (dtype == SA_BF16)
    hipLaunchKernelGGL(ssm_prepare_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)zx, zs, col0, conv_w, conv_b,
                       state, state_stride, conv_off, dtraw, A_log, dt_bias, seg_of_token, cu_q, state_slots, xbc, vout,
                       decay, T, H, P, C, taps, per);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The convolution's last taps - 1 inputs of every channel after the step: from the step's own tokens, and from the
// old state where the segment brought fewer than taps - 1.  grid (B, ceil(C / 256)).  Runs after every reader of the
// old state.
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void conv_state_update_kernel(
    const TA* __restrict__ zx, long long zs, int col0, float* __restrict__ state, long long state_stride,
    long long conv_off, const int* __restrict__ cu_q, const int* __restrict__ state_slots, int C, int taps) {
  const int seg = blockIdx.x;
  const int slot = state_slots[seg];
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (slot < 0 || c >= C) return;
  const int t0 = cu_q[seg], n = cu_q[seg + 1] - t0;
  float* cs = state + (size_t)slot * state_stride + conv_off;
  float nv[RS_MAX_TAPS - 1];
#pragma unroll
  for (int i = 0; i < RS_MAX_TAPS - 1; ++i) {
    if (i < taps - 1) {
      const int li = n - (taps - 1) + i;
      nv[i] = li >= 0 ? to_float(zx[(size_t)(t0 + li) * zs + col0 + c]) : cs[(size_t)(i + n) * C + c];
    }
  }
#pragma unroll
  for (int i = 0; i < RS_MAX_TAPS - 1; ++i)
    if (i < taps - 1) cs[(size_t)i * C + c] = nv[i];
}

extern "C" int sa_conv_state_update(const void* zx, int dtype, long long zs, int col0, float* state,
                                    long long state_stride, long long conv_off, const int* cu_q,
                                    const int* state_slots, int B, int C, int taps, hipStream_t stream) {
  if (B <= 0 || taps <= 1) return 0;
  if (!zx || !state || !cu_q || !state_slots || C <= 0 || taps > RS_MAX_TAPS || (C + 255) / 256 > 65535)
    return SA_ERR_ARG;
  dim3 grid(B, (C + 255) / 256), block(256);
  if (dtype == SA_F32)
    hipLaunchKernelGGL(conv_state_update_kernel<float>, grid, block, 0, stream, (const float*)zx, zs, col0, state,
                       state_stride, conv_off, cu_q, state_slots, C, taps);
  else if (dtype == SA_BF16)
    hipLaunchKernelGGL(conv_state_update_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)zx, zs, col0, state,
                       state_stride, conv_off, cu_q, state_slots, C, taps);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// What follows a recurrence's read-out o fp32 [T, n] (n = H dv), a wave per (token, norm group of `group` values):
//   u = o + skip_d[h] skip_x[t, i]                 (skip_x null: u = o)
//   gate_first:  u <- u silu(g[t, i]);  y = u / sqrt(mean_group(u^2) + eps) * w[i % wn]
//   else:        y = u / sqrt(mean_group(u^2) + eps) * w[i % wn] * silu(g[t, i])
// g: rows of gate_stride elements in the output's storage type, read from column gate_col on.
// ---------------------------------------------------------------------------------------------
// WAVES: how many waves share a group (1: a wave a group, four groups a workgroup of 256; 16: a workgroup of 1024 a
// group, for groups of thousands, where a few waves' chains of loads and divisions would decide the time of a
// decode step)
template <typename TA, int WAVES>
__global__ __launch_bounds__(WAVES == 1 ? 256 : 64 * WAVES) void gated_group_norm_kernel(
    const float* __restrict__ o, const float* __restrict__ skip_x, long long skip_stride,
    const float* __restrict__ skip_d, int dv, const TA* __restrict__ gate, long long gate_stride, int gate_col,
    const float* __restrict__ w, int wn, int group, int gate_first, float eps, TA* __restrict__ y, long long units,
    int n) {
  __shared__ float part[WAVES];
  constexpr int LANES = SA_WAVE * WAVES;
  const int lane = threadIdx.x & (LANES - 1);
  const long long unit = WAVES == 1 ? (long long)blockIdx.x * 4 + threadIdx.x / SA_WAVE : (long long)blockIdx.x;
  if (unit >= units) return;                    // (whole workgroups when a workgroup has one group)
  const int groups = n / group;
  const long long t = unit / groups;
  const int i0 = (int)(unit - t * groups) * group;
  const float* orow = o + (size_t)t * n;
  const TA* grow = gate + (size_t)t * gate_stride + gate_col;
  // a group of up to KEEP LANES values stays in registers between the two passes, and its loads are issued
  // together; a longer one is read twice
  constexpr int KEEP = 16;
  const bool kept = group <= KEEP * LANES;
  float ku[KEEP], kg[KEEP];
  float ss = 0.f;
  if (kept) {
    float ro[KEEP], rx[KEEP];
    TA rg[KEEP];
#pragma unroll
    for (int x = 0; x < KEEP; ++x) {               // the loads, with nothing between them that waits for one
      if (x * LANES >= group) break;
      const int i = i0 + min(lane + x * LANES, group - 1);
      ro[x] = orow[i];
      rx[x] = skip_x ? skip_x[(size_t)t * skip_stride + i] : 0.f;
      rg[x] = grow[i];
    }
#pragma unroll
    for (int x = 0; x < KEEP; ++x) {
      if (x * LANES >= group) break;
      const int e = lane + x * LANES, i = i0 + min(e, group - 1);
      float u = ro[x];
      if (skip_x) u = fmaf(skip_d[i / dv], rx[x], u);
      const float g = rs_silu(to_float(rg[x]));
      if (gate_first) u *= g;
      if (e >= group) u = 0.f;
      ku[x] = u;
      kg[x] = g;
      ss = fmaf(u, u, ss);
    }
  } else {
    for (int e = lane; e < group; e += LANES) {
      const int i = i0 + e;
      float u = orow[i];
      if (skip_x) u = fmaf(skip_d[i / dv], skip_x[(size_t)t * skip_stride + i], u);
      if (gate_first) u *= rs_silu(to_float(grow[i]));
      ss = fmaf(u, u, ss);
    }
  }
  ss = wave_sum(ss);
  if (WAVES > 1) {
    if ((threadIdx.x & (SA_WAVE - 1)) == 0) part[threadIdx.x / SA_WAVE] = ss;
    __syncthreads();
    ss = 0.f;
#pragma unroll
    for (int x = 0; x < WAVES; ++x) ss += part[x];
  }
  const float rs = 1.0f / sqrtf(ss / (float)group + eps);
  if (kept) {
#pragma unroll
    for (int x = 0; x < KEEP; ++x) {
      if (x * LANES >= group) break;
      const int e = lane + x * LANES, i = i0 + e;
      if (e < group) {
        float out = (ku[x] * rs) * w[i % wn];
        if (!gate_first) out *= kg[x];
        y[(size_t)t * n + i] = from_float<TA>(out);
      }
    }
    return;
  }
  for (int e = lane; e < group; e += LANES) {
    const int i = i0 + e;
    float u = orow[i];
    if (skip_x) u = fmaf(skip_d[i / dv], skip_x[(size_t)t * skip_stride + i], u);
    const float g = rs_silu(to_float(grow[i]));
    if (gate_first) u *= g;
    float out = (u * rs) * w[i % wn];
    if (!gate_first) out *= g;
    y[(size_t)t * n + i] = from_float<TA>(out);
  }
}

extern "C" int sa_gated_group_norm(const float* o, const float* skip_x, long long skip_stride, const float* skip_d,
                                   int dv, const void* gate, int dtype, long long gate_stride, int gate_col,
                                   const float* w, int wn, int group, int gate_first, float eps, void* y, int T, int n,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (!o || !gate || !w || !y || n <= 0 || group <= 0 || n % group || wn <= 0 || dv <= 0 || (skip_x && !skip_d))
    return SA_ERR_ARG;
  const long long units = (long long)T * (n / group);
  const bool whole = group >= 1024;             // a workgroup a group
  const long long blocks = whole ? units : (units + 3) / 4;
  if (blocks > 0x7fffffffLL) return SA_ERR_ARG;
  dim3 grid((unsigned)blocks), block(whole ? 1024 : 256);
#define GO(TA, W) hipLaunchKernelGGL((gated_group_norm_kernel<TA, W>), grid, block, 0, stream, o, skip_x, skip_stride, skip_d, dv, (const TA*)gate, gate_stride, gate_col, w, wn, group, gate_first, eps, (TA*)y, units, n)
  if (dtype == SA_F32) {
    if (whole) GO(float, 16); else GO(float, 1);
  } else if (dtype == SA_BF16) {
    if (whole) GO(bf16_t, 16); else GO(bf16_t, 1);
  } else {
    return SA_ERR_UNSUPPORTED;
  }
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}
