// Mixers whose memory is one fp32 matrix S [dk, dv] per head and request that decays and takes an outer product a token:
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t          a_t: a vector over dk, or one number a head
//
// A gated linear attention is this with a decay per key channel; a selective state-space mixer with S [state, head dim],
// k = B_t, q = C_t, v = dt_t x_t and the one decay exp(-exp(A_log) dt_t) a head.  What differs between such mixers lies
// in front of the recurrence (how q, k, v and the decays are made) and behind it (norm and gate of the read-out), so the
// file has the recurrence itself (`decay_scan`), the two preparations (`gla_decay`; `ssm_prepare` with the causal
// convolution, and `conv_state_update` for the convolution's last inputs) and one kernel for what follows (`gated_group_norm`).
// All arithmetic is fp32; template types are the storage of projections and outputs.
#include "common.h"

#define RS_MAX_TAPS 16

__device__ __forceinline__ float rs_silu(float z) { return z / (1.f + expf(-z)); }
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
    long long k_stride, long long v_stride, const float* __restrict__ decay, int per_channel, float q_scale,
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
      const float av = per_channel ? decay[(tok * H + h) * (size_t)dk + ic] : decay[tok * H + h];
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

// q, k: rows of `q_stride` / `k_stride` elements with head hk's dk values at hk dk (Hk heads; head h reads hk = h / (H / Hk));
// v: rows of `v_stride` with head h's dv values at h dv; decay fp32 [T, H, dk] (per_channel) or [T, H]; o fp32 [T, H, dv];
// state: a request's row at state + slot state_stride (the floats that sa_decay_scan_state_floats counts), slot < 0: a
// segment without a request, which starts from zeros and keeps nothing.
extern "C" int sa_decay_scan(const void* q, const void* k, const void* v, int dtype, long long q_stride,
                             long long k_stride, long long v_stride, const float* decay, int per_channel,
                             float q_scale, float* state, long long state_stride, const int* cu_q,
                             const int* state_slots, float* o, int B, int H, int Hk, int dk, int dv,
                             hipStream_t stream) {
  if (B <= 0) return 0;
  if (H <= 0 || Hk <= 0 || H % Hk || dk <= 0 || dk > 256 || dv <= 0 || !q || !k || !v || !decay || !state || !o ||
      !cu_q || !state_slots || B > 65535 || H > 65535)
    return SA_ERR_ARG;
  const int rpt = scan_rpt(dk), cpt = scan_cpt(dv);
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
// decay[t, c] = sigmoid(z[t, c] + b[c])^(1 / tau) = exp(ln sigmoid(z + b) / tau), c over H dk channels
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gla_decay_kernel(const float* __restrict__ z, const float* __restrict__ bias,
                                                        float inv_tau, float* __restrict__ decay, long long total,
                                                        int C) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % C);
  decay[idx] = expf(rs_logsigmoid(z[idx] + (bias ? bias[c] : 0.f)) * inv_tau);
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
// Per token and head: dt = softplus(dtraw + dt_bias), decay = exp(-exp(A_log) dt); v = dt x -> fp32 [T, H P].
// grid (T, ceil((C + H) / 256)).
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void ssm_prepare_kernel(
    const TA* __restrict__ zx, long long zs, int col0, const float* __restrict__ conv_w,
    const float* __restrict__ conv_b, const float* __restrict__ state, long long state_stride, long long conv_off,
    const float* __restrict__ dtraw, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
    const int* __restrict__ seg_of_token, const int* __restrict__ cu_q, const int* __restrict__ state_slots,
    float* __restrict__ xbc, float* __restrict__ vout, float* __restrict__ decay, int H, int P, int C, int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C + H) return;
  if (c >= C) {
    const int h = c - C;
    const float dt = rs_softplus(dtraw[(size_t)t * H + h] + dt_bias[h]);
    decay[(size_t)t * H + h] = expf(-expf(A_log[h]) * dt);
    return;
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
  if (c < H * P) {
    const int h = c / P;
    const float dt = rs_softplus(dtraw[(size_t)t * H + h] + dt_bias[h]);
    vout[(size_t)t * H * P + c] = dt * y;
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
  dim3 grid(T, (C + H + 255) / 256), block(256);
  if (dtype == SA_F32)
    hipLaunchKernelGGL(ssm_prepare_kernel<float>, grid, block, 0, stream, (const float*)zx, zs, col0, conv_w, conv_b,
                       state, state_stride, conv_off, dtraw, A_log, dt_bias, seg_of_token, cu_q, state_slots, xbc, vout,
                       decay, H, P, C, taps);
  else if (dtype == SA_BF16)
    hipLaunchKernelGGL(ssm_prepare_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)zx, zs, col0, conv_w, conv_b,
                       state, state_stride, conv_off, dtraw, A_log, dt_bias, seg_of_token, cu_q, state_slots, xbc, vout,
                       decay, H, P, C, taps);
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
template <typename TA>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
    const float* __restrict__ o, const float* __restrict__ skip_x, long long skip_stride,
    const float* __restrict__ skip_d, int dv, const TA* __restrict__ gate, long long gate_stride, int gate_col,
    const float* __restrict__ w, int wn, int group, int gate_first, float eps, TA* __restrict__ y, long long units,
    int n) {
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const long long unit = (long long)blockIdx.x * (256 / SA_WAVE) + threadIdx.x / SA_WAVE;
  if (unit >= units) return;
  const int groups = n / group;
  const long long t = unit / groups;
  const int i0 = (int)(unit - t * groups) * group;
  const float* orow = o + (size_t)t * n;
  const TA* grow = gate + (size_t)t * gate_stride + gate_col;
  float ss = 0.f;
  for (int e = lane; e < group; e += SA_WAVE) {
    const int i = i0 + e;
    float u = orow[i];
    if (skip_x) u = fmaf(skip_d[i / dv], skip_x[(size_t)t * skip_stride + i], u);
    if (gate_first) u *= rs_silu(to_float(grow[i]));
    ss = fmaf(u, u, ss);
  }
  ss = wave_sum(ss);
  const float rs = 1.0f / sqrtf(ss / (float)group + eps);
  for (int e = lane; e < group; e += SA_WAVE) {
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
  const long long blocks = (units + 3) / 4;
  if (blocks > 0x7fffffffLL) return SA_ERR_ARG;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == SA_F32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, grid, block, 0, stream, o, skip_x, skip_stride, skip_d, dv,
                       (const float*)gate, gate_stride, gate_col, w, wn, group, gate_first, eps, (float*)y, units, n);
  else if (dtype == SA_BF16)
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, grid, block, 0, stream, o, skip_x, skip_stride, skip_d, dv,
                       (const bf16_t*)gate, gate_stride, gate_col, w, wn, group, gate_first, eps, (bf16_t*)y, units, n);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
