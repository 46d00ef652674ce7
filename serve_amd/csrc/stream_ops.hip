// Elementwise kernels around the fp32 residual stream x [T, d] that are neither a norm of the stream nor a norm of
// one sublayer's output: an addition with an optional row vector, a second fp32 array and a copy, the mean of two
// normed outputs, the gate of a second, per-token embedding, and an embedding with a hashed row of the token pair.
// fp32 arithmetic; the storage types of activations are templated.
#include "common.h"

// y[t] as the sum of its parts (fp32 [parts, T, d] partial sums of a product, or one [T, d] array)
template <typename TD>
__device__ __forceinline__ float parts_at(const TD* y, int parts, size_t part_stride, size_t at) {
  float v = 0.f;
  for (int p = 0; p < parts; ++p) v += to_float(y[p * part_stride + at]);
  return v;
}

// ---------------------------------------------------------------------------------------------
// x[t] += y[t] + vec + extra[t]  (each may be missing; extra fp32 [T, d]), and h[t] = x[t] in the activation dtype
// (h may be missing).
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TD>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ x, const TD* __restrict__ y, int parts,
                                                         size_t part_stride, const float* __restrict__ vec,
                                                         const float* __restrict__ extra, TA* __restrict__ h, int d) {
  const size_t t = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
    const size_t at = t * d + i;
    float v = x[at];
    if (y) v += parts_at(y, parts, part_stride, at);
    if (extra) v += extra[at];
    if (vec) v += vec[i];
    x[at] = v;
    if (h) h[at] = from_float<TA>(v);
  }
}

template <typename TA>
static int launch_stream_add(float* x, const void* y, int y_dtype, int parts, const float* vec, const float* extra,
                             void* h, int T, int d, hipStream_t stream) {
  const size_t ps = (size_t)T * d;
  // a step of few rows: a value a thread, so that a row's loads are not a chain in one workgroup
  dim3 grid(T, T <= 64 ? (unsigned)((d + 255) / 256) : 1u), block(256);
  if (!y || y_dtype == SA_F32)
    hipLaunchKernelGGL((stream_add_kernel<TA, float>), grid, block, 0, stream, x, (const float*)y, parts, ps, vec, extra, (TA*)h, d);
  else if (y_dtype == SA_BF16)
    hipLaunchKernelGGL((stream_add_kernel<TA, bf16_t>), grid, block, 0, stream, x, (const bf16_t*)y, parts, ps, vec, extra, (TA*)h, d);
  else
    return SA_ERR_UNSUPPORTED;
  return 0;
}

extern "C" int sa_stream_add(float* x, const void* y, int y_dtype, int parts, const float* vec, const float* extra,
                             void* h, int h_dtype, int T, int d, hipStream_t stream) {
  if (T <= 0) return 0;
  if (!x || d <= 0 || parts < 1 || (parts > 1 && y_dtype != SA_F32)) return SA_ERR_ARG;
  int rc;
  if (h_dtype == SA_F32) rc = launch_stream_add<float>(x, y, y_dtype, parts, vec, extra, h, T, d, stream);
  else if (h_dtype == SA_BF16) rc = launch_stream_add<bf16_t>(x, y, y_dtype, parts, vec, extra, h, T, d, stream);
  else return SA_ERR_UNSUPPORTED;
  if (rc != 0) return rc;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Two mixers side by side: out[t] = ca N(a[t]) wa + cb N(b[t]) wb,  N(y) = y / sqrt(mean(y^2) + eps), fp32 out [T, d].
// a and b: [T, d] or fp32 [parts, T, d] each.  One workgroup a row; a thread keeps up to VMAX values of each.  A step
// of few rows takes workgroups of 1024 threads: a row's partial sums are then a few loads a thread, not a chain.
// ---------------------------------------------------------------------------------------------
template <typename TDA, typename TDB>
__global__ __launch_bounds__(1024) void dual_norm_mix_kernel(const TDA* __restrict__ a, int parts_a,
                                                            const TDB* __restrict__ b, int parts_b,
                                                            size_t part_stride, const float* __restrict__ wa,
                                                            const float* __restrict__ wb, float ca, float cb, float eps,
                                                            float* __restrict__ out, int d) {
  __shared__ float scratch[16];
  constexpr int VMAX = 8;
  const size_t t = blockIdx.x;
  const int bd = blockDim.x;
  float ka[VMAX], kb[VMAX];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int n = 0; n < VMAX; ++n) {
    const int i = threadIdx.x + n * bd;
    float va = 0.f, vb = 0.f;
    if (i < d) {
      va = parts_at(a, parts_a, part_stride, t * d + i);
      vb = parts_at(b, parts_b, part_stride, t * d + i);
    }
    ka[n] = va;
    kb[n] = vb;
    sa = fmaf(va, va, sa);
    sb = fmaf(vb, vb, sb);
  }
  for (int i = threadIdx.x + VMAX * bd; i < d; i += bd) {
    const float va = parts_at(a, parts_a, part_stride, t * d + i), vb = parts_at(b, parts_b, part_stride, t * d + i);
    sa = fmaf(va, va, sa);
    sb = fmaf(vb, vb, sb);
  }
  sa = block_sum(sa, scratch);
  sb = block_sum(sb, scratch);
  const float ra = 1.0f / sqrtf(sa / (float)d + eps), rb = 1.0f / sqrtf(sb / (float)d + eps);
#pragma unroll
  for (int n = 0; n < VMAX; ++n) {
    const int i = threadIdx.x + n * bd;
    if (i < d) out[t * d + i] = ca * ((ka[n] * ra) * wa[i]) + cb * ((kb[n] * rb) * wb[i]);
  }
  for (int i = threadIdx.x + VMAX * bd; i < d; i += bd) {
    const float va = parts_at(a, parts_a, part_stride, t * d + i), vb = parts_at(b, parts_b, part_stride, t * d + i);
    out[t * d + i] = ca * ((va * ra) * wa[i]) + cb * ((vb * rb) * wb[i]);
  }
}

extern "C" int sa_dual_norm_mix(const void* a, int a_dtype, int parts_a, const void* b, int b_dtype, int parts_b,
                                const float* wa, const float* wb, float ca, float cb, float eps, float* out, int T, int d,
                                hipStream_t stream) {
  if (T <= 0) return 0;
  if (!a || !b || !wa || !wb || !out || d <= 0 || parts_a < 1 || parts_b < 1 || (parts_a > 1 && a_dtype != SA_F32) ||
      (parts_b > 1 && b_dtype != SA_F32))
    return SA_ERR_ARG;
  const size_t ps = (size_t)T * d;
  dim3 grid(T), block(T <= 64 && d >= 1024 ? 1024 : 256);
#define GO(TDA, TDB)                                                                                             \
  hipLaunchKernelGGL((dual_norm_mix_kernel<TDA, TDB>), grid, block, 0, stream, (const TDA*)a, parts_a, (const TDB*)b, \
                     parts_b, ps, wa, wb, ca, cb, eps, out, d)
  if (a_dtype == SA_F32 && b_dtype == SA_F32) GO(float, float);
  else if (a_dtype == SA_F32 && b_dtype == SA_BF16) GO(float, bf16_t);
  else if (a_dtype == SA_BF16 && b_dtype == SA_F32) GO(bf16_t, float);
  else if (a_dtype == SA_BF16 && b_dtype == SA_BF16) GO(bf16_t, bf16_t);
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// g[t, j] = gelu_tanh(z[t, j]) * table[token_t, col0 + j], j < n: the gate of an input made from a second embedding
// row of the token.  The token of row t is tokens[t], or prev[src_row[t]] where src_row[t] >= 0 (a token that an
// earlier step sampled on the device).
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TW>
__global__ __launch_bounds__(256) void gelu_mul_rows_kernel(const TA* __restrict__ z, const TW* __restrict__ table,
                                                            long long table_stride, int col0,
                                                            const int* __restrict__ tokens,
                                                            const int* __restrict__ src_row, const int* __restrict__ prev,
                                                            TA* __restrict__ g, int n, int V) {
  const size_t t = blockIdx.x;
  int tok = tokens[t];
  if (src_row && src_row[t] >= 0) tok = prev[src_row[t]];
  tok = min(max(tok, 0), V - 1);
  const TW* row = table + (size_t)tok * table_stride + col0;
  for (int j = threadIdx.x; j < n; j += blockDim.x) {
    const float v = to_float(z[t * n + j]);
    const float act = 0.5f * v * (1.f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    g[t * n + j] = from_float<TA>(act * to_float(row[j]));
  }
}

extern "C" int sa_gelu_mul_rows(const void* z, int act_dtype, const void* table, int table_dtype, long long table_stride,
                                int col0, const int* tokens, const int* src_row, const int* prev, void* g, int T, int n,
                                int V, hipStream_t stream) {
  if (T <= 0) return 0;
  if (!z || !table || !tokens || !g || n <= 0 || V <= 0 || col0 < 0 || table_stride < col0 + n || (src_row && !prev))
    return SA_ERR_ARG;
  dim3 grid(T), block(n >= 256 ? 256 : 64);
#define GO(TA, TW)                                                                                                    \
  hipLaunchKernelGGL((gelu_mul_rows_kernel<TA, TW>), grid, block, 0, stream, (const TA*)z, (const TW*)table, table_stride, \
                     col0, tokens, src_row, prev, (TA*)g, n, V)
  if (act_dtype == SA_F32 && table_dtype == SA_F32) GO(float, float);
  else if (act_dtype == SA_BF16 && table_dtype == SA_BF16) GO(bf16_t, bf16_t);
  else if (act_dtype == SA_BF16 && table_dtype == SA_F32) GO(bf16_t, float);
  else if (act_dtype == SA_F32 && table_dtype == SA_BF16) GO(float, bf16_t);
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// An embedding with a second row for the pair (previous token, token):
//   x[t] = E[tok_t] + B[r_t],   r_t = (prev_t * mul_prev + tok_t * mul_cur) mod buckets,   r_t = buckets where the token
//   is its sequence's first (position 0): the table B has buckets + 1 rows.
// prev_t is the token before t in its segment, or, for a segment's first token, what the request's state row holds
// (`last` int32 [slots], by state_slot[segment]; slot < 0: a segment of no request, which takes row `buckets`).
// The token of row t is tokens[t], or sampled[src_row[t]] where src_row[t] >= 0 (a token that an earlier step
// sampled on the device).  `keep` (may be null) receives a second copy of x.  Grid (T, parts of a row).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int token_at(const int* __restrict__ tokens, const int* __restrict__ src_row,
                                        const int* __restrict__ sampled, int t, int V) {
  int tok = tokens[t];
  if (src_row && src_row[t] >= 0) tok = sampled[src_row[t]];
  return min(max(tok, 0), V - 1);
}

template <typename TW>
__global__ __launch_bounds__(256) void pair_embed_kernel(const TW* __restrict__ E, const TW* __restrict__ B,
                                                         const int* __restrict__ tokens, const int* __restrict__ src_row,
                                                         const int* __restrict__ sampled,
                                                         const int* __restrict__ positions,
                                                         const int* __restrict__ seg_of_token,
                                                         const int* __restrict__ cu_q, const int* __restrict__ state_slot,
                                                         int* __restrict__ last, float* __restrict__ x,
                                                         float* __restrict__ keep, int d, int V, int buckets,
                                                         long long mul_prev, long long mul_cur) {
  const int t = blockIdx.x;
  const int tok = token_at(tokens, src_row, sampled, t, V);
  const int seg = seg_of_token[t];
  const int begin = cu_q[seg];
  const int slot = state_slot[seg];
  int prev = -1;
  if (positions[t] > 0) {
    if (t > begin) prev = token_at(tokens, src_row, sampled, t - 1, V);
    else if (slot >= 0) prev = last[slot];
  }
  const long long r = prev < 0 ? (long long)buckets : ((long long)prev * mul_prev + (long long)tok * mul_cur) % buckets;
  const TW* er = E + (size_t)tok * d;
  const TW* br = B + (size_t)r * d;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
    const float v = to_float(er[i]) + to_float(br[i]);
    x[(size_t)t * d + i] = v;
    if (keep) keep[(size_t)t * d + i] = v;
  }
}

// after the embedding: last[slot] = the last token of every segment that belongs to a request.  A kernel of its own,
// so that no workgroup of the embedding reads a row that another has already replaced.
__global__ __launch_bounds__(256) void pair_embed_state_kernel(const int* __restrict__ tokens,
                                                               const int* __restrict__ src_row,
                                                               const int* __restrict__ sampled,
                                                               const int* __restrict__ cu_q,
                                                               const int* __restrict__ state_slot, int* __restrict__ last,
                                                               int B, int V) {
  const int seg = blockIdx.x * blockDim.x + threadIdx.x;
  if (seg >= B) return;
  const int slot = state_slot[seg];
  const int end = cu_q[seg + 1];
  if (slot >= 0 && end > cu_q[seg]) last[slot] = token_at(tokens, src_row, sampled, end - 1, V);
}

extern "C" int sa_pair_embed(const void* E, const void* B, int table_dtype, const int* tokens, const int* src_row,
                             const int* sampled, const int* positions, const int* seg_of_token, const int* cu_q,
                             const int* state_slot, int* last, float* x, float* keep, int T, int segments, int d, int V,
                             int buckets, long long mul_prev, long long mul_cur, hipStream_t stream) {
  if (T <= 0) return 0;
  if (!E || !B || !tokens || !positions || !seg_of_token || !cu_q || !state_slot || !last || !x || d <= 0 || V <= 0 ||
      buckets <= 0 || segments <= 0 || mul_prev < 0 || mul_cur < 0 || (src_row && !sampled))
    return SA_ERR_ARG;
  dim3 grid(T, T <= 64 ? (unsigned)((d + 255) / 256) : 1u), block(256);
  if (table_dtype == SA_F32)
    hipLaunchKernelGGL(pair_embed_kernel<float>, grid, block, 0, stream, (const float*)E, (const float*)B, tokens, src_row,
                       sampled, positions, seg_of_token, cu_q, state_slot, last, x, keep, d, V, buckets, mul_prev, mul_cur);
  else if (table_dtype == SA_BF16)
    hipLaunchKernelGGL(pair_embed_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)E, (const bf16_t*)B, tokens,
                       src_row, sampled, positions, seg_of_token, cu_q, state_slot, last, x, keep, d, V, buckets, mul_prev,
                       mul_cur);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  hipLaunchKernelGGL(pair_embed_state_kernel, dim3((segments + 255) / 256), dim3(256), 0, stream, tokens, src_row, sampled,
                     cu_q, state_slot, last, segments, V);
  SA_LAUNCH_CHECK();
  return 0;
}
