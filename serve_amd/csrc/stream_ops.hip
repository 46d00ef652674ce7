// Elementwise kernels around the fp32 residual stream x [T, d] that are neither a norm of the stream nor a norm of
// one sublayer's output: an addition with an optional row vector and copy, the mean of two normed outputs, and the
// gate of a second, per-token embedding.  fp32 arithmetic; the storage types of activations are templated.
#include "common.h"

// y[t] as the sum of its parts (fp32 [parts, T, d] partial sums of a product, or one [T, d] array)
template <typename TD>
__device__ __forceinline__ float parts_at(const TD* y, int parts, size_t part_stride, size_t at) {
  float v = 0.f;
  for (int p = 0; p < parts; ++p) v += to_float(y[p * part_stride + at]);
  return v;
}

// ---------------------------------------------------------------------------------------------
// x[t] += y[t] + vec  (either may be missing), and h[t] = x[t] in the activation dtype (h may be missing).
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TD>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ x, const TD* __restrict__ y, int parts,
                                                         size_t part_stride, const float* __restrict__ vec,
                                                         TA* __restrict__ h, int d) {
  const size_t t = blockIdx.x;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < d; i += blockDim.x * gridDim.y) {
    const size_t at = t * d + i;
    float v = x[at];
    if (y) v += parts_at(y, parts, part_stride, at);
    if (vec) v += vec[i];
    x[at] = v;
    if (h) h[at] = from_float<TA>(v);
  }
}

template <typename TA>
static int launch_stream_add(float* x, const void* y, int y_dtype, int parts, const float* vec, void* h, int T, int d,
                             hipStream_t stream) {
  const size_t ps = (size_t)T * d;
  // a step of few rows: a value a thread, so that a row's loads are not a chain in one workgroup
  dim3 grid(T, T <= 64 ? (unsigned)((d + 255) / 256) : 1u), block(256);
  if (!y || y_dtype == SA_F32)
    hipLaunchKernelGGL((stream_add_kernel<TA, float>), grid, block, 0, stream, x, (const float*)y, parts, ps, vec, (TA*)h, d);
  else if (y_dtype == SA_BF16)
    hipLaunchKernelGGL((stream_add_kernel<TA, bf16_t>), grid, block, 0, stream, x, (const bf16_t*)y, parts, ps, vec, (TA*)h, d);
  else
    return SA_ERR_UNSUPPORTED;
  return 0;
}

extern "C" int sa_stream_add(float* x, const void* y, int y_dtype, int parts, const float* vec, void* h, int h_dtype,
                             int T, int d, hipStream_t stream) {
  if (T <= 0) return 0;
  if (!x || d <= 0 || parts < 1 || (parts > 1 && y_dtype != SA_F32)) return SA_ERR_ARG;
  int rc;
  if (h_dtype == SA_F32) rc = launch_stream_add<float>(x, y, y_dtype, parts, vec, h, T, d, stream);
  else if (h_dtype == SA_BF16) rc = launch_stream_add<bf16_t>(x, y, y_dtype, parts, vec, h, T, d, stream);
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
