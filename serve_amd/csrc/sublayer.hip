// Elementwise kernels of layers whose norm sits on the sublayer's output:
//   x <- x + s * N(y),  N(y) = y / sqrt(mean(y^2) + eps) * w      (x: fp32 residual stream)
// and of feed-forwards with a plain activation between two products.  fp32 arithmetic; the
// storage types of activations are templated.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// x[t] += (N(y[t]) * w) * s, and h[t] = x[t] in the activation dtype for the sublayer that reads
// the stream next.  y is [T, d] in the activation dtype or fp32, or fp32 [parts, T, d] partial
// sums that are added in order (a product whose inner dimension was cut across workgroups, the
// experts of a token).  y == nullptr: only the copy h = x is made.  h == nullptr: no copy.
// nw != nullptr (with y and h): h[t] = N(x[t]) * nw instead, the norm (eps `neps`) of the new stream that the
// next sublayer reads: a layer with a norm behind one sublayer and another in front of the next needs one
// kernel between the two.
// One workgroup a row; a thread keeps up to VMAX of its values between the two passes, the rest
// is read again.
// ---------------------------------------------------------------------------------------------
template <typename TA, typename TD>
__global__ __launch_bounds__(256) void output_norm_add_kernel(float* __restrict__ x, const TD* __restrict__ y,
                                                              int parts, size_t part_stride,
                                                              const float* __restrict__ w,
                                                              const float* __restrict__ s, TA* __restrict__ h,
                                                              float eps, int d, const float* __restrict__ nw,
                                                              float neps) {
  __shared__ float scratch[16];
  constexpr int VMAX = 8;
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * d;
  TA* hr = h ? h + (size_t)t * d : nullptr;
  if (!y) {
    if (hr)
      for (int i = threadIdx.x; i < d; i += blockDim.x) hr[i] = from_float<TA>(xr[i]);
    return;
  }
  const TD* yr = y + (size_t)t * d;
  float keep[VMAX];
  float ss = 0.f;
  const int bd = blockDim.x;
#pragma unroll
  for (int n = 0; n < VMAX; ++n) {
    const int i = threadIdx.x + n * bd;
    float v = 0.f;
    if (i < d)
      for (int p = 0; p < parts; ++p) v += to_float(yr[p * part_stride + i]);
    keep[n] = v;
    ss += v * v;
  }
  for (int i = threadIdx.x + VMAX * bd; i < d; i += bd) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += to_float(yr[p * part_stride + i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rs = 1.0f / sqrtf(ss / (float)d + eps);
  const bool copy = hr && !nw;
  float ss2 = 0.f;
#pragma unroll
  for (int n = 0; n < VMAX; ++n) {
    const int i = threadIdx.x + n * bd;
    if (i < d) {
      const float nx = xr[i] + ((keep[n] * rs) * w[i]) * s[i];
      xr[i] = nx;
      keep[n] = nx;
      ss2 += nx * nx;
      if (copy) hr[i] = from_float<TA>(nx);
    }
  }
  for (int i = threadIdx.x + VMAX * bd; i < d; i += bd) {
    float v = 0.f;
    for (int p = 0; p < parts; ++p) v += to_float(yr[p * part_stride + i]);
    const float nx = xr[i] + ((v * rs) * w[i]) * s[i];
    xr[i] = nx;
    ss2 += nx * nx;
    if (copy) hr[i] = from_float<TA>(nx);
  }
  if (!hr || !nw) return;
  // the norm of the new stream (every thread reads back only what it wrote itself)
  ss2 = block_sum(ss2, scratch);
  const float rs2 = rsqrtf(ss2 / (float)d + neps);
#pragma unroll
  for (int n = 0; n < VMAX; ++n) {
    const int i = threadIdx.x + n * bd;
    if (i < d) hr[i] = from_float<TA>((keep[n] * rs2) * nw[i]);
  }
  for (int i = threadIdx.x + VMAX * bd; i < d; i += bd) hr[i] = from_float<TA>((xr[i] * rs2) * nw[i]);
}

// The same for d % 4 == 0 and d <= 8192: 16-byte vectors, and every load of a row (the parts of y, x, w, s) is
// issued before anything is added, so that a row costs one trip to memory.  PMAX: upper bound of `parts`; a part
// beyond `parts` is read from a clamped address and dropped.
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_bits_to_float(u.x & 0xffffu), bf16_bits_to_float(u.x >> 16),
                     bf16_bits_to_float(u.y & 0xffffu), bf16_bits_to_float(u.y >> 16));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  u.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

template <typename TA, typename TD, int PMAX, int NG>
__global__ __launch_bounds__(256) void output_norm_add_vec_kernel(float* __restrict__ x, const TD* __restrict__ y,
                                                                  int parts, size_t part_stride,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ s, TA* __restrict__ h,
                                                                  float eps, int d, const float* __restrict__ nw,
                                                                  float neps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * d;
  const TD* yr = y + (size_t)t * d;
  const int groups = d >> 2;
  float4 v[NG], xv[NG], wv[NG], sv[NG];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NG; ++k) {
    const int gi = threadIdx.x + k * 256;
    const int i = min(gi, groups - 1) * 4;
    float4 a[PMAX];
#pragma unroll
    for (int p = 0; p < PMAX; ++p) a[p] = ld4(yr + (size_t)min(p, parts - 1) * part_stride + i);
    xv[k] = ld4(xr + i);
    wv[k] = ld4(w + i);
    sv[k] = ld4(s + i);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int p = 0; p < PMAX; ++p) {
      const float on = p < parts ? 1.f : 0.f;
      acc.x += on * a[p].x; acc.y += on * a[p].y; acc.z += on * a[p].z; acc.w += on * a[p].w;
    }
    v[k] = acc;
    const float in = gi < groups ? 1.f : 0.f;
    ss += in * (acc.x * acc.x + acc.y * acc.y + acc.z * acc.z + acc.w * acc.w);
  }
  ss = block_sum(ss, scratch);
  const float rs = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
  for (int k = 0; k < NG; ++k) {
    const int gi = threadIdx.x + k * 256;
    if (gi < groups) {
      const int i = gi * 4;
      float4 nx;
      nx.x = xv[k].x + ((v[k].x * rs) * wv[k].x) * sv[k].x;
      nx.y = xv[k].y + ((v[k].y * rs) * wv[k].y) * sv[k].y;
      nx.z = xv[k].z + ((v[k].z * rs) * wv[k].z) * sv[k].z;
      nx.w = xv[k].w + ((v[k].w * rs) * wv[k].w) * sv[k].w;
      st4(xr + i, nx);
      if (h && !nw) st4(h + (size_t)t * d + i, nx);
      v[k] = nx;
    }
  }
  if (!h || !nw) return;
  // the norm of the new stream, from the values still in registers
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < NG; ++k) {
    const float in = threadIdx.x + k * 256 < groups ? 1.f : 0.f;
    ss2 += in * (v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w);
  }
  ss2 = block_sum(ss2, scratch);
  const float rs2 = rsqrtf(ss2 / (float)d + neps);
#pragma unroll
  for (int k = 0; k < NG; ++k) {
    const int gi = threadIdx.x + k * 256;
    if (gi < groups) {
      const int i = gi * 4;
      const float4 n4 = ld4(nw + i);
      st4(h + (size_t)t * d + i, make_float4((v[k].x * rs2) * n4.x, (v[k].y * rs2) * n4.y, (v[k].z * rs2) * n4.z,
                                             (v[k].w * rs2) * n4.w));
    }
  }
}

extern "C" int sa_output_norm_add(float* x, const void* y, int y_dtype, int parts, const float* w, const float* s,
                                  void* h, int act_dtype, float eps, int T, int d, const float* nw, float neps,
                                  hipStream_t stream) {
  if (T <= 0) return 0;
  if (d <= 0 || parts < 1) return SA_ERR_ARG;
  if (nw && (!y || !h)) return SA_ERR_ARG;
  if (y && (!w || !s)) return SA_ERR_ARG;
  if (y && y_dtype != act_dtype && y_dtype != SA_F32) return SA_ERR_UNSUPPORTED;
  if (y && parts > 1 && y_dtype != SA_F32) return SA_ERR_UNSUPPORTED;
  const size_t part_stride = (size_t)T * d;
  dim3 grid(T), block(d >= 1024 ? 256 : (d >= 256 ? 128 : 64));
  if (y && (d & 3) == 0 && d >= 256 && d <= 8192 && parts <= 8) {
    const int ng = (d / 4 + 255) / 256;          // groups of four a thread, 1 .. 8
#define GOV(TA, TD, PMAX, NG)                                                                                   \
  hipLaunchKernelGGL((output_norm_add_vec_kernel<TA, TD, PMAX, NG>), grid, dim3(256), 0, stream, x,             \
                     (const TD*)y, parts, part_stride, w, s, (TA*)h, eps, d, nw, neps)
#define GON(TA, TD, PMAX)                                                                                       \
  do {                                                                                                          \
    if (ng <= 1) GOV(TA, TD, PMAX, 1);                                                                          \
    else if (ng <= 2) GOV(TA, TD, PMAX, 2);                                                                     \
    else if (ng <= 4) GOV(TA, TD, PMAX, 4);                                                                     \
    else GOV(TA, TD, PMAX, 8);                                                                                  \
  } while (0)
#define GOP(TA, TD)                                                                                             \
  do {                                                                                                          \
    if (parts == 1) GON(TA, TD, 1);                                                                             \
    else if (parts <= 4) GON(TA, TD, 4);                                                                        \
    else GON(TA, TD, 8);                                                                                        \
  } while (0)
    if (act_dtype == SA_F32) GOP(float, float);
    else if (act_dtype == SA_BF16) { if (y_dtype == SA_F32) GOP(bf16_t, float); else GON(bf16_t, bf16_t, 1); }
    else return SA_ERR_UNSUPPORTED;
#undef GOP
#undef GON
#undef GOV
    SA_LAUNCH_CHECK();
    return 0;
  }
#define GO(TA, TD)                                                                                          \
  hipLaunchKernelGGL((output_norm_add_kernel<TA, TD>), grid, block, 0, stream, x, (const TD*)y, parts,      \
                     part_stride, w, s, (TA*)h, eps, d, nw, neps)
  const bool yfloat = !y || y_dtype == SA_F32;
  if (act_dtype == SA_F32) GO(float, float);
  else if (act_dtype == SA_BF16) { if (yfloat) GO(bf16_t, float); else GO(bf16_t, bf16_t); }
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// a[i] = act(a[i]) in place.  kind 0: gelu, tanh form: 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)));
// kind 1: silu.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh_f(float z) {
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  return 0.5f * z * (1.f + tanhf(u));
}

// kind 0: gelu (tanh form), 1: silu, 2: the square of relu
__device__ __forceinline__ float activate(float z, int kind) {
  if (kind == 0) return gelu_tanh_f(z);
  if (kind == 1) return z / (1.f + expf(-z));
  const float r = fmaxf(z, 0.f);
  return r * r;
}

template <typename TA>
__global__ void activation_kernel(TA* __restrict__ a, size_t n, int kind) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const float z = to_float(a[i]);
    a[i] = from_float<TA>(activate(z, kind));
  }
}

// the same, eight bf16 values a thread in 16-byte vectors (n % 8 == 0, 16-byte aligned)
__global__ __launch_bounds__(256) void activation_bf16x8_kernel(bf16_t* __restrict__ a, size_t groups, int kind) {
  for (size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gi < groups; gi += (size_t)gridDim.x * blockDim.x) {
    uint4 v = *reinterpret_cast<const uint4*>(a + gi * 8);
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float z0 = bf16_bits_to_float(w[k] & 0xffffu), z1 = bf16_bits_to_float(w[k] >> 16);
      const float r0 = activate(z0, kind), r1 = activate(z1, kind);
      w[k] = (uint32_t)float_to_bf16_bits(r0) | ((uint32_t)float_to_bf16_bits(r1) << 16);
    }
    *reinterpret_cast<uint4*>(a + gi * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

extern "C" int sa_activation(void* a, int act_dtype, long long n, int kind, hipStream_t stream) {
  if (n <= 0) return 0;
  if (kind < 0 || kind > 2) return SA_ERR_ARG;
  if (act_dtype == SA_BF16 && (n & 7) == 0 && ((uintptr_t)a & 15) == 0) {
    long long vb = (n / 8 + 255) / 256;
    if (vb > 65536) vb = 65536;
    hipLaunchKernelGGL(activation_bf16x8_kernel, dim3((unsigned)vb), dim3(256), 0, stream, (bf16_t*)a, (size_t)(n / 8), kind);
    SA_LAUNCH_CHECK();
    return 0;
  }
  long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  dim3 grid((unsigned)blocks), block(256);
  if (act_dtype == SA_F32) hipLaunchKernelGGL(activation_kernel<float>, grid, block, 0, stream, (float*)a, (size_t)n, kind);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL(activation_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)a, (size_t)n, kind);
  else return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// An element-wise output gate: a[i] *= sigmoid(g[i]), in place, a and g of one shape and dtype.
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ void sigmoid_mul_kernel(TA* __restrict__ a, const TA* __restrict__ g, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    a[i] = from_float<TA>(to_float(a[i]) / (1.f + expf(-to_float(g[i]))));
}

// the same, eight bf16 values a thread in 16-byte vectors (n % 8 == 0, 16-byte aligned)
__global__ __launch_bounds__(256) void sigmoid_mul_bf16x8_kernel(bf16_t* __restrict__ a, const bf16_t* __restrict__ g,
                                                                 size_t groups) {
  for (size_t gi = (size_t)blockIdx.x * blockDim.x + threadIdx.x; gi < groups; gi += (size_t)gridDim.x * blockDim.x) {
    const uint4 av = *reinterpret_cast<const uint4*>(a + gi * 8);
    const uint4 gv = *reinterpret_cast<const uint4*>(g + gi * 8);
    const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, gw[4] = {gv.x, gv.y, gv.z, gv.w};
    uint32_t w[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float r0 = bf16_bits_to_float(aw[k] & 0xffffu) / (1.f + expf(-bf16_bits_to_float(gw[k] & 0xffffu)));
      const float r1 = bf16_bits_to_float(aw[k] >> 16) / (1.f + expf(-bf16_bits_to_float(gw[k] >> 16)));
      w[k] = (uint32_t)float_to_bf16_bits(r0) | ((uint32_t)float_to_bf16_bits(r1) << 16);
    }
    *reinterpret_cast<uint4*>(a + gi * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

extern "C" int sa_sigmoid_mul(void* a, const void* g, int act_dtype, long long n, hipStream_t stream) {
  if (n <= 0) return 0;
  if (!a || !g) return SA_ERR_ARG;
  if (act_dtype == SA_BF16 && (n & 7) == 0 && (((uintptr_t)a | (uintptr_t)g) & 15) == 0) {
    long long vb = (n / 8 + 255) / 256;
    if (vb > 65536) vb = 65536;
    hipLaunchKernelGGL(sigmoid_mul_bf16x8_kernel, dim3((unsigned)vb), dim3(256), 0, stream, (bf16_t*)a, (const bf16_t*)g,
                       (size_t)(n / 8));
    SA_LAUNCH_CHECK();
    return 0;
  }
  long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  dim3 grid((unsigned)blocks), block(256);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL(sigmoid_mul_kernel<float>, grid, block, 0, stream, (float*)a, (const float*)g, (size_t)n);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL(sigmoid_mul_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)a, (const bf16_t*)g, (size_t)n);
  else return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
