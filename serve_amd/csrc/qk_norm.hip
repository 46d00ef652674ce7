// What lies between the q/k/v product and the attention of a mixer that norms its queries and keys:
//
//   q[t, h, :] = N(q[t, h, :]) * wq * temp(p_t)       N(y) = y / sqrt(mean(y^2) + eps), per head,
//   k[t, g, :] = N(k[t, g, :]) * wk                    one weight vector for all heads
//   temp(p)    = 1 + coef * ln(floor((p + 1) / every) + 1)   (every <= 0: 1)
//   v[t, g, :] = (1 - lambda) v[t, g, :] + lambda v_first[t, g, :]   (v_first null: v as it is)
//
// then k and v of every token go to its cache slot and q into rows of its own.  Keys and queries have D
// dims, values Dv; the cache and the attention kernels work on one head size Dp >= max(D, Dv) (a multiple
// of 16): the places behind D (in q and k) and behind Dv (in v) are written as zeros, so that scores and
// weighted sums are those of the unpadded heads.  All arithmetic is fp32, the template type is storage.
//
// Input rows are [Hq D | Hk D | Hk Dv] (one product); q_out [T, Hq Dp]; k pages [P, Hk, page_size, Dp],
// v pages [P, Hk, Dp, page_size]; slot[t] = page * page_size + offset, < 0: nothing stored.
//
// Two kernels: the general one (any sizes and alignments: a wave per (token, head), a lane an element at a time),
// and one for sizes that are multiples of 8 from aligned rows, which moves 8 elements a lane (16 bytes of bf16):
// its first blocks take the query and key heads, a group of lanes per head; its last blocks take the values with
// neighbouring lanes on neighbouring tokens, so that the writes into the transposed value pages, where the
// tokens of a page lie side by side, fall into common lines.
#include "common.h"

__device__ __forceinline__ float query_temp(const int* positions, int t, float coef, int every) {
  return every > 0 ? 1.f + coef * logf((float)((positions[t] + 1) / every) + 1.f) : 1.f;
}

template <typename TA>
__global__ __launch_bounds__(256) void qk_norm_kv_write_kernel(
    const TA* __restrict__ qkv, int row_stride, TA* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, TA* __restrict__ k_pages, TA* __restrict__ v_pages, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, float temp_coef, int temp_every, const TA* __restrict__ v_first,
    int v_first_stride, float lambda, int Hq, int Hk, int D, int Dv, int Dp, int page_size) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const int u = blockIdx.y * (blockDim.x / SA_WAVE) + threadIdx.x / SA_WAVE;      // the head this wave takes
  if (u >= Hq + 2 * Hk) return;
  const TA* row = qkv + (size_t)t * row_stride;
  const int s = slot ? slot[t] : -1;
  const int page = s >= 0 ? s / page_size : 0;
  const int off = s >= 0 ? s - page * page_size : 0;
  const TA zero = from_float<TA>(0.f);
  if (u < Hq + Hk) {
    // a query or a key head: norm over its D dims
    const bool is_q = u < Hq;
    const int g = is_q ? u : u - Hq;
    if (!is_q && s < 0) return;
    const TA* x = row + (size_t)u * D;
    float ss = 0.f;
    for (int i = lane; i < D; i += SA_WAVE) {
      const float v = to_float(x[i]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float rs = 1.0f / sqrtf(ss / (float)D + eps);
    const float temp = is_q ? query_temp(positions, t, temp_coef, temp_every) : 1.f;
    const float* w = is_q ? wq : wk;
    TA* dst = is_q ? q_out + ((size_t)t * Hq + g) * Dp : k_pages + (((size_t)page * Hk + g) * page_size + off) * Dp;
    for (int i = lane; i < Dp; i += SA_WAVE) {
      TA o = zero;
      if (i < D) {
        float v = (to_float(x[i]) * rs) * w[i];
        if (is_q) v *= temp;
        o = from_float<TA>(v);
      }
      dst[i] = o;
    }
    return;
  }
  if (s < 0) return;
  const int g = u - Hq - Hk;
  const TA* x = row + (size_t)(Hq + Hk) * D + (size_t)g * Dv;
  const TA* f = v_first ? v_first + (size_t)t * v_first_stride + (size_t)g * Dv : nullptr;
  TA* dst = v_pages + ((size_t)page * Hk + g) * (size_t)Dp * page_size + off;
  for (int i = lane; i < Dp; i += SA_WAVE) {
    TA o = zero;
    if (i < Dv) {
      float v = to_float(x[i]);
      if (f) v = (1.f - lambda) * v + lambda * to_float(f[i]);
      o = from_float<TA>(v);
    }
    dst[(size_t)i * page_size] = o;
  }
}

// eight consecutive elements from an address that is aligned for them
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    v[2 * k] = bf16_bits_to_float(w[k] & 0xffffu);
    v[2 * k + 1] = bf16_bits_to_float(w[k] >> 16);
  }
}
__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float (&v)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
    w[k] = (uint32_t)float_to_bf16_bits(v[2 * k]) | ((uint32_t)float_to_bf16_bits(v[2 * k + 1]) << 16);
  *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}

// D, Dv, Dp, the row strides multiples of 8, 16-byte aligned bases.  LPH lanes a head (a power of two, 8 LPH >= Dp).
// Blocks 0 .. qk_blocks - 1: the (token, query or key head) pairs, 256 / LPH a block.  The blocks behind them: the
// values, a thread per (token, key/value head, 8 dims), tokens fastest.
template <typename TA, int LPH>
__global__ __launch_bounds__(256) void qk_norm_kv_write_vec_kernel(
    const TA* __restrict__ qkv, int row_stride, TA* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, TA* __restrict__ k_pages, TA* __restrict__ v_pages, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, float temp_coef, int temp_every, const TA* __restrict__ v_first,
    int v_first_stride, float lambda, int T, int Hq, int Hk, int D, int Dv, int Dp, int page_size, int qk_blocks) {
  if ((int)blockIdx.x < qk_blocks) {
    const int sub = threadIdx.x % LPH;
    const long long unit = (long long)blockIdx.x * (256 / LPH) + threadIdx.x / LPH;
    const bool live = unit < (long long)T * (Hq + Hk);
    const long long uc = live ? unit : 0;
    const int t = (int)(uc / (Hq + Hk)), u = (int)(uc - (long long)t * (Hq + Hk));
    const bool is_q = u < Hq;
    const int i = sub * 8;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live && i < D) load8(qkv + (size_t)t * row_stride + (size_t)u * D + i, v);
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) ss += v[k] * v[k];
#pragma unroll
    for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, SA_WAVE);
    if (!live || i >= Dp) return;
    const float rs = 1.0f / sqrtf(ss / (float)D + eps);
    const float temp = is_q ? query_temp(positions, t, temp_coef, temp_every) : 1.f;
    if (i < D) {
      float w[8];
      load8((is_q ? wq : wk) + i, w);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        v[k] = (v[k] * rs) * w[k];
        if (is_q) v[k] *= temp;
      }
    }
    if (is_q) {
      store8(q_out + ((size_t)t * Hq + u) * Dp + i, v);
    } else {
      const int s = slot ? slot[t] : -1;
      if (s < 0) return;
      const int page = s / page_size, off = s - page * page_size;
      store8(k_pages + (((size_t)page * Hk + (u - Hq)) * page_size + off) * Dp + i, v);
    }
    return;
  }
  if (!slot) return;
  const int chunks = Dp >> 3;
  const long long idx = (long long)(blockIdx.x - qk_blocks) * 256 + threadIdx.x;
  if (idx >= (long long)T * Hk * chunks) return;
  const int t = (int)(idx % T);
  const int gc = (int)(idx / T);
  const int g = gc / chunks, i = (gc - g * chunks) * 8;
  const int s = slot[t];
  if (s < 0) return;
  const int page = s / page_size, off = s - page * page_size;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (i < Dv) {
    load8(qkv + (size_t)t * row_stride + (size_t)(Hq + Hk) * D + (size_t)g * Dv + i, v);
    if (v_first) {
      float f[8];
      load8(v_first + (size_t)t * v_first_stride + (size_t)g * Dv + i, f);
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = (1.f - lambda) * v[k] + lambda * f[k];
    }
  }
  TA* dst = v_pages + (((size_t)page * Hk + g) * Dp + i) * page_size + off;
#pragma unroll
  for (int k = 0; k < 8; ++k) dst[(size_t)k * page_size] = from_float<TA>(v[k]);
}

template <typename TA>
static int launch_qk_norm(const void* qkv, int row_stride, void* q_out, const int* positions, const int* slot,
                          void* k_pages, void* v_pages, const float* wq, const float* wk, float eps, float temp_coef,
                          int temp_every, const void* v_first, int v_first_stride, float lambda, int T, int Hq, int Hk,
                          int D, int Dv, int Dp, int page_size, hipStream_t stream) {
  const uintptr_t bits = (uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages |
                         (uintptr_t)v_first | (uintptr_t)wq | (uintptr_t)wk;
  const bool vec = ((D | Dv | Dp | row_stride | v_first_stride) & 7) == 0 && (bits & 15) == 0 && Dp <= 512;
  if (vec) {
    int lph = 2;
    while (lph * 8 < Dp) lph *= 2;
    const long long units = (long long)T * (Hq + Hk), per = 256 / lph;
    const long long qk_blocks = (units + per - 1) / per;
    const long long v_blocks = slot ? ((long long)T * Hk * (Dp >> 3) + 255) / 256 : 0;
    if (qk_blocks + v_blocks > 0x7fffffffLL) return SA_ERR_ARG;
    dim3 grid((unsigned)(qk_blocks + v_blocks)), block(256);
#define GOV(LPH)                                                                                                      \
  hipLaunchKernelGGL((qk_norm_kv_write_vec_kernel<TA, LPH>), grid, block, 0, stream, (const TA*)qkv, row_stride,       \
                     (TA*)q_out, positions, slot, (TA*)k_pages, (TA*)v_pages, wq, wk, eps, temp_coef, temp_every,     \
                     (const TA*)v_first, v_first_stride, lambda, T, Hq, Hk, D, Dv, Dp, page_size, (int)qk_blocks)
    switch (lph) {
      case 2: GOV(2); break;
      case 4: GOV(4); break;
      case 8: GOV(8); break;
      case 16: GOV(16); break;
      case 32: GOV(32); break;
      default: GOV(64); break;
    }
#undef GOV
    return 0;
  }
  const int units = Hq + 2 * Hk;
  if ((units + 3) / 4 > 65535) return SA_ERR_ARG;
  dim3 grid(T, (units + 3) / 4), block(256);
  hipLaunchKernelGGL(qk_norm_kv_write_kernel<TA>, grid, block, 0, stream, (const TA*)qkv, row_stride, (TA*)q_out,
                     positions, slot, (TA*)k_pages, (TA*)v_pages, wq, wk, eps, temp_coef, temp_every,
                     (const TA*)v_first, v_first_stride, lambda, Hq, Hk, D, Dv, Dp, page_size);
  return 0;
}

extern "C" int sa_qk_norm_kv_write(const void* qkv, int row_stride, void* q_out, int act_dtype, const int* positions,
                                   const int* slot, void* k_pages, void* v_pages, const float* wq, const float* wk,
                                   float eps, float temp_coef, int temp_every, const void* v_first, int v_first_stride,
                                   float lambda, int T, int Hq, int Hk, int D, int Dv, int Dp, int page_size,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || D <= 0 || Dv <= 0 || Dp < D || Dp < Dv || page_size <= 0 || !wq || !wk || !q_out)
    return SA_ERR_ARG;
  if (row_stride < Hq * D + Hk * (D + Dv) || (slot && (!k_pages || !v_pages)) || (temp_every > 0 && !positions))
    return SA_ERR_ARG;
  int rc;
  if (act_dtype == SA_F32)
    rc = launch_qk_norm<float>(qkv, row_stride, q_out, positions, slot, k_pages, v_pages, wq, wk, eps, temp_coef,
                               temp_every, v_first, v_first_stride, lambda, T, Hq, Hk, D, Dv, Dp, page_size, stream);
  else if (act_dtype == SA_BF16)
    rc = launch_qk_norm<bf16_t>(qkv, row_stride, q_out, positions, slot, k_pages, v_pages, wq, wk, eps, temp_coef,
                                temp_every, v_first, v_first_stride, lambda, T, Hq, Hk, D, Dv, Dp, page_size, stream);
  else
    return SA_ERR_UNSUPPORTED;
  if (rc != 0) return rc;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The same place in a mixer whose queries and keys are normed over the whole projection and then rotated:
//
//   q[t, :] = N(q[t, :]) * wq   over all Hq D values of the token at once (wq fp32 [Hq D]);  k likewise (wk fp32 [Hk D])
//   then in every head the first `rot` dims are rotated by the position: dim i pairs with i + rot/2,
//   (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * freq[i]
//
// Input rows [Hq D | Hk D | Hk Dv | ...]; outputs as above: q_out [T, Hq Dp], keys and values into the token's slot,
// every head padded with zeros up to Dp.  Blocks 0 .. T-1 take a token's queries and keys (two sums over the block,
// then an element a thread at a time); the blocks behind them take the values, a thread per (token, kv head, dim)
// with tokens fastest, so that writes into the transposed value pages fall into common lines.
// EXACT: sincosf of the float32 path; else the reduced-argument hardware sine and cosine.
// ---------------------------------------------------------------------------------------------
template <typename TA, bool EXACT>
__global__ __launch_bounds__(1024) void row_norm_rope_kv_write_kernel(
    const TA* __restrict__ qkv, long long row_stride, TA* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, TA* __restrict__ k_pages, TA* __restrict__ v_pages, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ freq, int rot, int T, int Hq, int Hk, int D,
    int Dv, int Dp, int page_size) {
  __shared__ float scratch[16];
  const TA zero = from_float<TA>(0.f);
  if ((int)blockIdx.x < T) {
    const int t = blockIdx.x;
    const TA* row = qkv + (size_t)t * row_stride;
    const int nq = Hq * D, nk = Hk * D;
    float sq = 0.f, sk = 0.f;
    for (int e = threadIdx.x; e < nq; e += blockDim.x) {
      const float v = to_float(row[e]);
      sq = fmaf(v, v, sq);
    }
    for (int e = threadIdx.x; e < nk; e += blockDim.x) {
      const float v = to_float(row[nq + e]);
      sk = fmaf(v, v, sk);
    }
    sq = block_sum(sq, scratch);
    sk = block_sum(sk, scratch);
    const float rq = 1.0f / sqrtf(sq / (float)nq + eps), rk = 1.0f / sqrtf(sk / (float)nk + eps);
    const float pos = (float)positions[t];
    const int s = slot ? slot[t] : -1;
    const int page = s >= 0 ? s / page_size : 0, off = s >= 0 ? s - page * page_size : 0;
    const int half = rot >> 1;
    const int total = (Hq + (s >= 0 ? Hk : 0)) * Dp;
    for (int idx = threadIdx.x; idx < total; idx += blockDim.x) {
      const int u = idx / Dp, i = idx - u * Dp;
      const bool is_q = u < Hq;
      const int g = is_q ? u : u - Hq;
      TA* dst = is_q ? q_out + ((size_t)t * Hq + g) * Dp : k_pages + (((size_t)page * Hk + g) * page_size + off) * Dp;
      TA out = zero;
      if (i < D) {
        const TA* x = row + (is_q ? 0 : nq) + (size_t)g * D;
        const float* w = (is_q ? wq : wk) + (size_t)g * D;
        const float rs = is_q ? rq : rk;
        float val = (to_float(x[i]) * rs) * w[i];
        if (i < rot) {
          const int j = i < half ? i : i - half;
          const int ip = i < half ? i + half : i - half;
          const float other = (to_float(x[ip]) * rs) * w[ip];
          const float a = pos * freq[j];
          float sn, cs;
          if (EXACT) sincosf(a, &sn, &cs);
          else sincos_reduced(a, &sn, &cs);
          val = i < half ? val * cs - other * sn : val * cs + other * sn;
        }
        out = from_float<TA>(val);
      }
      dst[i] = out;
    }
    return;
  }
  if (!slot) return;
  const long long idx = (long long)(blockIdx.x - T) * blockDim.x + threadIdx.x;
  if (idx >= (long long)T * Hk * Dp) return;
  const int t = (int)(idx % T);
  const int gi = (int)(idx / T);
  const int g = gi / Dp, i = gi - g * Dp;
  const int s = slot[t];
  if (s < 0) return;
  const int page = s / page_size, off = s - page * page_size;
  TA out = zero;
  if (i < Dv) out = qkv[(size_t)t * row_stride + (size_t)(Hq + Hk) * D + (size_t)g * Dv + i];
  v_pages[(((size_t)page * Hk + g) * Dp + i) * page_size + off] = out;
}

extern "C" int sa_row_norm_rope_kv_write(const void* qkv, long long row_stride, void* q_out, int act_dtype,
                                         const int* positions, const int* slot, void* k_pages, void* v_pages,
                                         const float* wq, const float* wk, float eps, const float* freq, int rot, int T,
                                         int Hq, int Hk, int D, int Dv, int Dp, int page_size, hipStream_t stream) {
  if (T <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || D <= 0 || Dv <= 0 || Dp < D || Dp < Dv || page_size <= 0 || !wq || !wk || !q_out || !positions)
    return SA_ERR_ARG;
  if (row_stride < (long long)Hq * D + (long long)Hk * (D + Dv) || (slot && (!k_pages || !v_pages)) || rot < 0 || rot % 2 ||
      rot > D || (rot > 0 && !freq))
    return SA_ERR_ARG;
  // a step of few tokens takes workgroups of 1024: a token's row is then two or three values a thread
  const int threads = T <= 64 ? 1024 : 256;
  const long long v_blocks = slot ? ((long long)T * Hk * Dp + threads - 1) / threads : 0;
  if ((long long)T + v_blocks > 0x7fffffffLL) return SA_ERR_ARG;
  dim3 grid((unsigned)(T + v_blocks)), block(threads);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL((row_norm_rope_kv_write_kernel<float, true>), grid, block, 0, stream, (const float*)qkv, row_stride,
                       (float*)q_out, positions, slot, (float*)k_pages, (float*)v_pages, wq, wk, eps, freq, rot, T, Hq, Hk,
                       D, Dv, Dp, page_size);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL((row_norm_rope_kv_write_kernel<bf16_t, false>), grid, block, 0, stream, (const bf16_t*)qkv,
                       row_stride, (bf16_t*)q_out, positions, slot, (bf16_t*)k_pages, (bf16_t*)v_pages, wq, wk, eps, freq,
                       rot, T, Hq, Hk, D, Dv, Dp, page_size);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// An output gate per head: a[t, h, :] *= sigmoid(g[t, h]), a [T, H Dp] in place; g: rows of g_stride elements, the
// heads' logits from column g_col on.
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void head_gate_kernel(TA* __restrict__ a, const TA* __restrict__ g, long long g_stride,
                                                        int g_col, long long total, int H, int Dp) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const long long th = idx / Dp;
  const long long t = th / H;
  const int h = (int)(th - t * H);
  const float z = to_float(g[(size_t)t * g_stride + g_col + h]);
  a[idx] = from_float<TA>(to_float(a[idx]) * (1.f / (1.f + expf(-z))));
}

extern "C" int sa_head_gate(void* a, const void* g, int dtype, long long g_stride, int g_col, int T, int H, int Dp,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (!a || !g || H <= 0 || Dp <= 0 || g_col < 0) return SA_ERR_ARG;
  const long long total = (long long)T * H * Dp;
  const long long blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return SA_ERR_ARG;
  if (dtype == SA_F32)
    hipLaunchKernelGGL(head_gate_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream, (float*)a, (const float*)g,
                       g_stride, g_col, total, H, Dp);
  else if (dtype == SA_BF16)
    hipLaunchKernelGGL(head_gate_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, (bf16_t*)a, (const bf16_t*)g,
                       g_stride, g_col, total, H, Dp);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Biases, a rotation of part of every head with a magnitude, and the cache write with padding, for an attention
// without norms on its queries and keys.  Rows qkv [T, Hq D | Hk D | Hk Dv] (row_stride elements apart):
//   value = qkv + bias (bias fp32 over the whole row, may be null)
//   the first `rot` dims of every query and key head turn by position * freq[j]; pair j is (j, j + rot / 2), or
//   (2j, 2j + 1) with `adjacent`; sine and cosine are multiplied by `magnitude`
// Queries go to q_out [T, Hq Dp], keys to k_pages [P, Hk, page, Dp], values to v_pages [P, Hk, Dp, page], each head
// padded with zeros up to Dp.  slot null: queries only; slot[t] < 0: nothing of token t is stored.
// Queries and keys: a thread an element of the padded output, the first element of a pair computes and writes both.
// Values: the last blocks of the grid, neighbouring lanes on neighbouring tokens (the tokens of a page lie side by
// side in the transposed value pages).
// ---------------------------------------------------------------------------------------------
template <typename TA, bool EXACT>
__global__ __launch_bounds__(256) void bias_rope_kv_write_kernel(
    const TA* __restrict__ qkv, long long row_stride, TA* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, TA* __restrict__ k_pages, TA* __restrict__ v_pages, const float* __restrict__ bias,
    const float* __restrict__ freq, int rot, int adjacent, float magnitude, int T, int Hq, int Hk, int D, int Dv, int Dp,
    int page_size, long long qk_blocks) {
  const TA zero = from_float<TA>(0.f);
  const int units = Hq + (slot ? Hk : 0);
  if ((long long)blockIdx.x < qk_blocks) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long long)T * units * Dp) return;
    const int i = (int)(idx % Dp);
    const long long tu = idx / Dp;
    const int u = (int)(tu % units), t = (int)(tu / units);
    const bool is_q = u < Hq;
    const int g = is_q ? u : u - Hq;
    TA* dst;
    if (is_q) {
      dst = q_out + ((size_t)t * Hq + g) * Dp;
    } else {
      const int s = slot[t];
      if (s < 0) return;
      const int page = s / page_size, off = s - page * page_size;
      dst = k_pages + (((size_t)page * Hk + g) * page_size + off) * Dp;
    }
    if (i >= D) {
      dst[i] = zero;
      return;
    }
    const size_t col = (is_q ? 0 : (size_t)Hq * D) + (size_t)g * D;
    const TA* x = qkv + (size_t)t * row_stride + col;
    const float* b = bias ? bias + col : nullptr;
    if (i >= rot) {
      dst[i] = from_float<TA>(to_float(x[i]) + (b ? b[i] : 0.f));
      return;
    }
    const int half = rot >> 1;
    const bool first = adjacent ? (i & 1) == 0 : i < half;
    if (!first) return;                              // (its partner writes both)
    const int ip = adjacent ? i + 1 : i + half;
    const int j = adjacent ? i >> 1 : i;
    const float a = (float)positions[t] * freq[j];
    float sn, cs;
    if (EXACT) sincosf(a, &sn, &cs);
    else sincos_reduced(a, &sn, &cs);
    sn *= magnitude;
    cs *= magnitude;
    const float p0 = to_float(x[i]) + (b ? b[i] : 0.f), p1 = to_float(x[ip]) + (b ? b[ip] : 0.f);
    dst[i] = from_float<TA>(p0 * cs - p1 * sn);
    dst[ip] = from_float<TA>(p1 * cs + p0 * sn);
    return;
  }
  if (!slot) return;
  const long long idx = ((long long)blockIdx.x - qk_blocks) * blockDim.x + threadIdx.x;
  if (idx >= (long long)T * Hk * Dp) return;
  const int t = (int)(idx % T);
  const int gi = (int)(idx / T);
  const int g = gi / Dp, i = gi - g * Dp;
  const int s = slot[t];
  if (s < 0) return;
  const int page = s / page_size, off = s - page * page_size;
  TA out = zero;
  if (i < Dv) {
    const size_t col = (size_t)(Hq + Hk) * D + (size_t)g * Dv + i;
    out = from_float<TA>(to_float(qkv[(size_t)t * row_stride + col]) + (bias ? bias[col] : 0.f));
  }
  v_pages[(((size_t)page * Hk + g) * Dp + i) * page_size + off] = out;
}

// The same for bf16 with pairs (j, j + rot / 2), rot % 16 == 0 and D, Dv, Dp and the row stride multiples of 8, from
// 16-byte aligned arrays: 16-byte vectors, `tpb` (1, 2, 4 or 8) consecutive tokens a block.  A thread takes eight dims of
// one head of one token: eight pairs (two loads, two stores) in the rotated part's first half, a plain copy behind the
// rotated part, zeros in the padding.  The values go through LDS: read as rows of tokens, written so that neighbouring
// lanes hold neighbouring tokens of one dim, which in the transposed page are neighbouring addresses when the tokens'
// slots are (a prompt portion's are).
__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    f[2 * k] = bf16_bits_to_float(w[k] & 0xffffu);
    f[2 * k + 1] = bf16_bits_to_float(w[k] >> 16);
  }
}

__device__ __forceinline__ uint4 pack8(const float* f) {
  uint32_t w[4];
#pragma unroll
  for (int k = 0; k < 4; ++k)
    w[k] = (uint32_t)float_to_bf16_bits(f[2 * k]) | ((uint32_t)float_to_bf16_bits(f[2 * k + 1]) << 16);
  return make_uint4(w[0], w[1], w[2], w[3]);
}

__device__ __forceinline__ void add8(float* f, const float* __restrict__ b) {
  if (!b) return;
  const float4 b0 = *reinterpret_cast<const float4*>(b), b1 = *reinterpret_cast<const float4*>(b + 4);
  f[0] += b0.x; f[1] += b0.y; f[2] += b0.z; f[3] += b0.w;
  f[4] += b1.x; f[5] += b1.y; f[6] += b1.z; f[7] += b1.w;
}

__global__ __launch_bounds__(1024) void bias_rope_kv_write_vec_kernel(
    const bf16_t* __restrict__ qkv, long long row_stride, bf16_t* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages,
    const float* __restrict__ bias, const float* __restrict__ freq, int rot, float magnitude, int T, int Hq, int Hk, int D,
    int Dv, int Dp, int page_size, int tpb) {
  extern __shared__ __attribute__((aligned(16))) unsigned char brk_lds[];
  const int t0 = blockIdx.x * tpb;
  const int nt = min(tpb, T - t0);
  const int half = rot >> 1;
  const int cph = Dp >> 3;                                   // chunks of eight dims a head
  const int units = Hq + (slot ? Hk : 0);
  const int per_token = units * cph;
  const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
  for (int idx = threadIdx.x; idx < nt * per_token; idx += blockDim.x) {
    const int i = idx / per_token;
    const int rem = idx - i * per_token;
    const int u = rem / cph;
    const int j0 = (rem - u * cph) * 8;
    if (j0 >= half && j0 < rot) continue;                    // (the second halves of the pairs: their partners write them)
    const int t = t0 + i;
    const bool is_q = u < Hq;
    const int g = is_q ? u : u - Hq;
    bf16_t* dst;
    if (is_q) {
      dst = q_out + ((size_t)t * Hq + g) * Dp;
    } else {
      const int s = slot[t];
      if (s < 0) continue;
      const int page = s / page_size;
      dst = k_pages + (((size_t)page * Hk + g) * page_size + (s - page * page_size)) * Dp;
    }
    if (j0 >= D) {
      *reinterpret_cast<uint4*>(dst + j0) = zero;
      continue;
    }
    const size_t col = (is_q ? 0 : (size_t)Hq * D) + (size_t)g * D;
    const bf16_t* x = qkv + (size_t)t * row_stride + col;
    const float* b = bias ? bias + col : nullptr;
    float lo[8];
    unpack8(*reinterpret_cast<const uint4*>(x + j0), lo);
    add8(lo, b ? b + j0 : nullptr);
    if (j0 >= rot) {
      *reinterpret_cast<uint4*>(dst + j0) = pack8(lo);
      continue;
    }
    float hi[8];
    unpack8(*reinterpret_cast<const uint4*>(x + half + j0), hi);
    add8(hi, b ? b + half + j0 : nullptr);
    const float pos = (float)positions[t];
    const float4 f0 = *reinterpret_cast<const float4*>(freq + j0), f1 = *reinterpret_cast<const float4*>(freq + j0 + 4);
    const float fr[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
    float o0[8], o1[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float sn, cs;
      sincos_reduced(pos * fr[k], &sn, &cs);
      sn *= magnitude;
      cs *= magnitude;
      o0[k] = lo[k] * cs - hi[k] * sn;
      o1[k] = hi[k] * cs + lo[k] * sn;
    }
    *reinterpret_cast<uint4*>(dst + j0) = pack8(o0);
    *reinterpret_cast<uint4*>(dst + half + j0) = pack8(o1);
  }
  if (!slot) return;
  // values (with their bias): rows of tokens into LDS (16 bytes of padding a row spread the tokens over the banks) ...
  const int HD = Hk * Dv;
  const int stride = HD + 8;                                  // elements
  uint16_t* tile = reinterpret_cast<uint16_t*>(brk_lds);
  const int vecs = HD >> 3;
  const size_t vcol = (size_t)(Hq + Hk) * D;
  for (int idx = threadIdx.x; idx < nt * vecs; idx += blockDim.x) {
    const int i = idx / vecs;
    const int e0 = (idx - i * vecs) * 8;
    uint4 v = *reinterpret_cast<const uint4*>(qkv + (size_t)(t0 + i) * row_stride + vcol + e0);
    if (bias) {
      float f[8];
      unpack8(v, f);
      add8(f, bias + vcol + e0);
      v = pack8(f);
    }
    *reinterpret_cast<uint4*>(tile + i * stride + e0) = v;
  }
  __syncthreads();
  // ... and out again with the token as the fastest index, every head padded with zeros up to Dp
  const int i = threadIdx.x & (tpb - 1);
  const int s = i < nt ? slot[t0 + i] : -1;
  if (s < 0) return;
  const int page = s / page_size;
  bf16_t* vp = v_pages + (size_t)page * Hk * Dp * page_size + (s - page * page_size);
  for (int e = threadIdx.x / tpb; e < Hk * Dp; e += blockDim.x / tpb) {
    const int g = e / Dp, d = e - g * Dp;
    vp[(size_t)e * page_size].v = d < Dv ? tile[i * stride + g * Dv + d] : (uint16_t)0;
  }
}

extern "C" int sa_bias_rope_kv_write(const void* qkv, long long row_stride, void* q_out, int act_dtype,
                                     const int* positions, const int* slot, void* k_pages, void* v_pages,
                                     const float* bias, const float* freq, int rot, int adjacent, float magnitude, int T,
                                     int Hq, int Hk, int D, int Dv, int Dp, int page_size, hipStream_t stream) {
  if (T <= 0) return 0;
  if (Hq <= 0 || Hk <= 0 || D <= 0 || Dv <= 0 || Dp < D || Dp < Dv || page_size <= 0 || !q_out || !positions || !qkv)
    return SA_ERR_ARG;
  if (row_stride < (long long)Hq * D + (long long)Hk * (D + Dv) || (slot && (!k_pages || !v_pages)) || rot < 0 || rot % 2 ||
      rot > D || (rot > 0 && !freq))
    return SA_ERR_ARG;
  int tpb = T >= 1024 ? 8 : (T >= 512 ? 4 : (T >= 256 ? 2 : 1));
  while (tpb > 1 && (size_t)tpb * ((size_t)Hk * Dv + 8) * 2 > 65536) tpb >>= 1;   // the values' tile has to fit LDS
  const size_t tile_bytes = (size_t)tpb * ((size_t)Hk * Dv + 8) * 2;
  const bool aligned = !(((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages | (uintptr_t)bias |
                          (uintptr_t)freq) & 15);
  if (act_dtype == SA_BF16 && !adjacent && (rot & 15) == 0 && !((D | Dv | Dp) & 7) && !(row_stride & 7) && aligned &&
      tile_bytes <= 65536) {
    const long long items = (long long)tpb * (Hq + (slot ? Hk : 0)) * (Dp >> 3);
    const int vthreads = (int)(items >= 1024 ? 1024 : (items <= 256 ? 256 : (items + 63) / 64 * 64));
    hipLaunchKernelGGL(bias_rope_kv_write_vec_kernel, dim3((T + tpb - 1) / tpb), dim3(vthreads), slot ? tile_bytes : 0,
                       stream, (const bf16_t*)qkv, row_stride, (bf16_t*)q_out, positions, slot, (bf16_t*)k_pages,
                       (bf16_t*)v_pages, bias, freq, rot, magnitude, T, Hq, Hk, D, Dv, Dp, page_size, tpb);
    SA_LAUNCH_CHECK();
    return 0;
  }
  const int threads = 256;
  const long long qk_blocks = ((long long)T * (Hq + (slot ? Hk : 0)) * Dp + threads - 1) / threads;
  const long long v_blocks = slot ? ((long long)T * Hk * Dp + threads - 1) / threads : 0;
  if (qk_blocks + v_blocks > 0x7fffffffLL) return SA_ERR_ARG;
  dim3 grid((unsigned)(qk_blocks + v_blocks)), block(threads);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL((bias_rope_kv_write_kernel<float, true>), grid, block, 0, stream, (const float*)qkv, row_stride,
                       (float*)q_out, positions, slot, (float*)k_pages, (float*)v_pages, bias, freq, rot, adjacent,
                       magnitude, T, Hq, Hk, D, Dv, Dp, page_size, qk_blocks);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL((bias_rope_kv_write_kernel<bf16_t, false>), grid, block, 0, stream, (const bf16_t*)qkv,
                       row_stride, (bf16_t*)q_out, positions, slot, (bf16_t*)k_pages, (bf16_t*)v_pages, bias, freq, rot,
                       adjacent, magnitude, T, Hq, Hk, D, Dv, Dp, page_size, qk_blocks);
  else
    return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
