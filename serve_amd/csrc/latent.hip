// Latent attention: every token keeps one normed latent vector c [R] and one rotated key part
// kr [dr] that all heads share; head h's key is [W_uk_h c | kr] and its value W_uv_h c.
//
// The scores are taken in the latent space:  q_h . (W_uk_h c) = (W_uk_h^T q_h) . c, so the cache row
// [c | kr] is the key of ONE key/value head that all query heads read (queries [W_uk_h^T q_h | rot(qr_h)]),
// the value row is c, and head h's output is W_uv_h (sum_j p_j c_j).  The paged attention kernels then
// run over these rows as they do over any other keys and values; the kernels here make the rows:
//
//   latent_kv_write   c = z[:R] / sqrt(mean(z[:R]^2) + eps) * w,  kr = rot(z[R:], position)  -> pages
//   head_linear       out[t, h, :] = in[t, h, :] W[h]  (W [H, K, N]): the queries into the latent
//                     space, and the latent outputs out of it
//                     (behind a head's outputs it can put the rotated part of the query and the row's padding,
//                     so that the queries are one kernel)
//
// Rotation: dimension i of the rotated part is paired with i + dr/2; (u, v) -> (u cos a - v sin a,
// v cos a + u sin a), a = position * inv_freq[i], in fp32.
#include "common.h"

template <typename TA>
__device__ __forceinline__ void sincos_for(float a, float* sn, float* cs) {
  if (sizeof(TA) == 2) sincos_reduced(a, sn, cs);      // 16-bit storage keeps 8 bits of the result
  else sincosf(a, sn, cs);
}

// ---------------------------------------------------------------------------------------------
// z [T, R + dr] -> k_pages [P, 1, page, Dp] rows [c | kr | 0], v_pages [P, 1, Dp, page] columns [c | 0].
// slot[t] = page * page_size + offset, < 0: nothing stored.  One workgroup a token.
// ---------------------------------------------------------------------------------------------
template <typename TA>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
    const TA* __restrict__ z, const float* __restrict__ w, const int* __restrict__ positions,
    const float* __restrict__ inv_freq, const int* __restrict__ slot, TA* __restrict__ k_pages,
    TA* __restrict__ v_pages, float eps, int R, int dr, int Dp, int page_size, float magnitude) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int s = slot[t];
  if (s < 0) return;                       // (uniform over the workgroup)
  const int page = s / page_size, off = s - page * page_size;
  const TA* zr = z + (size_t)t * (R + dr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = to_float(zr[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rs = 1.f / sqrtf(ss / (float)R + eps);
  TA* kp = k_pages + ((size_t)page * page_size + off) * Dp;
  TA* vp = v_pages + (size_t)page * Dp * page_size + off;
  const float pos = (float)positions[t];
  const int half = dr / 2;
  for (int i = threadIdx.x; i < Dp; i += blockDim.x) {
    float kvv = 0.f, vvv = 0.f;
    if (i < R) {
      kvv = vvv = (to_float(zr[i]) * rs) * w[i];
    } else if (i < R + dr) {
      const int jr = i - R;
      const int jf = jr < half ? jr : jr - half;
      float sn, cs;
      sincos_for<TA>(pos * inv_freq[jf], &sn, &cs);
      const float a = to_float(zr[R + jf]), b = to_float(zr[R + jf + half]);
      kvv = (jr < half ? a * cs - b * sn : b * cs + a * sn) * magnitude;
    }
    kp[i] = from_float<TA>(kvv);
    vp[(size_t)i * page_size] = from_float<TA>(vvv);
  }
}

extern "C" int sa_latent_kv_write(const void* z, int act_dtype, const float* w, const int* positions,
                                  const float* inv_freq, const int* slot, void* k_pages, void* v_pages, float eps,
                                  int T, int R, int dr, int Dp, int page_size, float magnitude, hipStream_t stream) {
  if (T <= 0) return 0;
  if (R <= 0 || dr < 0 || (dr & 1) || Dp < R + dr || page_size <= 0) return SA_ERR_ARG;
  dim3 grid(T), block(Dp > 128 ? 256 : 64);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL(latent_kv_write_kernel<float>, grid, block, 0, stream, (const float*)z, w, positions, inv_freq,
                       slot, (float*)k_pages, (float*)v_pages, eps, R, dr, Dp, page_size, magnitude);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL(latent_kv_write_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)z, w, positions,
                       inv_freq, slot, (bf16_t*)k_pages, (bf16_t*)v_pages, eps, R, dr, Dp, page_size, magnitude);
  else return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t, h, n] = sum_k in[t, h, k] W[h, k, n], fp32 sums.  in: row stride `is`, head stride `ihs`;
// out likewise.  grid (ceil(T / HL_TT), H, ceil(N / 256)): a workgroup takes HL_TT tokens of one head
// so that W[h] is read once per HL_TT tokens; thread = output column (W's rows are contiguous in n).
// ---------------------------------------------------------------------------------------------
#define HL_TT 8
#define HL_KC 128

// What may follow a head's N outputs in its row of `out` (the queries of latent attention): the `rot` inputs that
// lie behind the head's K inputs, rotated by the token's position, then zeros up to `tail` places.
struct HeadTail {
  const int* positions;      // nullptr: no tail
  const float* inv_freq;     // [rot / 2]
  int rot, tail;
  float magnitude;           // multiplies sine and cosine
};

template <typename TA>
__device__ __forceinline__ void write_tail(const HeadTail& ht, const TA* __restrict__ src, TA* __restrict__ dst, int t,
                                           int first, int step) {
  const float pos = (float)ht.positions[t];
  const int half = ht.rot / 2;
  for (int i = first; i < ht.tail; i += step) {
    float v = 0.f;
    if (i < ht.rot) {
      const int jf = i < half ? i : i - half;
      float sn, cs;
      sincos_for<TA>(pos * ht.inv_freq[jf], &sn, &cs);
      const float a = to_float(src[jf]), b = to_float(src[jf + half]);
      v = (i < half ? a * cs - b * sn : b * cs + a * sn) * ht.magnitude;
    }
    dst[i] = from_float<TA>(v);
  }
}

template <typename TA>
__global__ __launch_bounds__(256) void head_linear_kernel(const TA* __restrict__ in, int is, int ihs,
                                                          const TA* __restrict__ W, TA* __restrict__ out, int os,
                                                          int ohs, int T, int K, int N, HeadTail ht) {
  __shared__ float sin_[HL_TT][HL_KC];
  const int t0 = blockIdx.x * HL_TT;
  const int h = blockIdx.y;
  const int n = blockIdx.z * blockDim.x + threadIdx.x;
  const TA* Wh = W + (size_t)h * K * N;
  float acc[HL_TT];
#pragma unroll
  for (int tt = 0; tt < HL_TT; ++tt) acc[tt] = 0.f;
  for (int k0 = 0; k0 < K; k0 += HL_KC) {
    const int kc = min(HL_KC, K - k0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < HL_TT * HL_KC; idx += blockDim.x) {
      const int tt = idx / HL_KC, k = idx - tt * HL_KC;
      sin_[tt][k] = (t0 + tt < T && k < kc) ? to_float(in[(size_t)(t0 + tt) * is + (size_t)h * ihs + k0 + k]) : 0.f;
    }
    __syncthreads();
    if (n < N) {
      for (int k = 0; k < kc; ++k) {
        const float wv = to_float(Wh[(size_t)(k0 + k) * N + n]);
#pragma unroll
        for (int tt = 0; tt < HL_TT; ++tt) acc[tt] += sin_[tt][k] * wv;
      }
    }
  }
  if (n < N) {
#pragma unroll
    for (int tt = 0; tt < HL_TT; ++tt)
      if (t0 + tt < T) out[(size_t)(t0 + tt) * os + (size_t)h * ohs + n] = from_float<TA>(acc[tt]);
  }
  if (ht.positions && blockIdx.z == 0) {
    for (int tt = 0; tt < HL_TT && t0 + tt < T; ++tt)
      write_tail<TA>(ht, in + (size_t)(t0 + tt) * is + (size_t)h * ihs + K,
                     out + (size_t)(t0 + tt) * os + (size_t)h * ohs + N, t0 + tt, threadIdx.x, blockDim.x);
  }
}

// The same for few tokens (single decoded tokens): a workgroup per (token, head), the four waves cut K between
// them and add through LDS in a fixed order, a lane owns an output column and fetches sixteen rows of W at a time,
// so that the whole product is a few trips to memory.  K <= HL_SMALL_K.
#define HL_SMALL_K 1024

template <typename TA>
__global__ __launch_bounds__(256) void head_linear_small_kernel(const TA* __restrict__ in, int is, int ihs,
                                                                const TA* __restrict__ W, TA* __restrict__ out, int os,
                                                                int ohs, int K, int N, HeadTail ht) {
  __shared__ float sx[HL_SMALL_K];
  __shared__ float red[4][64];
  const int t = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const TA* xr = in + (size_t)t * is + (size_t)h * ihs;
  for (int k = threadIdx.x; k < K; k += blockDim.x) sx[k] = to_float(xr[k]);
  if (ht.positions) write_tail<TA>(ht, xr + K, out + (size_t)t * os + (size_t)h * ohs + N, t, threadIdx.x, blockDim.x);
  __syncthreads();
  const TA* Wh = W + (size_t)h * K * N;
  const int per = (K + 3) >> 2;
  const int kb = wave * per, ke = min(K, kb + per);
  for (int n0 = 0; n0 < N; n0 += 64) {
    const int n = min(n0 + lane, N - 1);
    float acc = 0.f;
    for (int k = kb; k < ke; k += 16) {
      float wv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) wv[u] = to_float(Wh[(size_t)min(k + u, ke - 1) * N + n]);
#pragma unroll
      for (int u = 0; u < 16; ++u) acc += (k + u < ke ? sx[min(k + u, HL_SMALL_K - 1)] : 0.f) * wv[u];
    }
    red[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && n0 + lane < N)
      out[(size_t)t * os + (size_t)h * ohs + n0 + lane] =
          from_float<TA>(((red[0][lane] + red[1][lane]) + red[2][lane]) + red[3][lane]);
    __syncthreads();
  }
}

extern "C" int sa_head_linear(const void* in, int is, int ihs, const void* W, void* out, int os, int ohs,
                              int act_dtype, int T, int H, int K, int N, const int* positions, const float* inv_freq,
                              int rot, int tail, float magnitude, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || K <= 0 || N <= 0 || H > 65535 || (N + 255) / 256 > 65535) return SA_ERR_ARG;
  if (positions && ((!inv_freq && rot > 0) || rot < 0 || (rot & 1) || tail < rot)) return SA_ERR_ARG;
  HeadTail ht = {positions, inv_freq, rot, tail, magnitude};
  if (T <= 64 && K <= HL_SMALL_K) {
    dim3 grid(T, H), block(256);
    if (act_dtype == SA_F32)
      hipLaunchKernelGGL(head_linear_small_kernel<float>, grid, block, 0, stream, (const float*)in, is, ihs,
                         (const float*)W, (float*)out, os, ohs, K, N, ht);
    else if (act_dtype == SA_BF16)
      hipLaunchKernelGGL(head_linear_small_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)in, is, ihs,
                         (const bf16_t*)W, (bf16_t*)out, os, ohs, K, N, ht);
    else return SA_ERR_UNSUPPORTED;
    SA_LAUNCH_CHECK();
    return 0;
  }
  const int bx = N >= 256 ? 256 : ((N + 63) / 64) * 64;
  dim3 grid((T + HL_TT - 1) / HL_TT, H, (N + bx - 1) / bx), block(bx);
  if (act_dtype == SA_F32)
    hipLaunchKernelGGL(head_linear_kernel<float>, grid, block, 0, stream, (const float*)in, is, ihs, (const float*)W,
                       (float*)out, os, ohs, T, K, N, ht);
  else if (act_dtype == SA_BF16)
    hipLaunchKernelGGL(head_linear_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)in, is, ihs,
                       (const bf16_t*)W, (bf16_t*)out, os, ohs, T, K, N, ht);
  else return SA_ERR_UNSUPPORTED;
  SA_LAUNCH_CHECK();
  return 0;
}
