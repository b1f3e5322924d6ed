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
// One workgroup a token; a wave takes a head at a time (q heads, then k heads, then v heads).
#include "common.h"

template <typename TA>
__global__ __launch_bounds__(256) void qk_norm_kv_write_kernel(
    const TA* __restrict__ qkv, int row_stride, TA* __restrict__ q_out, const int* __restrict__ positions,
    const int* __restrict__ slot, TA* __restrict__ k_pages, TA* __restrict__ v_pages, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, float temp_coef, int temp_every, const TA* __restrict__ v_first,
    int v_first_stride, float lambda, int Hq, int Hk, int D, int Dv, int Dp, int page_size) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & (SA_WAVE - 1);
  const int wave = threadIdx.x / SA_WAVE;
  const int waves = blockDim.x / SA_WAVE;
  const TA* row = qkv + (size_t)t * row_stride;
  const int s = slot ? slot[t] : -1;
  const int page = s >= 0 ? s / page_size : 0;
  const int off = s >= 0 ? s - page * page_size : 0;
  float temp = 1.f;
  if (temp_every > 0) temp = 1.f + temp_coef * logf((float)((positions[t] + 1) / temp_every) + 1.f);
  const TA zero = from_float<TA>(0.f);

  for (int u = wave; u < Hq + 2 * Hk; u += waves) {
    if (u < Hq + Hk) {
      // a query or a key head: norm over its D dims
      const bool is_q = u < Hq;
      const int g = is_q ? u : u - Hq;
      if (!is_q && s < 0) continue;
      const TA* x = row + (size_t)u * D;
      float ss = 0.f;
      for (int i = lane; i < D; i += SA_WAVE) {
        const float v = to_float(x[i]);
        ss += v * v;
      }
      ss = wave_sum(ss);
      const float rs = 1.0f / sqrtf(ss / (float)D + eps);
      const float* w = is_q ? wq : wk;
      TA* dst = is_q ? q_out + ((size_t)t * Hq + g) * Dp
                     : k_pages + (((size_t)page * Hk + g) * page_size + off) * Dp;
      for (int i = lane; i < Dp; i += SA_WAVE) {
        TA o = zero;
        if (i < D) {
          float v = (to_float(x[i]) * rs) * w[i];
          if (is_q) v *= temp;
          o = from_float<TA>(v);
        }
        dst[i] = o;
      }
    } else {
      if (s < 0) continue;
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
  }
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
  dim3 grid(T), block(256);
#define GO(TA)                                                                                                        \
  hipLaunchKernelGGL(qk_norm_kv_write_kernel<TA>, grid, block, 0, stream, (const TA*)qkv, row_stride, (TA*)q_out,     \
                     positions, slot, (TA*)k_pages, (TA*)v_pages, wq, wk, eps, temp_coef, temp_every,                 \
                     (const TA*)v_first, v_first_stride, lambda, Hq, Hk, D, Dv, Dp, page_size)
  if (act_dtype == SA_F32) GO(float);
  else if (act_dtype == SA_BF16) GO(bf16_t);
  else return SA_ERR_UNSUPPORTED;
#undef GO
  SA_LAUNCH_CHECK();
  return 0;
}
