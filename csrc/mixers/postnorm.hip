// Sublayers with a norm on both sides: the sublayer's output is normed before it joins the residual
// stream, and the input norm of the next sublayer follows in the same pass over the row.
//
//   post_norm_residual   u  = y + y_bias                                      (one branch)
//                        u  = (N0(y) pw1 + N0(y2) pw2) / 2                    (two branches, each normed first)
//                        x <- x + mult * N0(u) * (off + post_w) + extra
//                        n  = N0(x) * (off + next_w)                          N0(v) = v / sqrt(mean(v^2) + eps)
//                      x is the fp32 residual stream, updated in place; y / y2 are activation tensors (float or
//                      bf16, row-strided); extra is fp32 (rows added once, e.g. the embedding rows before a
//                      repeated run of layers). y == nullptr: only extra is added; next_w == nullptr: no n.
//   relu2                max(z + bias, 0)^2
//
// One workgroup per row; the row's running value sits in LDS between the reductions, every thread
// touching only the columns it owns.
#include "mixers_common.h"

namespace xgm {

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void post_norm_residual_kernel(
    float* __restrict__ x, const TY* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias,
    const TY* __restrict__ y2, int64_t ldy2, const float* __restrict__ pw1, const float* __restrict__ pw2,
    const float* __restrict__ post_w, float mult, const float* __restrict__ extra, const float* __restrict__ next_w,
    float off, float eps, TO* __restrict__ out, int W) {
  extern __shared__ float row[];   // [W]
  __shared__ float red[4];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * W;
  const float inv_w = 1.f / (float)W;
  float ssx = 0.f;
  if (y) {
    const TY* yr = y + (int64_t)t * ldy;
    float ssu = 0.f;
    if (y2) {
      const TY* zr = y2 + (int64_t)t * ldy2;
      float s1 = 0.f, s2 = 0.f;
      for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float a = ldf(yr + c), b = ldf(zr + c);
        s1 += a * a;
        s2 += b * b;
      }
      const float ra = 1.f / sqrtf(block_sum(s1, red) * inv_w + eps);
      const float rb = 1.f / sqrtf(block_sum(s2, red) * inv_w + eps);
      for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float u = 0.5f * (ldf(yr + c) * ra * pw1[c] + ldf(zr + c) * rb * pw2[c]);
        row[c] = u;
        ssu += u * u;
      }
    } else {
      for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float u = ldf(yr + c) + (y_bias ? y_bias[c] : 0.f);
        row[c] = u;
        ssu += u * u;
      }
    }
    const float ru = mult / sqrtf(block_sum(ssu, red) * inv_w + eps);
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      float v = xr[c] + row[c] * ru * (off + post_w[c]);
      if (extra) v += extra[(int64_t)t * W + c];
      xr[c] = v;
      row[c] = v;
      ssx += v * v;
    }
  } else {
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      float v = xr[c];
      if (extra) {
        v += extra[(int64_t)t * W + c];
        xr[c] = v;
      }
      row[c] = v;
      ssx += v * v;
    }
  }
  if (!next_w) return;
  const float rx = 1.f / sqrtf(block_sum(ssx, red) * inv_w + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(out + (int64_t)t * W + c, row[c] * rx * (off + next_w[c]));
}

template <typename T>
__global__ void relu2_kernel(const T* __restrict__ z, const float* __restrict__ bias, T* __restrict__ out, int64_t n,
                             int cols) {
  const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i >= n) return;
  if (i + 4 <= n && (cols & 3) == 0) {
    float v[4], b[4] = {0.f, 0.f, 0.f, 0.f};
    ld4(z + i, v);
    if (bias) ld4(bias + (int)(i % cols), b);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float a = fmaxf(v[e] + b[e], 0.f);
      v[e] = a * a;
    }
    st4(out + i, v);
  } else {
    for (int64_t j = i; j < n && j < i + 4; ++j) {
      const float a = fmaxf(ldf(z + j) + (bias ? bias[j % cols] : 0.f), 0.f);
      stf(out + j, a * a);
    }
  }
}

// ================================================================== host launchers
int post_norm_residual(float* x, const void* y, bool y_f32, int64_t ldy, const float* y_bias, const void* y2, int64_t ldy2,
                       const float* pw1, const float* pw2, const float* post_w, float mult, const float* extra,
                       const float* next_w, float off, float eps, void* out, bool out_f32, int T_, int W, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (W < 1 || W > 16000 || (y && !post_w) || (y2 && (!y || !pw1 || !pw2)) || (next_w && !out)) return -1;
  const size_t lds = (size_t)W * sizeof(float);
#define XGM_PN(TY, TO)                                                                                               \
  post_norm_residual_kernel<TY, TO><<<T_, 256, lds, st>>>(x, (const TY*)y, ldy, y_bias, (const TY*)y2, ldy2, pw1, pw2, \
                                                          post_w, mult, extra, next_w, off, eps, (TO*)out, W);
  if (y_f32) {
    if (out_f32) { XGM_PN(float, float) } else { XGM_PN(float, bf16) }
  } else {
    if (out_f32) { XGM_PN(bf16, float) } else { XGM_PN(bf16, bf16) }
  }
#undef XGM_PN
  return 0;
}

void relu2(const void* z, bool f32, const float* bias, void* out, int64_t n, int cols, hipStream_t st) {
  if (n <= 0) return;
  const int64_t threads = (n + 3) / 4;
  XGM_DISPATCH_T(f32, relu2_kernel<T><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>((const T*)z, bias, (T*)out, n,
                                                                                          cols);)
}

}  // namespace xgm
