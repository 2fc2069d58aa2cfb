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

// The same, for rows of up to 1024 * NV aligned columns: thread t owns columns 4 (t + 256 j) .. + 3, j < NV, in
// registers; every global load of the row is issued before the first reduction.
template <typename TY, typename TO, int NV>
__global__ __launch_bounds__(256) void post_norm_residual_vec_kernel(
    float* __restrict__ x, const TY* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias,
    const TY* __restrict__ y2, int64_t ldy2, const float* __restrict__ pw1, const float* __restrict__ pw2,
    const float* __restrict__ post_w, float mult, const float* __restrict__ extra, const float* __restrict__ next_w,
    float off, float eps, TO* __restrict__ out, int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * W;
  const float inv_w = 1.f / (float)W;
  float xv[NV][4], u[NV][4], e[NV][4];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = 4 * (threadIdx.x + 256 * j);
#pragma unroll
    for (int i = 0; i < 4; ++i) xv[j][i] = u[j][i] = e[j][i] = 0.f;
    if (c < W) {
      ld4(xr + c, xv[j]);
      if (y) ld4(y + (int64_t)t * ldy + c, u[j]);
      if (extra) ld4(extra + (int64_t)t * W + c, e[j]);
    }
  }
  float ssx = 0.f;
  if (y) {
    float ssu = 0.f;
    if (y2) {
      float b[NV][4], s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = 4 * (threadIdx.x + 256 * j);
#pragma unroll
        for (int i = 0; i < 4; ++i) b[j][i] = 0.f;
        if (c < W) ld4(y2 + (int64_t)t * ldy2 + c, b[j]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s1 += u[j][i] * u[j][i];
          s2 += b[j][i] * b[j][i];
        }
      }
      const float ra = 1.f / sqrtf(block_sum(s1, red) * inv_w + eps);
      const float rb = 1.f / sqrtf(block_sum(s2, red) * inv_w + eps);
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = 4 * (threadIdx.x + 256 * j);
        if (c < W) {
          float w1[4], w2[4];
          ld4(pw1 + c, w1);
          ld4(pw2 + c, w2);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            u[j][i] = 0.5f * (u[j][i] * ra * w1[i] + b[j][i] * rb * w2[i]);
            ssu += u[j][i] * u[j][i];
          }
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int c = 4 * (threadIdx.x + 256 * j);
        if (c < W) {
          float bb[4] = {0.f, 0.f, 0.f, 0.f};
          if (y_bias) ld4(y_bias + c, bb);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            u[j][i] += bb[i];
            ssu += u[j][i] * u[j][i];
          }
        }
      }
    }
    const float ru = mult / sqrtf(block_sum(ssu, red) * inv_w + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = 4 * (threadIdx.x + 256 * j);
      if (c < W) {
        float pw[4];
        ld4(post_w + c, pw);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          xv[j][i] = xv[j][i] + u[j][i] * ru * (off + pw[i]) + e[j][i];
          ssx += xv[j][i] * xv[j][i];
        }
        st4(xr + c, xv[j]);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int c = 4 * (threadIdx.x + 256 * j);
      if (c < W) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          xv[j][i] += e[j][i];
          ssx += xv[j][i] * xv[j][i];
        }
        if (extra) st4(xr + c, xv[j]);
      }
    }
  }
  if (!next_w) return;
  const float rx = 1.f / sqrtf(block_sum(ssx, red) * inv_w + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = 4 * (threadIdx.x + 256 * j);
    if (c < W) {
      float nw[4];
      ld4(next_w + c, nw);
#pragma unroll
      for (int i = 0; i < 4; ++i) nw[i] = xv[j][i] * rx * (off + nw[i]);
      st4(out + (int64_t)t * W + c, nw);
    }
  }
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
  // rows of aligned groups of four columns (16-byte fp32 / 8-byte bf16 accesses) go through the register form
  const int ysz = y_f32 ? 4 : 2;
  const bool vec = (W & 3) == 0 && W <= 8192 && (!y || ((ldy & 3) == 0 && (uintptr_t)y % (4 * ysz) == 0)) &&
                   (!y2 || ((ldy2 & 3) == 0 && (uintptr_t)y2 % (4 * ysz) == 0));
#define XGM_PV(TY, TO, NV)                                                                                            \
  post_norm_residual_vec_kernel<TY, TO, NV><<<T_, 256, 0, st>>>(x, (const TY*)y, ldy, y_bias, (const TY*)y2, ldy2, pw1,  \
                                                                pw2, post_w, mult, extra, next_w, off, eps, (TO*)out, W);
#define XGM_PN(TY, TO)                                                                                                \
  if (vec && W <= 2048) {                                                                                             \
    XGM_PV(TY, TO, 2)                                                                                                 \
  } else if (vec && W <= 4096) {                                                                                      \
    XGM_PV(TY, TO, 4)                                                                                                 \
  } else if (vec) {                                                                                                   \
    XGM_PV(TY, TO, 8)                                                                                                 \
  } else {                                                                                                            \
    post_norm_residual_kernel<TY, TO><<<T_, 256, lds, st>>>(x, (const TY*)y, ldy, y_bias, (const TY*)y2, ldy2, pw1,    \
                                                            pw2, post_w, mult, extra, next_w, off, eps, (TO*)out, W);  \
  }
  if (y_f32) {
    if (out_f32) { XGM_PN(float, float) } else { XGM_PN(float, bf16) }
  } else {
    if (out_f32) { XGM_PN(bf16, float) } else { XGM_PN(bf16, bf16) }
  }
#undef XGM_PN
#undef XGM_PV
  return 0;
}

void relu2(const void* z, bool f32, const float* bias, void* out, int64_t n, int cols, hipStream_t st) {
  if (n <= 0) return;
  const int64_t threads = (n + 3) / 4;
  XGM_DISPATCH_T(f32, relu2_kernel<T><<<(unsigned)((threads + 255) / 256), 256, 0, st>>>((const T*)z, bias, (T*)out, n,
                                                                                          cols);)
}

}  // namespace xgm
