// Residual update of a block whose sublayers all read the same normed input, fused with the
// norm that the next block (or the model's head) reads:
//
//   x <- x + a1 * y1 + a2 * (y2 + y3)          a1, a2: per-channel scales (nullptr = 1)
//   n  = x / sqrt(mean(x^2) + eps) * g         written as fp32 and / or as an activation tensor
//
// x is the fp32 residual stream, updated in place; y1 / y2 are activation tensors (float or
// bf16, row-strided), y3 is fp32 (a sum formed in fp32, e.g. the weighted sum over experts).
// Any of y1, y2, y3 may be nullptr. With g == nullptr only the sum is formed.
//
// groups > 1: the norm treats `groups` equal consecutive parts of the row separately (each divided by its own
// root mean square). bw1 / bw2: y1 and y2 are the outputs of two branches whose mean joins the residual after
// each was RMS-normed over the whole row with a plain weight: x <- x + (N0(y1) bw1 + N0(y2) bw2) / 2 + y3.
// dest != nullptr: y3 holds the rows of a routed mixture in their sorted layout, and what is added for token t is
// sum_j cw[t][j] * y3[dest[t][j]] over its `top` choices in order (cw == nullptr: weights 1).
#include "mixers_common.h"

namespace xgm {

constexpr int kMaxNormGroups = 256;

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void residual_norm_kernel(float* __restrict__ x, const TY* __restrict__ y1, int64_t ld1,
                                                            const float* __restrict__ a1, const TY* __restrict__ y2,
                                                            int64_t ld2, const float* __restrict__ y3,
                                                            const float* __restrict__ a2, const float* __restrict__ g,
                                                            float eps, float* __restrict__ n32, TO* __restrict__ nact,
                                                            int W, int vec, int groups, const float* __restrict__ bw1,
                                                            const float* __restrict__ bw2,
                                                            const int32_t* __restrict__ dest,
                                                            const float* __restrict__ cw, int top) {
  __shared__ float red[4];
  __shared__ float rinv[kMaxNormGroups];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * W;
  // the fp32 term at columns c .. c + 3 / at column c: a dense row, or the token's routed rows summed in order
  auto y3_quad = [&](int c, float (&u)[4]) {
    if (!dest) {
      ld4(y3 + (int64_t)t * W + c, u);
      return;
    }
    u[0] = u[1] = u[2] = u[3] = 0.f;
    for (int j = 0; j < top; ++j) {
      float r[4];
      ld4(y3 + (int64_t)dest[(int64_t)t * top + j] * W + c, r);
      const float wj = cw ? cw[(int64_t)t * top + j] : 1.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) u[e] += wj * r[e];
    }
  };
  auto y3_one = [&](int c) -> float {
    if (!dest) return y3[(int64_t)t * W + c];
    float u = 0.f;
    for (int j = 0; j < top; ++j)
      u += (cw ? cw[(int64_t)t * top + j] : 1.f) * y3[(int64_t)dest[(int64_t)t * top + j] * W + c];
    return u;
  };
  // two branches: their inverse root mean squares first (one pass over y1 and y2), folded into the sum below
  float b1 = 1.f, b2 = 1.f;
  if (bw1) {
    float s1 = 0.f, s2 = 0.f;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float u = ldf(y1 + (int64_t)t * ld1 + c), v = ldf(y2 + (int64_t)t * ld2 + c);
      s1 += u * u, s2 += v * v;
    }
    s1 = block_sum(s1, red);
    s2 = block_sum(s2, red);
    b1 = 0.5f / sqrtf(s1 / (float)W + eps);
    b2 = 0.5f / sqrtf(s2 / (float)W + eps);
  }
  const int gw = W / groups;   // columns per norm group
  for (int gi = 0; gi < groups; ++gi) {
    const int c0 = gi * gw, c1 = c0 + gw;
    float ss = 0.f;
    if (vec) {
      for (int c = c0 + 4 * threadIdx.x; c < c1; c += 4 * blockDim.x) {
        float v[4], u[4], s[4];
        ld4(xr + c, v);
        if (bw1) {
          float u2[4], s2[4];
          ld4(y1 + (int64_t)t * ld1 + c, u);
          ld4(y2 + (int64_t)t * ld2 + c, u2);
          ld4(bw1 + c, s);
          ld4(bw2 + c, s2);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += b1 * u[e] * s[e] + b2 * u2[e] * s2[e];
          if (y3) {
            y3_quad(c, u);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += u[e];
          }
        } else {
          if (y1) {
            ld4(y1 + (int64_t)t * ld1 + c, u);
            if (a1) ld4(a1 + c, s);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += (a1 ? s[e] : 1.f) * u[e];
          }
          if (y2 || y3) {
            float f[4] = {0.f, 0.f, 0.f, 0.f};
            if (y2) ld4(y2 + (int64_t)t * ld2 + c, f);
            if (y3) {
              y3_quad(c, u);
#pragma unroll
              for (int e = 0; e < 4; ++e) f[e] += u[e];
            }
            if (a2) ld4(a2 + c, s);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += (a2 ? s[e] : 1.f) * f[e];
          }
        }
        st4(xr + c, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += v[e] * v[e];
      }
    } else {
      for (int c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
        float v = xr[c];
        if (bw1) {
          v += b1 * ldf(y1 + (int64_t)t * ld1 + c) * bw1[c] + b2 * ldf(y2 + (int64_t)t * ld2 + c) * bw2[c];
          if (y3) v += y3_one(c);
        } else {
          if (y1) v += (a1 ? a1[c] : 1.f) * ldf(y1 + (int64_t)t * ld1 + c);
          if (y2 || y3) {
            float f = y2 ? ldf(y2 + (int64_t)t * ld2 + c) : 0.f;
            if (y3) f += y3_one(c);
            v += (a2 ? a2[c] : 1.f) * f;
          }
        }
        xr[c] = v;
        ss += v * v;
      }
    }
    if (!g) continue;
    ss = block_sum(ss, red);
    if (threadIdx.x == 0) rinv[gi] = 1.f / sqrtf(ss / (float)gw + eps);
  }
  if (!g) return;
  __syncthreads();
  // each thread re-reads only what it wrote itself
  for (int gi = 0; gi < groups; ++gi) {
    const int c0 = gi * gw, c1 = c0 + gw;
    const float r = rinv[gi];
    if (vec) {
      for (int c = c0 + 4 * threadIdx.x; c < c1; c += 4 * blockDim.x) {
        float v[4], gwt[4];
        ld4(xr + c, v);
        ld4(g + c, gwt);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = v[e] * r * gwt[e];
        if (n32) st4(n32 + (int64_t)t * W + c, v);
        if (nact) st4(nact + (int64_t)t * W + c, v);
      }
    } else {
      for (int c = c0 + threadIdx.x; c < c1; c += blockDim.x) {
        const float o = xr[c] * r * g[c];
        if (n32) n32[(int64_t)t * W + c] = o;
        if (nact) stf(nact + (int64_t)t * W + c, o);
      }
    }
  }
}

int residual_norm(float* x, const void* y1, int64_t ld1, const float* a1, const void* y2, int64_t ld2, const float* y3,
                  const float* a2, bool y_f32, const float* g, float eps, float* n32, void* nact, bool nact_f32, int T_,
                  int W, int groups, const float* bw1, const float* bw2, const int32_t* dest, const float* cw, int top,
                  hipStream_t st) {
  if (T_ <= 0) return 0;
  if (groups < 1 || groups > kMaxNormGroups || W % groups != 0 || (bw1 != nullptr) != (bw2 != nullptr) ||
      (bw1 && (!y1 || !y2 || a1 || a2)) || (dest && (!y3 || top < 1)))
    return -1;
  // the 4-wide path needs 16-byte (float) / 8-byte (bf16) aligned rows and whole quads per norm group
  const int ysz = y_f32 ? 4 : 2;
  const int vec = ((W / groups) & 3) == 0 && (!y1 || ((ld1 & 3) == 0 && (uintptr_t)y1 % (4 * ysz) == 0)) &&
                  (!y2 || ((ld2 & 3) == 0 && (uintptr_t)y2 % (4 * ysz) == 0));
#define XGM_RN(TY, TO)                                                                                                   \
  residual_norm_kernel<TY, TO><<<T_, 256, 0, st>>>(x, (const TY*)y1, ld1, a1, (const TY*)y2, ld2, y3, a2, g, eps, n32, \
                                                   (TO*)nact, W, vec, groups, bw1, bw2, dest, cw, top);
  if (y_f32) {
    if (nact_f32) { XGM_RN(float, float) } else { XGM_RN(float, bf16) }
  } else {
    if (nact_f32) { XGM_RN(bf16, float) } else { XGM_RN(bf16, bf16) }
  }
#undef XGM_RN
  return 0;
}

}  // namespace xgm
