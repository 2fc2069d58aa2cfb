// Gated feed-forward pieces and a routed mixture of small experts.
//
//   glu_act          [gate | up] rows -> act(gate) * up':
//                      kGluGeluTanh   0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u
//                      kGluClamped    g' = min(g, limit), u' = clamp(u, -limit, limit):  g' sigmoid(alpha g') (u' + 1)
//   grouped_router   fp32 router logits -> sigmoid scores; selection score = score + correction; the experts are
//                    split into `count` contiguous groups of equal size, a group is rated by the sum of its two
//                    highest selection scores, members of the `keep` highest-rated groups stay eligible (all
//                    others are excluded outright: selection score -inf); the `top` highest eligible selection
//                    scores win; weight = score * scale (the correction does not enter it, no normalisation).
//                    For steps of few rows the logits x . rw[e] (fp32 rows and router weights) are formed here
//                    by a four-wave workgroup per token, eight experts per sweep over the row, instead of being
//                    read (the waves then repeat the same selection, so every barrier is met by all of them).
//   moe_align        (token, choice) pairs sorted by expert into tiles of `tm` rows (padded with -1)
//   grouped_gemm     per tile: rows x expert weights, in one of three modes:
//                      kGemmRows    A rows as they lie in the sorted layout -> fp32 rows (the second product)
//                      kGemmGated   A rows gathered by token; weights [gate | up]; output glu(gate, up)
//                      kGemmAct     A rows gathered by token; output act(s * (W a)), s = row_scale[pair] (nullptr = 1):
//                                   a routing weight that multiplies the expert's INPUT is applied to the fp32
//                                   accumulator of the (linear) first product.  kActRelu2: max(z, 0)^2
//   moe_combine      out[t] = sum_j weight[t, j] * y[row of pair (t, j)]   (fixed order: bit-stable; weights
//                    nullptr = 1)
//
// Activations / weights are T = float or bf16; router, weights of the sum and the sum itself are fp32.
#include "mixers_common.h"

#include <algorithm>

namespace xgm {

constexpr int kGluGeluTanh = 0, kGluClamped = 1, kActRelu2 = 2;
constexpr int kGemmRows = 0, kGemmGated = 1, kGemmAct = 2;

__device__ __forceinline__ float act1(int kind, float z) {
  (void)kind;  // kActRelu2
  const float r = fmaxf(z, 0.f);
  return r * r;
}

__device__ __forceinline__ float glu(int kind, float g, float u, float limit, float alpha) {
  if (kind == kGluGeluTanh) {
    const float c = 0.7978845608028654f;  // sqrt(2 / pi)
    return 0.5f * g * (1.f + tanhf(c * (g + 0.044715f * g * g * g))) * u;
  }
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoidf(alpha * g) * (u + 1.f);
}

template <typename T>
__global__ void glu_act_kernel(const T* __restrict__ in, int64_t ld, T* __restrict__ out, int F, int64_t total, int kind,
                               float limit, float alpha) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / F;
    const int c = (int)(i % F);
    const T* row = in + t * ld;
    stf(out + i, glu(kind, ldf(row + c), ldf(row + F + c), limit, alpha));
  }
}

// ------------------------------------------------------------------ router: one wave per token
constexpr int kMaxEPL = 8;  // experts per lane: E <= 512

constexpr int kRouterSweep = 8;   // experts per sweep over the row when the logits are formed here

__global__ __launch_bounds__(256) void grouped_router_kernel(const float* __restrict__ logits, const float* __restrict__ corr,
                                                             int E, int count, int keep, int top, float scale,
                                                             int32_t* __restrict__ ids, float* __restrict__ wts,
                                                             const float* __restrict__ x, const float* __restrict__ rw,
                                                             int W) {
  extern __shared__ float sm[];
  float* cs = sm;              // [E] choice scores
  float* gs = sm + E;          // [count] group scores
  int* kept = (int*)(gs + count);  // [count]
  float* lg = (float*)(kept + count);   // [E] logits formed here (x != nullptr)
  float* part = lg + E;                 // [waves][kRouterSweep] partial sums
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int per = E / count;
  if (x) {
    const float* xr = x + (int64_t)t * W;
    const bool vec = (W & 3) == 0;
    for (int e0 = 0; e0 < E; e0 += kRouterSweep) {
      float acc[kRouterSweep];
#pragma unroll
      for (int j = 0; j < kRouterSweep; ++j) acc[j] = 0.f;
      if (vec) {
        for (int c = 4 * threadIdx.x; c < W; c += 4 * blockDim.x) {
          float a[4];
          ld4(xr + c, a);
#pragma unroll
          for (int j = 0; j < kRouterSweep; ++j)
            if (e0 + j < E) {
              float b[4];
              ld4(rw + (int64_t)(e0 + j) * W + c, b);
              acc[j] += a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
            }
        }
      } else {
        for (int c = threadIdx.x; c < W; c += blockDim.x) {
          const float a = xr[c];
#pragma unroll
          for (int j = 0; j < kRouterSweep; ++j)
            if (e0 + j < E) acc[j] += a * rw[(int64_t)(e0 + j) * W + c];
        }
      }
#pragma unroll
      for (int j = 0; j < kRouterSweep; ++j) acc[j] = wave_sum(acc[j]);
      if (lane == 0) {
#pragma unroll
        for (int j = 0; j < kRouterSweep; ++j) part[wave * kRouterSweep + j] = acc[j];
      }
      __syncthreads();
      if (threadIdx.x < kRouterSweep && e0 + threadIdx.x < E) {
        float v = 0.f;
        for (int w = 0; w < nw; ++w) v += part[w * kRouterSweep + threadIdx.x];
        lg[e0 + threadIdx.x] = v;
      }
      __syncthreads();
    }
  }
  float sc[kMaxEPL], ch[kMaxEPL];
#pragma unroll
  for (int i = 0; i < kMaxEPL; ++i) {
    const int e = lane + 64 * i;
    sc[i] = 0.f, ch[i] = -INFINITY;
    if (e < E) {
      sc[i] = sigmoidf(x ? lg[e] : logits[(int64_t)t * E + e]);
      ch[i] = sc[i] + (corr ? corr[e] : 0.f);
      cs[e] = ch[i];
    }
  }
  __syncthreads();
  for (int g = lane; g < count; g += 64) {  // sum of the group's two largest choice scores
    float a = -INFINITY, b = -INFINITY;
    for (int j = 0; j < per; ++j) {
      const float v = cs[g * per + j];
      if (v > a) b = a, a = v;
      else if (v > b) b = v;
    }
    gs[g] = per > 1 ? a + b : a;
  }
  __syncthreads();
  for (int g = lane; g < count; g += 64) {  // rank among the groups (ties: the lower index first)
    int rank = 0;
    const float v = gs[g];
    for (int o = 0; o < count; ++o) rank += (gs[o] > v || (gs[o] == v && o < g)) ? 1 : 0;
    kept[g] = rank < keep ? 1 : 0;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kMaxEPL; ++i) {
    const int e = lane + 64 * i;
    if (e < E && !kept[e / per]) ch[i] = -INFINITY;
  }
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY, bs = 0.f;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kMaxEPL; ++i) {
      const int e = lane + 64 * i;
      if (e < E && (ch[i] > bv || (ch[i] == bv && e < be))) bv = ch[i], be = e, bs = sc[i];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64), os = __shfl_xor(bs, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (ov > bv || (ov == bv && oe < be)) bv = ov, be = oe, bs = os;
    }
    if (be >= E) be = 0, bs = 0.f;  // fewer candidates than `top`: expert 0 with weight 0
    if (lane == 0) {
      ids[(int64_t)t * top + j] = be;
      wts[(int64_t)t * top + j] = bs * scale;
    }
#pragma unroll
    for (int i = 0; i < kMaxEPL; ++i)
      if (lane + 64 * i == be) ch[i] = -INFINITY;
  }
}

// ------------------------------------------------------------------ pairs -> expert tiles (one workgroup)
__global__ __launch_bounds__(1024) void moe_align_kernel(const int32_t* __restrict__ ids, int pairs, int E, int cap,
                                                         int kTileM, int32_t* __restrict__ rows,
                                                         int32_t* __restrict__ tile_expert, int32_t* __restrict__ dest) {
  extern __shared__ int si[];
  int* cnt = si;          // [E]
  int* off = si + E;      // [E + 1] padded starts
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) atomicAdd(&cnt[ids[i]], 1);
  for (int i = threadIdx.x; i < cap; i += blockDim.x) rows[i] = -1;
  for (int i = threadIdx.x; i < cap / kTileM; i += blockDim.x) tile_expert[i] = -1;
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o;
      o += (cnt[e] + kTileM - 1) / kTileM * kTileM;
    }
    off[E] = o;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += blockDim.x) {
    for (int tl = off[e] / kTileM; tl < off[e + 1] / kTileM; ++tl) tile_expert[tl] = e;
    cnt[e] = 0;  // becomes the fill cursor
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = ids[i];
    const int r = off[e] + atomicAdd(&cnt[e], 1);
    rows[r] = i;
    dest[i] = r;
  }
}

// ------------------------------------------------------------------ grouped GEMM, general form
// Tile = 16 rows x 64 columns, 256 threads: thread (tr = tid / 16, tc = tid % 16) owns row tr and
// columns tc + 16 j. K runs through LDS in chunks of 32. GATED: the weight holds [gate (F rows) | up (F rows)]
// and the output column f is glu(gate_f, up_f); A rows are gathered through rows[] / top. `tm` = rows per
// expert tile of the layout (a multiple of 16).
template <typename T, int MODE>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(const T* __restrict__ A, int64_t lda, const T* __restrict__ Wt,
                                                           const int32_t* __restrict__ rows,
                                                           const int32_t* __restrict__ tile_expert, int tm, int top,
                                                           int Nout, int K, void* __restrict__ out, int kind, float limit,
                                                           float alpha, const float* __restrict__ row_scale) {
  constexpr bool GATED = MODE == kGemmGated, FIRST = MODE != kGemmRows;
  __shared__ float As[16][33];
  __shared__ float Ws[64][33];
  __shared__ float Us[GATED ? 64 : 1][33];
  const int rbase = blockIdx.x * 16;
  const int e = tile_expert[rbase / tm];
  if (e < 0) return;
  const int n0 = blockIdx.y * 64;
  const int tr = threadIdx.x >> 4, tc = threadIdx.x & 15;
  const int r = rbase + tr;
  const int pr = rows[r];
  const int64_t wrows = GATED ? 2 * (int64_t)Nout : (int64_t)Nout;
  const T* We = Wt + (int64_t)e * wrows * K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, accu[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    __syncthreads();
    for (int i = threadIdx.x; i < 16 * 32; i += 256) {
      const int rr = i >> 5, kk = i & 31;
      const int p2 = rows[rbase + rr];
      float v = 0.f;
      if (p2 >= 0 && k0 + kk < K) v = ldf(A + (int64_t)(FIRST ? p2 / top : rbase + rr) * lda + k0 + kk);
      As[rr][kk] = v;
    }
    for (int i = threadIdx.x; i < 64 * 32; i += 256) {
      const int nn = i >> 5, kk = i & 31;
      const bool ok = n0 + nn < Nout && k0 + kk < K;
      Ws[nn][kk] = ok ? ldf(We + (int64_t)(n0 + nn) * K + k0 + kk) : 0.f;
      if (GATED) Us[nn][kk] = ok ? ldf(We + (int64_t)(Nout + n0 + nn) * K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < 32; ++kk) {
      const float a = As[tr][kk];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] += a * Ws[tc + 16 * j][kk];
        if (GATED) accu[j] += a * Us[tc + 16 * j][kk];
      }
    }
  }
  if (pr < 0) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tc + 16 * j;
    if (n >= Nout) continue;
    if (GATED) stf((T*)out + (int64_t)r * Nout + n, glu(kind, acc[j], accu[j], limit, alpha));
    else if (FIRST) stf((T*)out + (int64_t)r * Nout + n, act1(kind, acc[j] * (row_scale ? row_scale[pr] : 1.f)));
    else ((float*)out)[(int64_t)r * Nout + n] = acc[j];
  }
}

// ---- matrix-core form (bf16; K % 32 == 0, Nout % 16 == 0). A / B fragments come straight from global
// memory (16 or 32 bytes per lane and step), accumulators are fp32. For steps with few rows per expert (layout
// tiles of 16 rows). Two shapes of one kernel:
//   SPLITK = false: a workgroup owns 16 MT rows x 4 x 16 NT columns, each wave 16 NT of the columns over the whole K
//            (a long loop, four steps' loads in flight);
//   SPLITK = true:  a workgroup owns 16 rows x 16 NT columns, its four waves a quarter of K each; the partial sums
//            meet in LDS.
using xgk::as_frag;
using xgk::f32x4_t;
using xgk::ld16;
using xgk::mfma16x16x32;

template <int MODE, int MT, int NT, bool SPLITK, bool K64>
__global__ __launch_bounds__(256) void grouped_gemm_mfma_kernel(const bf16* __restrict__ A, int64_t lda,
                                                                const bf16* __restrict__ Wt,
                                                                const int32_t* __restrict__ rows,
                                                                const int32_t* __restrict__ tile_expert, int top,
                                                                int Nout, int K, void* __restrict__ out, int kind,
                                                                float limit, float alpha,
                                                                const float* __restrict__ row_scale) {
  constexpr bool GATED = MODE == kGemmGated, FIRST = MODE != kGemmRows;
  constexpr int NG = GATED ? NT : 1;
  __shared__ float red[SPLITK ? 3 : 1][SPLITK ? MT * (NT + NG) : 1][64][4];
  const int tile = blockIdx.x;          // layout tile of 16 MT rows
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = SPLITK ? blockIdx.y * 16 * NT : (blockIdx.y * 4 + wave) * 16 * NT;
  if (n0 >= Nout) return;               // (SPLITK: uniform over the workgroup)
  const int l16 = lane & 15, kg = lane >> 4;
  const int64_t wrows = GATED ? 2 * (int64_t)Nout : (int64_t)Nout;
  const bf16* We = Wt + (int64_t)e * wrows * K;
  const int rbase = tile * 16 * MT;
  const bf16* arow[MT];
  bool aok[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int pa = rows[rbase + 16 * i + l16];
    aok[i] = pa >= 0;
    arow[i] = A + (int64_t)(FIRST ? max(pa, 0) / top : rbase + 16 * i + l16) * lda + kg * (K64 ? 16 : 8);
  }
  f32x4_t acc[MT][NT], accu[MT][NG];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NG; ++j) accu[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  // K64: a lane takes 32 contiguous bytes of a row per step (the four lanes of a row 128 bytes) and feeds them
  // to two MFMAs. A and B use the same assignment of k to (lane, MFMA), and a sum over k has no order.
  constexpr int KS = K64 ? 64 : 32, KL = K64 ? 16 : 8;
  const int kper = SPLITK ? ((K / KS + 3) / 4) * KS : K;
  const int kbeg = SPLITK ? wave * kper : 0, kend = min(K, kbeg + kper);
#pragma unroll(SPLITK ? 2 : 4)
  for (int k0 = kbeg; k0 < kend; k0 += KS) {
    uint4 av[MT][K64 ? 2 : 1], bv[NT][K64 ? 2 : 1], uv[NG][K64 ? 2 : 1];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int h = 0; h < (K64 ? 2 : 1); ++h)
        av[i][h] = aok[i] ? ld16(arow[i] + k0 + 8 * h) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = min(n0 + 16 * j, Nout - 16) + l16;  // whole 16-column tiles (Nout % 16 == 0); clamped ones are not stored
#pragma unroll
      for (int h = 0; h < (K64 ? 2 : 1); ++h) {
        bv[j][h] = ld16(We + (int64_t)n * K + k0 + kg * KL + 8 * h);
        if (GATED) uv[j][h] = ld16(We + (int64_t)(Nout + n) * K + k0 + kg * KL + 8 * h);
      }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int h = 0; h < (K64 ? 2 : 1); ++h) {
          // D = A (rows x k) B (k x cols): accumulator entry r of lane (l16, kg) is row kg * 4 + r, column l16
          acc[i][j] = mfma16x16x32(as_frag(av[i][h]), as_frag(bv[j][h]), acc[i][j]);
          if (GATED) accu[i][j] = mfma16x16x32(as_frag(av[i][h]), as_frag(uv[j][h]), accu[i][j]);
        }
  }
  if (SPLITK) {  // waves 1..3 hand their partial sums to wave 0
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) red[wave - 1][i * (NT + NG) + j][lane][r] = acc[i][j][r];
        if (GATED) {
#pragma unroll
          for (int j = 0; j < NG; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[wave - 1][i * (NT + NG) + NT + j][lane][r] = accu[i][j][r];
        }
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][j][r] += red[w][i * (NT + NG) + j][lane][r];
        if (GATED) {
#pragma unroll
          for (int j = 0; j < NG; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) accu[i][j][r] += red[w][i * (NT + NG) + NT + j][lane][r];
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n0 + 16 * j + l16;
      if (n0 + 16 * j >= Nout) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rr = rbase + 16 * i + kg * 4 + r;
        const int pr = rows[rr];
        if (pr < 0) continue;
        if (GATED) ((bf16*)out)[(int64_t)rr * Nout + n] = f2bf(glu(kind, acc[i][j][r], accu[i][GATED ? j : 0][r], limit, alpha));
        else if (FIRST) ((bf16*)out)[(int64_t)rr * Nout + n] = f2bf(act1(kind, acc[i][j][r] * (row_scale ? row_scale[pr] : 1.f)));
        else ((float*)out)[(int64_t)rr * Nout + n] = acc[i][j][r];
      }
    }
}

// ---- prompt-sized steps (layout tiles of 64 or 128 rows): a workgroup owns 16 MT rows x 4 x 16 NT columns. The A rows
// (gathered token rows, shared by the four waves) go through LDS, KS = 32 or 64 k at a time in two buffers, one barrier
// per step; every wave streams its own B columns from global memory into registers, with PF one step ahead of their
// use (measured: 64-wide steps with the loads ahead gain about a tenth for one weight block per expert, and lose for the
// gated form, whose two weight blocks per step then cost a third of the occupancy).
template <int MODE, int MT, int NT, int KS, bool PF>
__global__ __launch_bounds__(256) void grouped_gemm_mfma_lds_kernel(const bf16* __restrict__ A, int64_t lda,
                                                                    const bf16* __restrict__ Wt,
                                                                    const int32_t* __restrict__ rows,
                                                                    const int32_t* __restrict__ tile_expert, int tm,
                                                                    int top, int Nout, int K, void* __restrict__ out,
                                                                    int kind, float limit, float alpha,
                                                                    const float* __restrict__ row_scale) {
  constexpr bool GATED = MODE == kGemmGated, FIRST = MODE != kGemmRows;
  constexpr int LDA = KS + 8, NG = GATED ? NT : 1, RPT = MT / 4;  // RPT: staged rows per thread
  constexpr int KH = KS / 32;                                     // 32-wide k halves (MFMA depth) per step
  __shared__ __attribute__((aligned(16))) uint16_t As[2][16 * MT * LDA];
  const int tile = blockIdx.x;  // 16 MT rows of a layout tile of tm rows
  const int e = tile_expert[tile * 16 * MT / tm];
  if (e < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.y * 4 + wave) * 16 * NT;
  const int l16 = lane & 15, kg = lane >> 4;
  const int64_t wrows = GATED ? 2 * (int64_t)Nout : (int64_t)Nout;
  const bf16* We = Wt + (int64_t)e * wrows * K;
  const int rbase = tile * 16 * MT;
  // staging: thread -> (rows tid / 4 + 64 r, 16-byte chunks tid % 4 (+ 4)) of the (16 MT) x KS A block
  const int srow = threadIdx.x >> 2, sch = threadIdx.x & 3;
  int pa[RPT];
  const bf16* asrc[RPT];
#pragma unroll
  for (int r = 0; r < RPT; ++r) {
    pa[r] = rows[rbase + srow + 64 * r];
    asrc[r] = A + (int64_t)(FIRST ? max(pa[r], 0) / top : rbase + srow + 64 * r) * lda + sch * 8;
  }
  f32x4_t acc[MT][NT], accu[MT][NG];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < NG; ++j) accu[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  const bool wave_on = n0 < Nout;
  // this wave's B rows (whole 16-column tiles; clamped ones are not stored)
  const bf16* brow[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) brow[j] = We + (int64_t)(min(n0 + 16 * j, Nout - 16) + l16) * K + kg * 8;
  uint4 bv[NT][KH], uv[NG][KH];
  auto load_b = [&](int k0, uint4 (&b)[NT][KH], uint4 (&u)[NG][KH]) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int h = 0; h < KH; ++h) {
        b[j][h] = ld16(brow[j] + k0 + 32 * h);
        if (GATED) u[GATED ? j : 0][h] = ld16(brow[j] + (int64_t)Nout * K + k0 + 32 * h);
      }
  };
#pragma unroll
  for (int r = 0; r < RPT; ++r)
#pragma unroll
    for (int h = 0; h < KH; ++h)
      xgk::st16(&As[0][(srow + 64 * r) * LDA + sch * 8 + 32 * h],
                pa[r] >= 0 ? ld16(asrc[r] + 32 * h) : make_uint4(0, 0, 0, 0));
  if (PF && wave_on) load_b(0, bv, uv);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += KS, buf ^= 1) {
    const bool more = k0 + KS < K;
    uint4 anext[RPT][KH], bn[NT][KH], un[NG][KH];
#pragma unroll
    for (int r = 0; r < RPT; ++r)
#pragma unroll
      for (int h = 0; h < KH; ++h)
        anext[r][h] = (more && pa[r] >= 0) ? ld16(asrc[r] + k0 + KS + 32 * h) : make_uint4(0, 0, 0, 0);
    if (wave_on) {
      if (!PF) load_b(k0, bv, uv);
      else if (more) load_b(k0 + KS, bn, un);
#pragma unroll
      for (int h = 0; h < KH; ++h)
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const uint4 av = ld16(&As[buf][(16 * i + l16) * LDA + 32 * h + kg * 8]);
#pragma unroll
          for (int j = 0; j < NT; ++j) {
            acc[i][j] = mfma16x16x32(as_frag(av), as_frag(bv[j][h]), acc[i][j]);
            if (GATED) accu[i][j] = mfma16x16x32(as_frag(av), as_frag(uv[GATED ? j : 0][h]), accu[i][GATED ? j : 0]);
          }
        }
      if (PF && more) {
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int h = 0; h < KH; ++h) {
            bv[j][h] = bn[j][h];
            if (GATED) uv[GATED ? j : 0][h] = un[GATED ? j : 0][h];
          }
      }
    }
    if (more) {
#pragma unroll
      for (int r = 0; r < RPT; ++r)
#pragma unroll
        for (int h = 0; h < KH; ++h) xgk::st16(&As[buf ^ 1][(srow + 64 * r) * LDA + sch * 8 + 32 * h], anext[r][h]);
    }
    __syncthreads();
  }
  if (!wave_on) return;
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int n = n0 + 16 * j + l16;
      if (n0 + 16 * j >= Nout) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int rr = rbase + 16 * i + kg * 4 + r;
        const int pr = rows[rr];
        if (pr < 0) continue;
        if (GATED) ((bf16*)out)[(int64_t)rr * Nout + n] = f2bf(glu(kind, acc[i][j][r], accu[i][GATED ? j : 0][r], limit, alpha));
        else if (FIRST) ((bf16*)out)[(int64_t)rr * Nout + n] = f2bf(act1(kind, acc[i][j][r] * (row_scale ? row_scale[pr] : 1.f)));
        else ((float*)out)[(int64_t)rr * Nout + n] = acc[i][j][r];
      }
    }
}

__global__ void moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ dest,
                                   const float* __restrict__ wts, int top, int W, float* __restrict__ out) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j)
      acc += (wts ? wts[(int64_t)t * top + j] : 1.f) * y[(int64_t)dest[(int64_t)t * top + j] * W + c];
    out[(int64_t)t * W + c] = acc;
  }
}

// ================================================================== host launchers
void glu_act(const void* in, bool f32, int64_t ld, void* out, int T_, int F, int kind, float limit, float alpha,
             hipStream_t st) {
  const int64_t total = (int64_t)T_ * F;
  if (total <= 0) return;
  const int blocks = (int)std::min<int64_t>((total + 255) / 256, 1 << 16);
  XGM_DISPATCH_T(f32, glu_act_kernel<T><<<blocks, 256, 0, st>>>((const T*)in, ld, (T*)out, F, total, kind, limit, alpha);)
}

int grouped_router(const float* logits, const float* corr, int T_, int E, int count, int keep, int top, float scale,
                   int32_t* ids, float* wts, const float* x, const float* rw, int W, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (E < 1 || E > 64 * kMaxEPL || count < 1 || E % count != 0 || keep < 1 || keep > count || top < 1 ||
      top > keep * (E / count))
    return -1;
  if ((x != nullptr) != (rw != nullptr) || (x && W < 1) || (!x && !logits)) return -2;
  const int nth = x ? 256 : 64;
  const size_t lds = (2 * E + 2 * count + 4 * kRouterSweep) * sizeof(float);
  grouped_router_kernel<<<T_, nth, lds, st>>>(logits, corr, E, count, keep, top, scale, ids, wts, x, rw, W);
  return 0;
}

int moe_align(const int32_t* ids, int pairs, int E, int cap, int tm, int32_t* rows, int32_t* tile_expert, int32_t* dest,
              hipStream_t st) {
  if (pairs <= 0) return 0;
  if (E < 1 || E > 4096 || tm < 16 || tm % 16 != 0 || cap % tm != 0 || cap < pairs + E * (tm - 1)) return -1;
  moe_align_kernel<<<1, 1024, (2 * E + 1) * sizeof(int), st>>>(ids, pairs, E, cap, tm, rows, tile_expert, dest);
  return 0;
}

int grouped_gemm(const void* A, bool f32, int64_t lda, const void* Wt, const int32_t* rows, const int32_t* tile_expert,
                 int cap, int tm, int top, int Nout, int K, int mode, void* out, int kind, float limit, float alpha,
                 const float* row_scale, bool mfma, hipStream_t st) {
  if (cap <= 0) return 0;
  if ((tm != 16 && tm != 32 && tm != 64 && tm != 128) || cap % tm != 0 || Nout < 1 || K < 1 || mode < kGemmRows || mode > kGemmAct ||
      (mode == kGemmGated && kind != kGluGeluTanh && kind != kGluClamped) || (mode == kGemmAct && kind != kActRelu2) ||
      (row_scale && mode != kGemmAct))
    return -1;
  if (!f32 && mfma && K % 32 == 0 && Nout % 16 == 0 && lda % 8 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)Wt % 16 == 0) {
  // few rows per expert: layout tiles of 16 rows, or of 32 once many experts would fill more than one such tile (an
  // expert's weights are then streamed once instead of once per 16 rows)
#define XGM_GG2(MODE, MT, K64)                                                                                      \
  grouped_gemm_mfma_kernel<MODE, MT, 2, true, K64><<<dim3(cap / tm, (Nout + 31) / 32), 256, 0, st>>>(                \
      (const bf16*)A, lda, (const bf16*)Wt, rows, tile_expert, top, Nout, K, out, kind, limit, alpha, row_scale);
#define XGM_GG(MODE, K64)     \
  if (tm == 32) {             \
    XGM_GG2(MODE, 2, K64)     \
  } else {                    \
    XGM_GG2(MODE, 1, K64)     \
  }
#define XGM_GL2(MODE, MT, NT, KS, PF)                                                                                  \
  grouped_gemm_mfma_lds_kernel<MODE, MT, NT, KS, PF>                                                                   \
      <<<dim3(cap / (16 * MT), (Nout + 64 * NT - 1) / (64 * NT)), 256, 0, st>>>(                                       \
          (const bf16*)A, lda, (const bf16*)Wt, rows, tile_expert, tm, top, Nout, K, out, kind, limit, alpha, row_scale);
#define XGM_GL(MODE, MT, NT)                 \
  if (MODE != kGemmGated && K % 64 == 0) {   \
    XGM_GL2(MODE, MT, NT, 64, true)          \
  } else {                                   \
    XGM_GL2(MODE, MT, NT, 32, false)         \
  }
    if (tm == 128) {         // gated: 64 x 128 per workgroup (two accumulator sets); one weight block: 128 x 128
      if (mode == kGemmGated) { XGM_GL(kGemmGated, 4, 2) } else if (mode == kGemmAct) { XGM_GL(kGemmAct, 8, 2) } else { XGM_GL(kGemmRows, 8, 2) }
    } else if (tm == 64) {   // gated: 64 x 128; one weight block: 64 x 256
      if (mode == kGemmGated) { XGM_GL(kGemmGated, 4, 2) } else if (mode == kGemmAct) { XGM_GL(kGemmAct, 4, 4) } else { XGM_GL(kGemmRows, 4, 4) }
    } else if (K % 64 == 0) {
      if (mode == kGemmGated) { XGM_GG(kGemmGated, true) } else if (mode == kGemmAct) { XGM_GG(kGemmAct, true) } else { XGM_GG(kGemmRows, true) }
    } else {
      if (mode == kGemmGated) { XGM_GG(kGemmGated, false) } else if (mode == kGemmAct) { XGM_GG(kGemmAct, false) } else { XGM_GG(kGemmRows, false) }
    }
#undef XGM_GL
#undef XGM_GL2
#undef XGM_GG
#undef XGM_GG2
    return 0;
  }
  dim3 grid(cap / 16, (Nout + 63) / 64);
#define XGM_G0(MODE)                                                                                                    \
  XGM_DISPATCH_T(f32, grouped_gemm_kernel<T, MODE><<<grid, 256, 0, st>>>((const T*)A, lda, (const T*)Wt, rows, tile_expert, \
                                                                          tm, top, Nout, K, out, kind, limit, alpha,     \
                                                                          row_scale);)
  if (mode == kGemmGated) { XGM_G0(kGemmGated) } else if (mode == kGemmAct) { XGM_G0(kGemmAct) } else { XGM_G0(kGemmRows) }
#undef XGM_G0
  return 0;
}

void moe_combine(const float* y, const int32_t* dest, const float* wts, int T_, int top, int W, float* out, hipStream_t st) {
  if (T_ <= 0) return;
  moe_combine_kernel<<<T_, 256, 0, st>>>(y, dest, wts, top, W, out);
}

}  // namespace xgm
