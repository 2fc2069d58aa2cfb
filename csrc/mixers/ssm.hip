// Selective state-space recurrence with a scalar decay per head (the "state-space duality" layer),
// carried per sequence slot, and the gated group norm that follows it.
//
//   ssm_scan          per head h (group g = h / (H / G)), state S [N x P] fp32 per (slot, head):
//                       dt_t = softplus(dt_raw_t + dt_bias_h)            (not limited to a range)
//                       S_t  = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T
//                       y_t  = S_t^T C_t + D_h x_t
//                     x / B / C are columns of one activation row [x (H P) | B (G N) | C (G N)] (already
//                     through their short convolution and activation), dt_raw a column block of another.
//   gated_group_norm  v = y * silu(z) (v = y without z);  each of `ng` equal parts of v divided by its own root
//                     mean square, times w (gated first, normed second); w repeats with period wn. With
//                     `gate_after` the norm is taken of y itself and silu(z) multiplies the normed, weighted result.
//
// One workgroup = (sequence, head, 64 state columns), NW waves: lane p owns column p, wave w owns rows
// [w * NI, (w + 1) * NI) of it in registers (state rows are read and written 256 bytes at a time). B / C / x /
// dt of TT tokens at a time are staged in LDS (two buffers: the next tile's global loads are issued before the
// current tile's steps and stored after them). Per token a wave does 2 FMAs per owned state element; the
// waves' partial sums of y meet in LDS once per tile. Eight waves (two per SIMD) hide the LDS and dependency
// latency of the serial token loop.
#include "mixers_common.h"

namespace xgm {

constexpr int kScanCols = 64;   // state columns per workgroup

template <typename T, int NI, int TT, int NW>
__global__ __launch_bounds__(64 * NW) void ssm_scan_kernel(const T* __restrict__ xbc, int64_t ld_x, const T* __restrict__ dt_raw,
                                                       int64_t ld_dt, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dskip,
                                                       float* __restrict__ state, const int32_t* __restrict__ qsl,
                                                       const int32_t* __restrict__ seq_lens,
                                                       const int32_t* __restrict__ slots, float* __restrict__ y, int H,
                                                       int G, int N, int P) {
  constexpr int NB = NW * NI;                // padded state rows
  constexpr int NTH = 64 * NW;
  constexpr int ROW = 2 * NB + kScanCols;    // staged floats per token: [B | C | x]
  constexpr int PER = (TT * ROW + NTH - 1) / NTH;
  __shared__ __attribute__((aligned(16))) float stage[2][TT][ROW];
  __shared__ float dts[2][TT], decs[2][TT];
  __shared__ float ypart[TT][NW][kScanCols];
  const int s = blockIdx.x, h = blockIdx.y;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int ctx = seq_lens[s] - q;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p0 = blockIdx.z * kScanCols, p = p0 + lane;
  const bool pok = p < P;
  const int g = h / (H / G);
  const int inner = H * P;
  const float rate = expf(A_log[h]), bias = dt_bias[h], dsk = Dskip[h];
  float* Sg = state + (((int64_t)slot * H + h) * N) * P;
  float S[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = wave * NI + i;
    S[i] = (ctx > 0 && pok && n < N) ? Sg[(int64_t)n * P + p] : 0.f;
  }
  float pre[PER], pre_dt = 0.f;
  auto fetch = [&](int t0) {  // global loads of the tile starting at token t0 (zeros past the end / the sizes)
    const int nt = min(TT, q - t0);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + NTH * j;
      const int tt = e / ROW, c = e % ROW;
      float v = 0.f;
      if (tt < nt) {
        const T* row = xbc + (int64_t)(q0 + t0 + tt) * ld_x;
        if (c < NB) {
          if (c < N) v = ldf(row + inner + g * N + c);
        } else if (c < 2 * NB) {
          if (c - NB < N) v = ldf(row + inner + G * N + g * N + (c - NB));
        } else if (p0 + c - 2 * NB < P) {
          v = ldf(row + h * P + p0 + c - 2 * NB);
        }
      }
      pre[j] = v;
    }
    if (threadIdx.x < nt) pre_dt = ldf(dt_raw + (int64_t)(q0 + t0 + threadIdx.x) * ld_dt + h);
  };
  auto commit = [&](int buf, int t0) {
    const int nt = min(TT, q - t0);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + NTH * j;
      if (e < TT * ROW) (&stage[buf][0][0])[e] = pre[j];
    }
    if (threadIdx.x < nt) {
      const float d = softplusf(pre_dt + bias);
      dts[buf][threadIdx.x] = d;
      decs[buf][threadIdx.x] = expf(-rate * d);
    }
  };
  fetch(0);
  commit(0, 0);
  __syncthreads();
  int buf = 0;
  for (int t0 = 0; t0 < q; t0 += TT, buf ^= 1) {
    const int nt = min(TT, q - t0);
    const bool more = t0 + TT < q;
    if (more) fetch(t0 + TT);
    for (int tt = 0; tt < nt; ++tt) {
      const float* Br = &stage[buf][tt][wave * NI];
      const float* Cr = &stage[buf][tt][NB + wave * NI];
      const float a = decs[buf][tt], dx = dts[buf][tt] * stage[buf][tt][2 * NB + lane];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        S[i] = a * S[i] + dx * Br[i];
        acc += S[i] * Cr[i];
      }
      ypart[tt][wave][lane] = acc;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nt * kScanCols; e += NTH) {
      const int tt = e / kScanCols, c = e % kScanCols;
      if (p0 + c < P) {
        float v = dsk * stage[buf][tt][2 * NB + c];
#pragma unroll
        for (int w = 0; w < NW; ++w) v += ypart[tt][w][c];
        y[(int64_t)(q0 + t0 + tt) * inner + h * P + p0 + c] = v;
      }
    }
    if (more) commit(buf ^ 1, t0 + TT);
    __syncthreads();
  }
  if (pok) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = wave * NI + i;
      if (n < N) Sg[(int64_t)n * P + p] = S[i];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z,
                                                               int64_t ld_z, const float* __restrict__ w, int wn,
                                                               float eps, T* __restrict__ out, int inner, int gs,
                                                               int gate_after) {
  __shared__ float red[4];
  const int t = blockIdx.x, c0 = blockIdx.y * gs;
  const bool pre = z && !gate_after, post = z && gate_after;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    float v = y[(int64_t)t * inner + c0 + c];
    if (pre) v *= siluf(ldf(z + (int64_t)t * ld_z + c0 + c));
    ss += v * v;
  }
  const float r = 1.f / sqrtf(block_sum(ss, red) / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    float v = y[(int64_t)t * inner + c0 + c];
    if (pre) v *= siluf(ldf(z + (int64_t)t * ld_z + c0 + c));
    v = v * r * w[(c0 + c) % wn];
    if (post) v *= siluf(ldf(z + (int64_t)t * ld_z + c0 + c));
    stf(out + (int64_t)t * inner + c0 + c, v);
  }
}

// ================================================================== host launchers
int ssm_scan(const void* xbc, bool f32, int64_t ld_x, const void* dt_raw, int64_t ld_dt, const float* dt_bias,
             const float* A_log, const float* Dskip, float* state, const int32_t* qsl, const int32_t* seq_lens,
             const int32_t* slots, float* y, int ns, int H, int G, int N, int P, hipStream_t st) {
  if (ns <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G != 0 || N < 1 || N > 256 || P < 1) return -1;
  dim3 grid(ns, H, (P + kScanCols - 1) / kScanCols);
#define XGM_SS(NI, TT, NW)                                                                                           \
  XGM_DISPATCH_T(f32, ssm_scan_kernel<T, NI, TT, NW><<<grid, 64 * NW, 0, st>>>((const T*)xbc, ld_x, (const T*)dt_raw, \
                                                                                ld_dt, dt_bias, A_log, Dskip, state,  \
                                                                                qsl, seq_lens, slots, y, H, G, N, P);) \
  return 0;
  if (N <= 16) { XGM_SS(4, 16, 4) }
  if (N <= 32) { XGM_SS(8, 16, 4) }
  if (N <= 64) { XGM_SS(8, 8, 8) }
  if (N <= 128) { XGM_SS(16, 8, 8) }
  XGM_SS(32, 8, 8)
#undef XGM_SS
}

void gated_group_norm(const float* y, const void* z, bool f32, int64_t ld_z, const float* w, int wn, float eps, void* out,
                      int T_, int inner, int ng, bool gate_after, hipStream_t st) {
  if (T_ <= 0) return;
  // small groups (one per head): fewer threads per group
  const int gs = inner / ng, nth = gs <= 64 ? 64 : gs <= 128 ? 128 : 256;
  XGM_DISPATCH_T(f32, gated_group_norm_kernel<T><<<dim3(T_, ng), nth, 0, st>>>(y, (const T*)z, ld_z, w, wn, eps, (T*)out,
                                                                                inner, gs, gate_after ? 1 : 0);)
}

}  // namespace xgm
