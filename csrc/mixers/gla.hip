// Gated linear recurrence with one decay per state row (gated linear attention; with k = 1 - f the
// write strength is the complement of the forget gate), carried per sequence slot.
//
//   lower_bound_gates  from a fused projection row: q = silu(z_q);  f = l + (1 - l) * sigmoid(z_f + b)
//                      (a forget gate bounded below by l, per channel), both fp32
//   decay_gates        q = z_q * q_scale, k = z_k and a decay per key channel f = sigmoid(z + b)^(1 / tau),
//                      evaluated as exp(-softplus(-(z + b)) / tau), all fp32 (the inputs of gated_linear_scan with k)
//   gated_linear_scan  per head, state S [dk x dv] fp32 per (slot, head):
//                        S_t = diag(f_t) S_(t-1) + k_t v_t^T        (k_t = 1 - f_t when k == nullptr)
//                        o_t = S_t^T q_t
//                      q / f / k are fp32 tensors, or (raw form) q and f are taken straight from the fused
//                      projection row and pass silu / the lower-bounded sigmoid while they are staged
//
// One workgroup = (sequence, head, 64 or 32 state columns), NW waves: a lane owns one column and NI rows of it in
// registers (64 columns: wave w owns rows [w * NI, (w + 1) * NI); 32 columns: each half of a wave its own NI rows). f / k / q / v of TT tokens at a time are staged in LDS (two buffers:
// the next tile's global loads are issued before the current tile's steps and stored after them). Per token
// a wave does 2 FMAs per owned state element; the waves' partial sums of o meet in LDS once per tile, in
// wave order.
//
// Long portions, so that a few sequences still fill the chip: the recurrence is linear in S, so a chunk of kScanChunk
// tokens is summed up by (A, B) with S_end = diag(A) S_start + B. A first launch (pass 1) runs every chunk from a
// zero state without outputs and stores its A [dk] and B [dk x dv] (and sets the sequence's incoming state aside);
// a second launch (pass 2) folds the chunks before its own onto the incoming state, in order, and runs its chunk
// with outputs; the chunk that holds the last token writes the state back. Chunk slot of (sequence s, chunk z):
// q0_s / kScanChunk + s + z, distinct for all chunks of a step and below T / kScanChunk + ns + 1.
#include "mixers_common.h"

namespace xgm {

template <typename T>
__global__ void lower_bound_gates_kernel(const T* __restrict__ proj, int64_t ld, int off_q, int off_f, int n,
                                         const float* __restrict__ f_bias, const float* __restrict__ lower,
                                         float* __restrict__ q, float* __restrict__ f, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / n;
  const int c = (int)(i % n);
  const T* row = proj + t * ld;
  q[i] = siluf(ldf(row + off_q + c));
  const float l = lower[c];
  f[i] = l + (1.f - l) * sigmoidf(ldf(row + off_f + c) + (f_bias ? f_bias[c] : 0.f));
}

template <typename T>
__global__ void decay_gates_kernel(const T* __restrict__ proj, int64_t ld, int off_q, int off_k, int n, float q_scale,
                                   const T* __restrict__ z, int64_t ld_z, const float* __restrict__ z_bias, float inv_tau,
                                   float* __restrict__ q, float* __restrict__ f, float* __restrict__ k, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / n;
  const int c = (int)(i % n);
  const T* row = proj + t * ld;
  q[i] = ldf(row + off_q + c) * q_scale;
  k[i] = ldf(row + off_k + c);
  const float zz = ldf(z + t * ld_z + c) + (z_bias ? z_bias[c] : 0.f);
  f[i] = expf(-softplusf(-zz) * inv_tau);   // log sigmoid(z) = -softplus(-z)
}

// State columns per workgroup: COLS = 64 (lane = column) or 32 (lanes 0-31 and 32-63 hold the same 32 columns for
// different rows, their partial sums meet by one cross-lane add): the narrow form keeps all lanes busy for value sizes
// up to 32.

// RAW: q and f are read as columns [off_q, off_q + H dk) / [off_f, ..) of the activation rows `raw` and go
// through silu / the lower-bounded sigmoid while they are staged (no pass of their own, half the bytes), and the
// write strength is 1 - f. Otherwise q, f (and k, or 1 - f when k == nullptr) are fp32 tensors [T, H dk].
constexpr int kScanChunk = 256;

template <typename T, int NI, int TT, int NW, bool RAW, int COLS>
__global__ __launch_bounds__(64 * NW) void gated_linear_scan_kernel(
    const float* __restrict__ q, const float* __restrict__ f, const float* __restrict__ k, const T* __restrict__ raw,
    int64_t ld_raw, int off_q, int off_f, const float* __restrict__ f_bias, const float* __restrict__ lower,
    const T* __restrict__ v, int64_t ld_v, float* __restrict__ state, const int32_t* __restrict__ qsl,
    const int32_t* __restrict__ seq_lens, const int32_t* __restrict__ slots, float* __restrict__ o, int H, int dk,
    int dv, int pass, int nc, float* __restrict__ chA, float* __restrict__ chB, float* __restrict__ s_in) {
  constexpr int HALVES = 64 / COLS;          // row groups per wave
  constexpr int NB = NW * HALVES * NI;       // padded state rows
  constexpr int NTH = 64 * NW;
  constexpr int NQ = RAW ? 2 : 3;            // staged row blocks: [f | q | (k)]
  constexpr int ROW = NQ * NB + COLS;        // staged floats per token: [f | q | (k) | v]
  constexpr int PER = (TT * ROW + NTH - 1) / NTH;
  __shared__ __attribute__((aligned(16))) float stage[2][TT][ROW];
  __shared__ float opart[TT][NW][COLS];
  // pass 0: the whole portion in one workgroup; 1 / 2: chunk z of it (see above)
  const int s = pass ? blockIdx.x / nc : blockIdx.x, z = pass ? blockIdx.x % nc : 0, h = blockIdx.y;
  const int q0 = qsl[s], qn = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || qn <= 0) return;
  const int c0 = pass ? z * kScanChunk : 0, c1 = pass ? min(qn, c0 + kScanChunk) : qn;   // this workgroup's tokens
  if (c0 >= qn) return;
  const int ctx = seq_lens[s] - qn;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane % COLS, rg = wave * HALVES + lane / COLS;   // column within the block, row group
  const int p0 = blockIdx.z * COLS, p = p0 + col;
  const bool pok = p < dv;
  const int nqk = H * dk, nv = H * dv;
  float* Sg = state + (((int64_t)slot * H + h) * dk) * dv;
  float S[NI], Ap[NI];
  const int64_t cs0 = pass ? q0 / kScanChunk + s : 0;   // the sequence's first chunk slot
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = rg * NI + i;
    const bool ok = pok && n < dk;
    Ap[i] = 1.f;
    if (pass == 0) {
      S[i] = (ctx > 0 && ok) ? Sg[(int64_t)n * dv + p] : 0.f;
    } else if (pass == 1) {
      if (z == 0 && ok) s_in[(((int64_t)s * H + h) * dk + n) * dv + p] = ctx > 0 ? Sg[(int64_t)n * dv + p] : 0.f;
      S[i] = 0.f;
    } else {
      S[i] = ok ? s_in[(((int64_t)s * H + h) * dk + n) * dv + p] : 0.f;
      for (int zc = 0; zc < z; ++zc) {
        const int64_t cr = ((cs0 + zc) * H + h) * dk + n;
        if (ok) S[i] = chA[cr] * S[i] + chB[cr * dv + p];
      }
    }
  }
  float pre[PER];
  auto fetch = [&](int t0) {  // global loads of the tile starting at token t0 (zeros past the end / the sizes)
    const int nt = min(TT, c1 - t0);
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + NTH * j;
      const int tt = e / ROW, c = e % ROW;
      float val = 0.f;
      if (tt < nt) {
        const int64_t tok = q0 + t0 + tt;
        const int blk = c / NB, cc = c % NB;
        if (blk < NQ) {
          if (cc < dk) {
            if (RAW) {
              val = ldf(raw + tok * ld_raw + (blk == 0 ? off_f : off_q) + h * dk + cc);
            } else if (blk == 0) {
              val = f[tok * nqk + h * dk + cc];
            } else if (blk == 1) {
              val = q[tok * nqk + h * dk + cc];
            } else {
              val = k ? k[tok * nqk + h * dk + cc] : 1.f - f[tok * nqk + h * dk + cc];
            }
          }
        } else if (p0 + c - NQ * NB < dv) {
          val = ldf(v + tok * ld_v + h * dv + p0 + c - NQ * NB);
        }
      }
      pre[j] = val;
    }
  };
  auto commit = [&](int buf) {
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int e = threadIdx.x + NTH * j;
      if (e < TT * ROW) {
        float val = pre[j];
        if (RAW) {
          const int c = e % ROW, blk = c / NB, cc = c % NB;
          if (blk < NQ && cc < dk) {
            if (blk == 0) {
              const float l = lower[h * dk + cc];
              val = l + (1.f - l) * sigmoidf(val + (f_bias ? f_bias[h * dk + cc] : 0.f));
            } else {
              val = siluf(val);
            }
          }
        }
        (&stage[buf][0][0])[e] = val;
      }
    }
  };
  fetch(c0);
  commit(0);
  __syncthreads();
  int buf = 0;
  for (int t0 = c0; t0 < c1; t0 += TT, buf ^= 1) {
    const int nt = min(TT, c1 - t0);
    const bool more = t0 + TT < c1;
    if (more) fetch(t0 + TT);
    auto step = [&](int tt) {
      const float* fr = &stage[buf][tt][rg * NI];
      const float* qr = &stage[buf][tt][NB + rg * NI];
      const float* kr = &stage[buf][tt][(NQ - 1) * NB + rg * NI];   // RAW: unused
      const float vv = stage[buf][tt][NQ * NB + col];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        // k = 1 - f:  f S + (1 - f) v = v + f (S - v), one operation less per element
        S[i] = RAW ? fmaf(fr[i], S[i] - vv, vv) : fmaf(fr[i], S[i], kr[i] * vv);
        acc = fmaf(S[i], qr[i], acc);
      }
      if (pass == 1) {   // the chunk's decay product; no outputs in this pass
#pragma unroll
        for (int i = 0; i < NI; ++i) Ap[i] *= fr[i];
        return;
      }
      if (HALVES == 2) acc += __shfl_xor(acc, 32, 64);
      if (lane < COLS) opart[tt][wave][col] = acc;
    };
    if (nt == TT) {  // whole tile: a fixed trip count lets the LDS reads of several steps be in flight together
#pragma unroll 4
      for (int tt = 0; tt < TT; ++tt) step(tt);
    } else {
      for (int tt = 0; tt < nt; ++tt) step(tt);
    }
    __syncthreads();
    for (int e = threadIdx.x; pass != 1 && e < nt * COLS; e += NTH) {
      const int tt = e / COLS, c = e % COLS;
      if (p0 + c < dv) {
        float val = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) val += opart[tt][w][c];
        o[(int64_t)(q0 + t0 + tt) * nv + h * dv + p0 + c] = val;
      }
    }
    if (more) commit(buf ^ 1);
    __syncthreads();
  }
  if (pass == 1) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = rg * NI + i;
      const int64_t cr = ((cs0 + z) * H + h) * dk + n;
      if (pok && n < dk) chB[cr * dv + p] = S[i];
      if (p == 0 && n < dk) chA[cr] = Ap[i];
    }
    return;
  }
  if (pok && c1 == qn) {   // the workgroup that holds the last token
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = rg * NI + i;
      if (n < dk) Sg[(int64_t)n * dv + p] = S[i];
    }
  }
}

// ================================================================== host launchers
void lower_bound_gates(const void* proj, bool f32, int64_t ld, int off_q, int off_f, int n, const float* f_bias,
                       const float* lower, float* q, float* f, int T_, hipStream_t st) {
  if (T_ <= 0 || n <= 0) return;
  const int64_t total = (int64_t)T_ * n;
  XGM_DISPATCH_T(f32, lower_bound_gates_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, st>>>(
                          (const T*)proj, ld, off_q, off_f, n, f_bias, lower, q, f, total);)
}

void decay_gates(const void* proj, bool f32, int64_t ld, int off_q, int off_k, int n, float q_scale, const void* z,
                 int64_t ld_z, const float* z_bias, float inv_tau, float* q, float* f, float* k, int T_, hipStream_t st) {
  if (T_ <= 0 || n <= 0) return;
  const int64_t total = (int64_t)T_ * n;
  XGM_DISPATCH_T(f32, decay_gates_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, st>>>(
                          (const T*)proj, ld, off_q, off_k, n, q_scale, (const T*)z, ld_z, z_bias, inv_tau, q, f, k, total);)
}

int64_t gated_linear_scan_scratch_floats(int T_, int ns, int H, int dk, int dv) {
  const int64_t cslots = T_ / kScanChunk + ns + 1;
  return (cslots * (dv + 1) + (int64_t)ns * dv) * H * dk;
}

int gated_linear_scan(const float* q, const float* f, const float* k, const void* raw, int64_t ld_raw, int off_q, int off_f,
                      const float* f_bias, const float* lower, const void* v, bool v_f32, int64_t ld_v, float* state,
                      const int32_t* qsl, const int32_t* seq_lens, const int32_t* slots, float* o, int ns, int H, int dk,
                      int dv, int cols_hint, float* scratch, int max_q, int T_, hipStream_t st) {
  if (ns <= 0) return 0;
  if (H <= 0 || dk < 1 || dk > 256 || dv < 1 || (raw ? !lower : (!q || !f))) return -1;
  // long portions (scratch given): chunks of kScanChunk tokens over the whole grid, in two launches
  const bool chunked = scratch && max_q > kScanChunk;
  const int nc = chunked ? (max_q + kScanChunk - 1) / kScanChunk : 1;
  const int64_t cslots = T_ / kScanChunk + ns + 1;
  float* chA = scratch;
  float* chB = chunked ? chA + cslots * H * dk : nullptr;
  float* s_in = chunked ? chB + cslots * H * dk * dv : nullptr;
  // 32-column workgroups for small value sizes (no idle lanes), or on request. Doubling the workgroups of a step that
  // leaves compute units idle measured no faster: the scan is bound by the latency of a token step, not by lanes.
  const bool narrow = cols_hint == 32 || (cols_hint != 64 && dv <= 32);
  const int cols = narrow ? 32 : 64;
  dim3 grid(ns * nc, H, (dv + cols - 1) / cols);
#define XGM_GL4(NI, TT, NW, RAW, COLS, PASS)                                                                           \
  gated_linear_scan_kernel<T, NI, TT, NW, RAW, COLS><<<grid, 64 * NW, 0, st>>>(                                         \
      q, f, k, (const T*)raw, ld_raw, off_q, off_f, f_bias, lower, (const T*)v, ld_v, state, qsl, seq_lens, slots, o, H, \
      dk, dv, PASS, nc, chA, chB, s_in);
#define XGM_GL3(NI, TT, NW, RAW, COLS)                                               \
  XGM_DISPATCH_T(v_f32, if (chunked) {                                               \
    XGM_GL4(NI, TT, NW, RAW, COLS, 1)                                                \
    XGM_GL4(NI, TT, NW, RAW, COLS, 2)                                                \
  } else { XGM_GL4(NI, TT, NW, RAW, COLS, 0) })
  // NI rows per lane: the narrow form covers twice the rows per wave, so it takes half of them per lane
#define XGM_GL2(NI, TT, NW, RAW)          \
  if (narrow) {                           \
    XGM_GL3((NI / 2), TT, NW, RAW, 32)    \
  } else {                                \
    XGM_GL3(NI, TT, NW, RAW, 64)          \
  }
  // tokens per staged tile: the raw form stages two row blocks instead of three and takes longer tiles
#define XGM_GL(NI, TT, TTR, NW)           \
  if (raw) {                              \
    XGM_GL2(NI, TTR, NW, true)            \
  } else {                                \
    XGM_GL2(NI, TT, NW, false)            \
  }                                       \
  return 0;
  if (dk <= 16) { XGM_GL(4, 16, 32, 4) }
  if (dk <= 32) { XGM_GL(8, 16, 32, 4) }
  if (dk <= 64) { XGM_GL(8, 8, 16, 8) }
  if (dk <= 128) { XGM_GL(16, 8, 8, 8) }
  XGM_GL(32, 4, 4, 8)
#undef XGM_GL
#undef XGM_GL2
#undef XGM_GL3
#undef XGM_GL4
}

}  // namespace xgm
