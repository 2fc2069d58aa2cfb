// Minimal gated recurrence (minGRU), one state value per channel and sequence slot:
//
//   z = sigmoid(p_z + b_z),  u = p_x + b_x,  c(u) = u + 1/2 (u >= 0), sigmoid(u) (u < 0)
//   S_t = (1 - z_t) S_(t-1) + z_t c(u_t)                 out_t = S_t * silu(p_g)
//
// p_z, p_x, p_g are column blocks of one fused projection row (float or bf16); gate, candidate, the recurrence and
// the state are fp32. Gate and candidate depend on the current token only, so S_t = a_t S_(t-1) + b_t is a linear
// recurrence and a portion of a prompt is scanned in pieces:
//
//   mingru_scan_kernel   workgroup = (sequence, 64 channels), NW waves, lane = channel. Wave w takes the w-th piece
//                        of the sequence's tokens: it first reduces its piece to (A, B) with S_end = A S_start + B,
//                        the pieces meet in LDS, every wave folds the pieces before it onto the carried state (in
//                        order), and then runs its piece again from the right start, writing the outputs.
//   mingru_pieces_kernel / mingru_chunks_kernel   long portions, so that a few sequences still fill the chip:
//                        workgroup = (sequence, 64 channels, chunk of kChunk tokens), wave = piece of kChunk / 16
//                        tokens. The first launch reduces every piece and every chunk to its (A, B) and sets the
//                        sequence's incoming state aside; the second folds the chunks and pieces before its own
//                        onto that state (in order) and runs its piece, writing the outputs and the final state.
//   mingru_step_kernel   steps of single tokens: one thread per (sequence, channel).
#include "mixers_common.h"

namespace xgm {

__device__ __forceinline__ void mingru_terms(float pz, float px, float& z, float& c) {
  z = sigmoidf(pz);
  c = px >= 0.f ? px + 0.5f : sigmoidf(px);
}

template <typename T, typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void mingru_scan_kernel(const T* __restrict__ proj, int64_t ld, int off_z, int off_x,
                                                              int off_g, int n, const float* __restrict__ bz,
                                                              const float* __restrict__ bx, float* __restrict__ state,
                                                              const int32_t* __restrict__ qsl,
                                                              const int32_t* __restrict__ seq_lens,
                                                              const int32_t* __restrict__ slots, TO* __restrict__ out) {
  __shared__ float sa[NW][64], sb[NW][64];
  const int s = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.y * 64 + lane;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (q <= 0) return;
  const bool ok = c < n;
  if (slot < 0) {  // padding rows still get defined outputs
    for (int t = wave; t < q; t += NW)
      if (ok) stf(out + (int64_t)(q0 + t) * n + c, 0.f);
    return;
  }
  const int ctx = seq_lens[s] - q;
  const int per = (q + NW - 1) / NW;
  const int t0 = min(q, wave * per), t1 = min(q, t0 + per);
  const float bzc = (bz && ok) ? bz[c] : 0.f, bxc = (bx && ok) ? bx[c] : 0.f;
  const int cc = ok ? c : 0;
  const T* base = proj + (int64_t)q0 * ld + cc;
  float A = 1.f, B = 0.f;
  if (NW > 1) {
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
      const T* row = base + (int64_t)t * ld;
      float z, cd;
      mingru_terms(ldf(row + off_z) + bzc, ldf(row + off_x) + bxc, z, cd);
      A *= 1.f - z;
      B = (1.f - z) * B + z * cd;
    }
    sa[wave][lane] = A;
    sb[wave][lane] = B;
    __syncthreads();
  }
  float S = (ctx > 0 && ok) ? state[(int64_t)slot * n + c] : 0.f;
  for (int w = 0; w < wave; ++w) S = sa[w][lane] * S + sb[w][lane];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const T* row = base + (int64_t)t * ld;
    float z, cd;
    mingru_terms(ldf(row + off_z) + bzc, ldf(row + off_x) + bxc, z, cd);
    S = (1.f - z) * S + z * cd;
    if (ok) stf(out + (int64_t)(q0 + t) * n + c, S * siluf(ldf(row + off_g)));
  }
  if (ok && t0 < t1 && t1 == q) state[(int64_t)slot * n + c] = S;   // the wave that holds the last token
}

// ---- long portions in two launches. Chunk slot of (sequence s, chunk z): q0_s / kChunk + s + z -- distinct for all
// chunks of a step and below T / kChunk + ns + 1. Scratch (floats): pieces [slots][kPieces][2][n], chunks
// [slots][2][n], incoming state [ns][n].
constexpr int kChunk = 256, kPieces = 16, kPieceLen = kChunk / kPieces;

template <typename T>
__global__ __launch_bounds__(64 * kPieces) void mingru_pieces_kernel(const T* __restrict__ proj, int64_t ld, int off_z,
                                                                     int off_x, int n, const float* __restrict__ bz,
                                                                     const float* __restrict__ bx,
                                                                     const float* __restrict__ state,
                                                                     const int32_t* __restrict__ qsl,
                                                                     const int32_t* __restrict__ seq_lens,
                                                                     const int32_t* __restrict__ slots,
                                                                     float* __restrict__ pieces, float* __restrict__ chunks,
                                                                     float* __restrict__ s_in) {
  __shared__ float sa[kPieces][64], sb[kPieces][64];
  const int s = blockIdx.x, z = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.y * 64 + lane;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || z * kChunk >= q) return;
  const bool ok = c < n;
  const int cc = ok ? c : 0;
  const int64_t cs = q0 / kChunk + s + z;
  if (z == 0 && wave == 0 && ok) s_in[(int64_t)s * n + c] = seq_lens[s] - q > 0 ? state[(int64_t)slot * n + c] : 0.f;
  const int t0 = min(q, z * kChunk + wave * kPieceLen), t1 = min(q, t0 + kPieceLen);
  const float bzc = (bz && ok) ? bz[c] : 0.f, bxc = (bx && ok) ? bx[c] : 0.f;
  const T* base = proj + (int64_t)q0 * ld + cc;
  float A = 1.f, B = 0.f;
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const T* row = base + (int64_t)t * ld;
    float zz, cd;
    mingru_terms(ldf(row + off_z) + bzc, ldf(row + off_x) + bxc, zz, cd);
    A *= 1.f - zz;
    B = (1.f - zz) * B + zz * cd;
  }
  if (ok) {
    float* pp = pieces + ((cs * kPieces + wave) * 2) * n + c;
    pp[0] = A;
    pp[n] = B;
  }
  sa[wave][lane] = A;
  sb[wave][lane] = B;
  __syncthreads();
  if (wave == 0 && ok) {   // the chunk as a whole, its pieces folded in order
    float At = 1.f, Bt = 0.f;
#pragma unroll
    for (int w = 0; w < kPieces; ++w) {
      Bt = sa[w][lane] * Bt + sb[w][lane];
      At *= sa[w][lane];
    }
    chunks[(cs * 2) * n + c] = At;
    chunks[(cs * 2 + 1) * n + c] = Bt;
  }
}

template <typename T, typename TO>
__global__ __launch_bounds__(64 * kPieces) void mingru_chunks_kernel(const T* __restrict__ proj, int64_t ld, int off_z,
                                                                     int off_x, int off_g, int n,
                                                                     const float* __restrict__ bz,
                                                                     const float* __restrict__ bx, float* __restrict__ state,
                                                                     const int32_t* __restrict__ qsl,
                                                                     const int32_t* __restrict__ slots,
                                                                     const float* __restrict__ pieces,
                                                                     const float* __restrict__ chunks,
                                                                     const float* __restrict__ s_in, TO* __restrict__ out) {
  const int s = blockIdx.x, z = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = blockIdx.y * 64 + lane;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (z * kChunk >= q || c >= n) return;
  const int t0 = min(q, z * kChunk + wave * kPieceLen), t1 = min(q, t0 + kPieceLen);
  if (slot < 0) {  // padding rows still get defined outputs
    for (int t = t0; t < t1; ++t) stf(out + (int64_t)(q0 + t) * n + c, 0.f);
    return;
  }
  const int64_t cs0 = q0 / kChunk + s;
  float S = s_in[(int64_t)s * n + c];
  for (int zc = 0; zc < z; ++zc) S = chunks[((cs0 + zc) * 2) * n + c] * S + chunks[((cs0 + zc) * 2 + 1) * n + c];
  for (int w = 0; w < wave; ++w) {
    const float* pp = pieces + (((cs0 + z) * kPieces + w) * 2) * n + c;
    S = pp[0] * S + pp[n];
  }
  const float bzc = bz ? bz[c] : 0.f, bxc = bx ? bx[c] : 0.f;
  const T* base = proj + (int64_t)q0 * ld + c;
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const T* row = base + (int64_t)t * ld;
    float zz, cd;
    mingru_terms(ldf(row + off_z) + bzc, ldf(row + off_x) + bxc, zz, cd);
    S = (1.f - zz) * S + zz * cd;
    stf(out + (int64_t)(q0 + t) * n + c, S * siluf(ldf(row + off_g)));
  }
  if (t0 < t1 && t1 == q) state[(int64_t)slot * n + c] = S;   // the piece that holds the last token
}

template <typename T, typename TO>
__global__ __launch_bounds__(256) void mingru_step_kernel(const T* __restrict__ proj, int64_t ld, int off_z, int off_x,
                                                          int off_g, int n, const float* __restrict__ bz,
                                                          const float* __restrict__ bx, float* __restrict__ state,
                                                          const int32_t* __restrict__ qsl,
                                                          const int32_t* __restrict__ seq_lens,
                                                          const int32_t* __restrict__ slots, TO* __restrict__ out) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (q <= 0 || c >= n) return;
  if (slot < 0) {
    stf(out + (int64_t)q0 * n + c, 0.f);
    return;
  }
  const T* row = proj + (int64_t)q0 * ld + c;
  float z, cd;
  mingru_terms(ldf(row + off_z) + (bz ? bz[c] : 0.f), ldf(row + off_x) + (bx ? bx[c] : 0.f), z, cd);
  float* sp = state + (int64_t)slot * n + c;
  const float S0 = seq_lens[s] - q > 0 ? *sp : 0.f;
  const float S = (1.f - z) * S0 + z * cd;
  *sp = S;
  stf(out + (int64_t)q0 * n + c, S * siluf(ldf(row + off_g)));
}

int64_t mingru_scratch_floats(int T_, int ns, int n) {
  const int64_t cslots = T_ / kChunk + ns + 1;
  return (cslots * (kPieces + 1) * 2 + ns) * (int64_t)n;
}

int mingru_scan(const void* proj, bool f32, int64_t ld, int off_z, int off_x, int off_g, int n, const float* bz,
                const float* bx, float* state, const int32_t* qsl, const int32_t* seq_lens, const int32_t* slots, void* out,
                bool out_f32, int ns, int max_q, float* scratch, int T_, hipStream_t st) {
  if (ns <= 0 || max_q <= 0) return 0;
  if (n < 1 || f32 != out_f32) return -1;
  if (scratch && max_q > kChunk) {   // long portions: pieces and chunks over the whole grid
    const int64_t cslots = T_ / kChunk + ns + 1;
    float* pieces = scratch;
    float* chunks = pieces + cslots * kPieces * 2 * n;
    float* s_in = chunks + cslots * 2 * n;
    dim3 grid(ns, (n + 63) / 64, (max_q + kChunk - 1) / kChunk);
    XGM_DISPATCH_T(f32, mingru_pieces_kernel<T><<<grid, 64 * kPieces, 0, st>>>((const T*)proj, ld, off_z, off_x, n, bz, bx,
                                                                               state, qsl, seq_lens, slots, pieces, chunks,
                                                                               s_in);
                   mingru_chunks_kernel<T, T><<<grid, 64 * kPieces, 0, st>>>((const T*)proj, ld, off_z, off_x, off_g, n, bz,
                                                                             bx, state, qsl, slots, pieces, chunks, s_in,
                                                                             (T*)out);)
    return 0;
  }
  if (max_q == 1) {
    dim3 grid((n + 255) / 256, ns);
    XGM_DISPATCH_T(f32, mingru_step_kernel<T, T><<<grid, 256, 0, st>>>((const T*)proj, ld, off_z, off_x, off_g, n, bz, bx,
                                                                        state, qsl, seq_lens, slots, (T*)out);)
    return 0;
  }
  dim3 grid(ns, (n + 63) / 64);
#define XGM_MG(NW)                                                                                                      \
  XGM_DISPATCH_T(f32, mingru_scan_kernel<T, T, NW><<<grid, 64 * NW, 0, st>>>((const T*)proj, ld, off_z, off_x, off_g, n, \
                                                                             bz, bx, state, qsl, seq_lens, slots,       \
                                                                             (T*)out);)
  if (max_q <= 16) { XGM_MG(1) } else if (max_q <= 128) { XGM_MG(4) } else { XGM_MG(16) }
#undef XGM_MG
  return 0;
}

}  // namespace xgm
