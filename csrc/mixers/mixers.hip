// Sequence-mixer kernels for stateful / latent-cache decoder layers (gfx950, wave64).
//
// One ragged step is [tokens of sequence 0 | tokens of sequence 1 | ...]; a sequence is
// described by qsl[s] (first row), seq_lens[s] (tokens held after this step) and
// slots[s] (its row in every per-sequence state tensor, < 0 = padding row). A sequence
// whose context is empty (seq_len == q_len) starts from zero state whatever its slot
// holds, so a slot needs no clearing when it is handed to another request.
//
//   embed_rows          token ids -> fp32 residual rows
//   canon_conv          h + causal depthwise conv over time, carried by [taps-1] rows of state
//   scaled_add_rmsnorm  x <- rmsnorm(alpha * x + y + bias) * (offset + w)   (fp32 residual)
//   latent_prep         query latent norm; key/value latent norm + rotated shared key -> paged latent cache
//   latent_attention    windowed softmax attention in latent space (all heads share the cached rows)
//   delta_scan          S <- diag(w) S - (a u)(u^T S) + k v^T ; o = S^T r   (fp32 state per slot)
//   delta_out           per-head unit-rms, weight and sigmoid gate
//   xielu, tanh_cols    activations
//
// Activations / caches are T = float or bf16 (raw uint16_t); everything the recurrences,
// norms, softmax and rotations touch is fp32.
#include "mixers_common.h"

#include <algorithm>

namespace xgm {

// ------------------------------------------------------------------ embedding
// out = table[id] * scale; pos_table != nullptr: + pos_table[positions[t]] (a learned vector per position, unscaled;
// rows outside the table add nothing)
template <typename TW>
__global__ void embed_rows_kernel(const int32_t* __restrict__ ids, const TW* __restrict__ table, float* __restrict__ out,
                                  int W, int V, const TW* __restrict__ pos_table, const int32_t* __restrict__ positions,
                                  int P, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const int p = pos_table ? positions[t] : -1;
  const bool pk = p >= 0 && p < P;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = ok ? ldf(table + (int64_t)id * W + c) * scale : 0.f;
    if (pk) v += ldf(pos_table + (int64_t)p * W + c);
    out[(int64_t)t * W + c] = v;
  }
}

// ------------------------------------------------------------------ causal conv with carried inputs
constexpr int kMaxTaps = 8;

// state[slot][k][c], k in [0, taps-1): the input at position ctx - (taps-1) + k (zero before the start).
// x is row-strided (ld_in) and float or bf16; out_t = [x_t if residual] + bias + sum_j w[:, j] x_(t-taps+1+j),
// through silu when `act`; the state keeps raw inputs in fp32.
template <typename TI, typename TO>
__global__ void canon_conv_kernel(const TI* __restrict__ x, int64_t ld_in, const float* __restrict__ w,
                                  const float* __restrict__ bias, float* __restrict__ state,
                                  const int32_t* __restrict__ qsl, const int32_t* __restrict__ seq_lens,
                                  const int32_t* __restrict__ slots, TO* __restrict__ out, int W, int taps, int tile,
                                  int write_state, int residual, int act) {
  const int s = blockIdx.z;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int t0 = blockIdx.y * tile;
  if (t0 >= q) return;
  const int t1 = min(q, t0 + tile);
  const int ctx = seq_lens[s] - q;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int nh = taps - 1;
  float hist[kMaxTaps - 1], wt[kMaxTaps];
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) wt[j] = j < taps ? w[(int64_t)c * taps + j] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  float* st = state + ((int64_t)slot * nh) * W + c;
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j) {
    float v = 0.f;
    if (j < nh) {
      const int li = t0 - nh + j;  // local index of the input this tap history starts with
      if (li >= 0) v = ldf(x + (int64_t)(q0 + li) * ld_in + c);
      else if (ctx + li >= 0) v = st[(int64_t)(nh + li) * W];
    }
    hist[j] = v;
  }
  for (int t = t0; t < t1; ++t) {
    const float cur = ldf(x + (int64_t)(q0 + t) * ld_in + c);
    float acc = (residual ? cur : 0.f) + b;
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j)
      if (j < nh) acc += wt[j] * hist[j];
    acc += wt[nh] * cur;
    if (act) acc = siluf(acc);
    stf(out + (int64_t)(q0 + t) * W + c, acc);
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j) {  // shift; the newest input goes last
      const float nxt = j + 1 < kMaxTaps - 1 ? hist[j + 1] : 0.f;
      hist[j] = j == nh - 1 ? cur : nxt;
    }
  }
  if (write_state) {
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j)
      if (j < nh) st[(int64_t)j * W] = hist[j];
  }
}

// the carried rows after a step whose sequences were convolved by several tiles
template <typename TI>
__global__ void canon_state_kernel(const TI* __restrict__ x, int64_t ld_in, float* __restrict__ state,
                                   const int32_t* __restrict__ qsl, const int32_t* __restrict__ seq_lens,
                                   const int32_t* __restrict__ slots, int W, int taps) {
  const int s = blockIdx.y;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int ctx = seq_lens[s] - q;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int nh = taps - 1;
  float* st = state + ((int64_t)slot * nh) * W + c;
  float v[kMaxTaps - 1];
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j) {
    v[j] = 0.f;
    if (j < nh) {
      const int li = q - nh + j;
      if (li >= 0) v[j] = ldf(x + (int64_t)(q0 + li) * ld_in + c);
      else if (ctx + li >= 0) v[j] = st[(int64_t)(nh + li) * W];
    }
  }
#pragma unroll
  for (int j = 0; j < kMaxTaps - 1; ++j)
    if (j < nh) st[(int64_t)j * W] = v[j];
}

// ------------------------------------------------------------------ norm after the (scaled) residual sum
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void scaled_add_rmsnorm_kernel(const float* x, const TY* __restrict__ y,
                                                                 int64_t y_stride, const float* __restrict__ bias,
                                                                 float alpha, const float* __restrict__ w, float w_offset,
                                                                 float eps, float* x_out,
                                                                 TO* __restrict__ out, int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const float* xr = x + (int64_t)t * W;
  const TY* yr = y ? y + (int64_t)t * y_stride : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = alpha * xr[c];
    if (yr) v += ldf(yr + c);
    if (bias) v += bias[c];
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = alpha * xr[c];
    if (yr) v += ldf(yr + c);
    if (bias) v += bias[c];
    const float o = v * r * (w_offset + w[c]);
    if (x_out) x_out[(int64_t)t * W + c] = o;
    if (out) stf(out + (int64_t)t * W + c, o);
  }
}

// one pass, 4 elements per access: W % 4 == 0, W <= 1024 NV, y rows 8-byte aligned
template <typename TY, typename TO, int NV>
__global__ __launch_bounds__(256) void scaled_add_rmsnorm_vec_kernel(const float* x, const TY* __restrict__ y,
                                                                     int64_t y_stride, const float* __restrict__ bias,
                                                                     float alpha, const float* __restrict__ w,
                                                                     float w_offset, float eps, float* x_out,
                                                                     TO* __restrict__ out, int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  float v[NV][4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = 4 * (threadIdx.x + 256 * j);
    if (c < W) {
      ld4(x + (int64_t)t * W + c, v[j]);
      float a[4] = {0.f, 0.f, 0.f, 0.f}, b[4] = {0.f, 0.f, 0.f, 0.f};
      if (y) ld4(y + (int64_t)t * y_stride + c, a);
      if (bias) ld4(bias + c, b);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[j][e] = alpha * v[j][e] + a[e] + b[e];
        ss += v[j][e] * v[j][e];
      }
    }
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = 4 * (threadIdx.x + 256 * j);
    if (c < W) {
      float g[4], res[4];
      ld4(w + c, g);
#pragma unroll
      for (int e = 0; e < 4; ++e) res[e] = v[j][e] * r * (w_offset + g[e]);
      if (x_out) st4(x_out + (int64_t)t * W + c, res);
      if (out) st4(out + (int64_t)t * W + c, res);
    }
  }
}

// ------------------------------------------------------------------ latent attention: projections -> cache
// proj row: [.. | q latent (Rq) at off_q | kv latent (R) + shared rotary key (rd) at off_kv | ..]
// rot table: [positions][rot_dims/2][2] = (cos, sin) of position * base^(-2i/rot_dims)
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ proj, int64_t ld, int off_q, int Rq,
                                                          int off_kv, int R, int rd, const float* __restrict__ wq,
                                                          const float* __restrict__ wkv, float eps,
                                                          const int32_t* __restrict__ positions,
                                                          const int32_t* __restrict__ slot_mapping,
                                                          const float* __restrict__ rot, int rot_dims,
                                                          T* __restrict__ cq, T* __restrict__ cache) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = proj + (int64_t)t * ld;
  {
    float ss = 0.f;
    for (int i = threadIdx.x; i < Rq; i += blockDim.x) {
      const float v = ldf(row + off_q + i);
      ss += v * v;
    }
    ss = block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)Rq + eps);
    for (int i = threadIdx.x; i < Rq; i += blockDim.x) stf(cq + (int64_t)t * Rq + i, ldf(row + off_q + i) * r * wq[i]);
  }
  if (off_kv < 0) return;
  const int slot = slot_mapping[t];
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ldf(row + off_kv + i);
    ss += v * v;
  }
  ss = block_sum(ss, red);
  if (slot < 0) return;
  const float r = 1.f / sqrtf(ss / (float)R + eps);
  T* dst = cache + (int64_t)slot * (R + rd);
  for (int i = threadIdx.x; i < R; i += blockDim.x) stf(dst + i, ldf(row + off_kv + i) * r * wkv[i]);
  const int pos = positions[t];
  const int half = rot_dims >> 1;
  const T* kr = row + off_kv + R;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float c = rot[((int64_t)pos * half + i) * 2], s = rot[((int64_t)pos * half + i) * 2 + 1];
    const float u = ldf(kr + 2 * i), v = ldf(kr + 2 * i + 1);
    stf(dst + R + 2 * i, u * c - v * s);
    stf(dst + R + 2 * i + 1, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < rd; i += blockDim.x) stf(dst + R + i, ldf(kr + i));
}

// ------------------------------------------------------------------ latent attention over the paged latent cache
// Every head scores the same cached row [kv latent (R) | rotated key (rd)]: the query is
// [W_uk^T q_unrotated (R) | rotated q (rd)], the value is the latent itself, and the
// per-head value projection follows as a GEMM. One workgroup = one token x kHPB heads;
// a tile of KT keys is staged in LDS once and read by all its heads.
constexpr int kHPB = 8;  // heads per workgroup (4 waves x 2)

template <typename T, int NR>
__global__ __launch_bounds__(256) void latent_attention_kernel(
    const T* __restrict__ qabs, const T* __restrict__ q, int64_t q_stride, int dq, int dn, const T* __restrict__ gate,
    int64_t gate_stride, const T* __restrict__ cache, const int32_t* __restrict__ block_tables, int bt_width, int bs,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq, const float* __restrict__ rot,
    int rot_dims, T* __restrict__ out, int Ttot, int H, int R, int rd, int window, float scale, int KT) {
  extern __shared__ float smem[];
  const int Dk = R + rd, ldt = Dk + 1;
  float* tile = smem;                      // [KT][Dk + 1]
  float* qs = smem + (size_t)KT * ldt;     // [kHPB][Dk]
  const int t = blockIdx.x, hb = blockIdx.y * kHPB;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int s = token_seq[t];
  if (s < 0) {
    for (int hl = wave; hl < kHPB && hb + hl < H; hl += 4)
      for (int d = lane; d < R; d += 64) stf(out + ((int64_t)(hb + hl) * Ttot + t) * R + d, 0.f);
    return;
  }
  const int pos = positions[t];
  const int j0 = max(0, pos - window + 1);
  // queries of this workgroup's heads -> LDS (scaled; rotated part rotated here)
  const int half = rot_dims >> 1;
  for (int hl = wave; hl < kHPB; hl += 4) {
    const int h = hb + hl;
    float* qh = qs + hl * Dk;
    if (h >= H) {
      for (int d = lane; d < Dk; d += 64) qh[d] = 0.f;
      continue;
    }
    for (int d = lane; d < R; d += 64) qh[d] = ldf(qabs + ((int64_t)h * Ttot + t) * R + d) * scale;
    const T* qr = q + (int64_t)t * q_stride + (int64_t)h * dq + dn;
    for (int i = lane; i < half; i += 64) {
      const float c = rot[((int64_t)pos * half + i) * 2], sn = rot[((int64_t)pos * half + i) * 2 + 1];
      const float u = ldf(qr + 2 * i), v = ldf(qr + 2 * i + 1);
      qh[R + 2 * i] = (u * c - v * sn) * scale;
      qh[R + 2 * i + 1] = (v * c + u * sn) * scale;
    }
    for (int i = rot_dims + lane; i < rd; i += 64) qh[R + i] = ldf(qr + i) * scale;
  }
  const int LPK = 64 / KT;  // lanes per key in the score phase
  const int kj = lane / LPK, part = lane % LPK;
  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  float acc[2][NR];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[a][i] = 0.f;
  const int32_t* bt = block_tables + (int64_t)s * bt_width;
  for (int k0 = j0; k0 <= pos; k0 += KT) {
    const int n = min(KT, pos - k0 + 1);
    __syncthreads();  // the previous tile is consumed (and qs is written, on the first pass)
    for (int jj = wave; jj < n; jj += 4) {
      const int key = k0 + jj;
      const T* src = cache + ((int64_t)bt[key / bs] * bs + key % bs) * Dk;
      for (int d = lane; d < Dk; d += 64) tile[jj * ldt + d] = ldf(src + d);
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      const int hl = wave + 4 * a;
      if (hb + hl >= H) continue;
      const float* qh = qs + hl * Dk;
      float sc = 0.f;
      if (kj < n) {
        const float* kr = tile + kj * ldt;
        for (int d = part; d < Dk; d += LPK) sc += qh[d] * kr[d];
      }
      for (int o = 1; o < LPK; o <<= 1) sc += __shfl_xor(sc, o, 64);
      if (kj >= n) sc = -INFINITY;
      const float mn = fmaxf(m[a], wave_max(sc));
      const float p = kj < n ? expf(sc - mn) : 0.f;
      const float corr = m[a] == -INFINITY ? 0.f : expf(m[a] - mn);
      l[a] = l[a] * corr + wave_sum(part == 0 ? p : 0.f);
      m[a] = mn;
#pragma unroll
      for (int i = 0; i < NR; ++i) acc[a][i] *= corr;
      for (int j = 0; j < n; ++j) {
        const float pj = __shfl(p, j * LPK, 64);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int d = lane + 64 * i;
          if (d < R) acc[a][i] += pj * tile[j * ldt + d];
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int h = hb + wave + 4 * a;
    if (h >= H) continue;
    const float g = sigmoidf(ldf(gate + (int64_t)t * gate_stride + h)) / l[a];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = lane + 64 * i;
      if (d < R) stf(out + ((int64_t)h * Ttot + t) * R + d, acc[a][i] * g);
    }
  }
}

// ---- MFMA form (bf16 activations / cache; R % 16 == 0, rd % 8 == 0)
// One wave = 16 query slots: 16 tokens of one head (prompt portions) or one token of up to
// 16 heads (single-token rows); a workgroup's 4 waves take 4 heads (or head tiles) of the same
// tokens and share each staged tile of 64 cached rows. S^T = K . Q^T on
// v_mfma_f32_16x16x32_bf16 (a lane owns one query's scores), whose accumulator is, packed,
// the B operand of O^T += V^T . P^T; V^T fragments are transposed LDS reads of the same tile.
constexpr int kKT = 64;

template <int NMT_MAX, bool SPLIT, int WPE>
__global__ __launch_bounds__(256, WPE) void latent_attention_mfma_kernel(
    const bf16* __restrict__ qabs, const bf16* __restrict__ q, int dq, int dn, const bf16* __restrict__ gate,
    int64_t gate_stride, const bf16* __restrict__ cache, const int32_t* __restrict__ block_tables, int bt_width, int bs,
    const int32_t* __restrict__ qsl, const int32_t* __restrict__ seq_lens, const int32_t* __restrict__ slots,
    const float* __restrict__ rot, int rot_dims, bf16* __restrict__ out, int Ttot, int H, int R, int rd, int window,
    float scale, int TPT, int HPT, int nsplit_arg, float* __restrict__ part_o, float* __restrict__ part_ml) {
  constexpr int NKK_MAX = NMT_MAX / 2 + 4;
  const int nsplit = SPLIT ? nsplit_arg : 1;  // prompt portions compile the key shares out (registers -> occupancy)
  extern __shared__ __attribute__((aligned(16))) uint16_t tile_lds[];
  const int Dk = R + rd, nkk = (Dk + 31) >> 5, nmt = R >> 4, LDK = nkk * 32 + 8;
  const int s = blockIdx.y;
  const int q0 = qsl[s], qn = qsl[s + 1] - q0;
  if (slots[s] < 0 || qn <= 0) return;
  // nsplit > 1 (single-token steps): blockIdx.x is a share of the window's key tiles, merged by
  // latent_attention_combine_kernel; else it is the tile of TPT tokens
  const int t0 = nsplit > 1 ? 0 : blockIdx.x * TPT;
  if (t0 >= qn) return;
  const int ctx = seq_lens[s] - qn;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, g = lane >> 4;
  const int h0 = (blockIdx.z * 4 + wave) * HPT;
  const bool wave_on = h0 < H;
  const int tl = li / HPT, head = h0 + li % HPT, tok = t0 + tl;
  const bool valid = wave_on && tl < TPT && tok < qn && head < H;
  const int pos_q = ctx + tok;
  int pos_last = ctx + min(qn, t0 + TPT) - 1;
  int kmin = max(0, ctx + t0 - window + 1);
  if (nsplit > 1) {
    const int tiles = (pos_last - kmin + kKT) / kKT, per = (tiles + nsplit - 1) / nsplit;
    kmin += blockIdx.x * per * kKT;
    pos_last = min(pos_last, kmin + per * kKT - 1);  // may leave this share empty
  }
  const int32_t* bt = block_tables + (int64_t)s * bt_width;

  // this lane's query slot as B fragments: [W_uk^T q (R) | rotated q (rd)], 8 dims at 32 kk + 8 g
  xgk::bf16x8_t qf[NKK_MAX];
  const int half = rot_dims >> 1;
#pragma unroll
  for (int kk = 0; kk < NKK_MAX; ++kk) {
    uint4 v = make_uint4(0, 0, 0, 0);
    const int d0 = kk * 32 + g * 8;
    if (kk < nkk && valid && d0 < Dk) {
      if (d0 < R) {
        v = xgk::ld16(qabs + ((int64_t)head * Ttot + q0 + tok) * R + d0);
      } else {
        const int i0 = d0 - R;
        const bf16* src = q + ((int64_t)(q0 + tok) * H + head) * dq + dn + i0;
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float a = bf2f(src[e]), b = bf2f(src[e + 1]);
          if (i0 + e < rot_dims) {
            const int pi = (i0 + e) >> 1;
            const float c = rot[((int64_t)pos_q * half + pi) * 2], sn = rot[((int64_t)pos_q * half + pi) * 2 + 1];
            f[e] = a * c - b * sn;
            f[e + 1] = b * c + a * sn;
          } else {
            f[e] = a;
            f[e + 1] = b;
          }
        }
        v = xgk::pack8(f);
      }
    }
    qf[kk] = xgk::as_frag(v);
  }

  xgk::f32x4_t o[NMT_MAX];
#pragma unroll
  for (int mt = 0; mt < NMT_MAX; ++mt) o[mt] = xgk::f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  // staging: thread -> (row = tid / 4, quarter = tid % 4) takes the row's 16-byte chunks quarter, quarter + 4, ..
  // (4 nkk chunks per row, zero padded to 32 nkk dims): one page lookup per thread and tile, all loads of a
  // tile in flight together; latency is hidden by the other workgroups of the SIMD (two waves per SIMD up to a
  // latent size of 256), single-token steps get them from the key shares
  const int srow = threadIdx.x >> 2, squad = threadIdx.x & 3;
  uint4 stage[NKK_MAX];
  auto fetch = [&](int k0) {
    const int kabs = k0 + srow;
    const bool ok = kabs <= pos_last;
    const bf16* src = ok ? cache + ((int64_t)bt[kabs / bs] * bs + kabs % bs) * Dk : cache;
#pragma unroll
    for (int it = 0; it < NKK_MAX; ++it) {
      const int ch = squad + 4 * it;
      stage[it] = (it < nkk && ok && ch * 8 < Dk) ? xgk::ld16(src + ch * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int it = 0; it < NKK_MAX; ++it)
      if (it < nkk) xgk::st16(tile_lds + srow * LDK + (squad + 4 * it) * 8, stage[it]);
  };
  for (int k0 = kmin; k0 <= pos_last; k0 += kKT) {
    __syncthreads();
    fetch(k0);
    commit();
    __syncthreads();
    if (!wave_on) continue;
    xgk::f32x4_t sacc[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      sacc[n] = xgk::f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NKK_MAX; ++kk)
        if (kk < nkk)
          sacc[n] = xgk::mfma16x16x32(xgk::as_frag(xgk::ld16(tile_lds + (n * 16 + li) * LDK + kk * 32 + g * 8)), qf[kk],
                                      sacc[n]);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kabs = k0 + n * 16 + g * 4 + r;
        float v = sacc[n][r] * scale;
        if (!valid || kabs > pos_q || kabs <= pos_q - window) v = -INFINITY;
        sacc[n][r] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float alpha = m_new == -INFINITY ? 1.f : __expf(m - m_new);
    float rs = 0.f;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = m_new == -INFINITY ? 0.f : __expf(sacc[n][r] - m_new);
        sacc[n][r] = p;
        rs += p;
      }
    rs += __shfl_xor(rs, 16, 64);
    rs += __shfl_xor(rs, 32, 64);
    l = l * alpha + rs;
    m = m_new;
#pragma unroll
    for (int mt = 0; mt < NMT_MAX; ++mt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[mt][r] *= alpha;
    // O^T += V^T . P^T over two 32-key chunks (keys in the order the score accumulator holds them)
#pragma unroll
    for (int sc = 0; sc < 2; ++sc) {
      uint4 pb;
      pb.x = xgk::pack2(sacc[2 * sc][0], sacc[2 * sc][1]);
      pb.y = xgk::pack2(sacc[2 * sc][2], sacc[2 * sc][3]);
      pb.z = xgk::pack2(sacc[2 * sc + 1][0], sacc[2 * sc + 1][1]);
      pb.w = xgk::pack2(sacc[2 * sc + 1][2], sacc[2 * sc + 1][3]);
      const xgk::bf16x8_t pfrag = xgk::as_frag(pb);
      const int qq = li >> 2, pp = li & 3;
      const int r0 = sc * 32 + 4 * g + qq, r1 = r0 + 16;
#pragma unroll
      for (int mt = 0; mt < NMT_MAX; ++mt)
        if (mt < nmt) {
          const xgk::bf16x4_t a0 = xgk::lds_read_tr16(tile_lds + r0 * LDK + mt * 16 + 4 * pp);
          const xgk::bf16x4_t a1 = xgk::lds_read_tr16(tile_lds + r1 * LDK + mt * 16 + 4 * pp);
          const xgk::bf16x8_t vfrag = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
          o[mt] = xgk::mfma16x16x32(vfrag, pfrag, o[mt]);
        }
    }
  }
  if (valid && nsplit > 1) {  // unnormalised share: (m, l) and the weighted latent sum
    const int64_t row = ((int64_t)blockIdx.x * H + head) * Ttot + q0 + tok;
    if (g == 0) {
      part_ml[2 * row] = m;
      part_ml[2 * row + 1] = l;
    }
#pragma unroll
    for (int mt = 0; mt < NMT_MAX; ++mt)
      if (mt < nmt)
        *reinterpret_cast<float4*>(part_o + row * R + mt * 16 + 4 * g) = make_float4(o[mt][0], o[mt][1], o[mt][2], o[mt][3]);
  } else if (valid) {
    const float gl = sigmoidf(bf2f(gate[(int64_t)(q0 + tok) * gate_stride + head])) * (l > 0.f ? 1.f / l : 0.f);
    bf16* op = out + ((int64_t)head * Ttot + q0 + tok) * R;
#pragma unroll
    for (int mt = 0; mt < NMT_MAX; ++mt)
      if (mt < nmt) {
        uint2 w;
        w.x = xgk::pack2(o[mt][0] * gl, o[mt][1] * gl);
        w.y = xgk::pack2(o[mt][2] * gl, o[mt][3] * gl);
        *reinterpret_cast<uint2*>(op + mt * 16 + 4 * g) = w;
      }
  }
}

// merge the key shares of a single-token step: out = sum_s e^(m_s - M) o_s / sum_s e^(m_s - M) l_s, gated
__global__ void latent_attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                const bf16* __restrict__ gate, int64_t gate_stride,
                                                const int32_t* __restrict__ slots, bf16* __restrict__ out, int Ttot, int H,
                                                int R, int nsplit) {
  const int t = blockIdx.x, h = blockIdx.y;
  if (slots[t] < 0) return;  // single-token steps: row t is sequence t
  float M = -INFINITY;
  for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, part_ml[2 * (((int64_t)sp * H + h) * Ttot + t)]);
  float L = 0.f;
  for (int sp = 0; sp < nsplit; ++sp) {
    const int64_t row = ((int64_t)sp * H + h) * Ttot + t;
    const float ms = part_ml[2 * row];
    if (ms != -INFINITY) L += __expf(ms - M) * part_ml[2 * row + 1];
  }
  const float gl = sigmoidf(bf2f(gate[(int64_t)t * gate_stride + h])) * (L > 0.f ? 1.f / L : 0.f);
  for (int d = 4 * threadIdx.x; d < R; d += 4 * blockDim.x) {  // R % 16 == 0
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < nsplit; ++sp) {
      const int64_t row = ((int64_t)sp * H + h) * Ttot + t;
      const float ms = part_ml[2 * row];
      if (ms != -INFINITY) {
        const float e = __expf(ms - M);
        float v[4];
        ld4(part_o + row * R + d, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += e * v[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= gl;
    st4(out + ((int64_t)h * Ttot + t) * R + d, acc);
  }
}

// ------------------------------------------------------------------ generalized delta rule
// One workgroup = (head, sequence); thread (col, ks) owns rows ks, ks + 4, .. of column col
// of the [D x D] state, so u^T S and S^T r reduce over 4 neighbouring lanes only.
constexpr int kKS = 4;

template <typename T, int MAXR>
__global__ void delta_scan_kernel(const T* __restrict__ proj, int64_t ld, int off_r, int off_k, int off_v, int off_a,
                                  const T* __restrict__ wl, int64_t ld_wl, const float* __restrict__ a_bias,
                                  const float* __restrict__ w0, float* __restrict__ state,
                                  const int32_t* __restrict__ qsl, const int32_t* __restrict__ seq_lens,
                                  const int32_t* __restrict__ slots, float* __restrict__ o, int H, int D) {
  const int h = blockIdx.x, s = blockIdx.y;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int ctx = seq_lens[s] - q;
  const int col = threadIdx.x / kKS, ks = threadIdx.x % kKS;
  const bool live = col < D;
  const int cc = live ? col : 0;
  float S[MAXR], ab[MAXR], wb[MAXR];
  float* st = state + ((int64_t)slot * H + h) * D * D;
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    const int i = ks + kKS * r;
    const bool ok = i < D;
    S[r] = (ok && ctx > 0) ? st[(int64_t)i * D + cc] : 0.f;
    ab[r] = ok ? a_bias[h * D + i] : 0.f;
    wb[r] = ok ? w0[h * D + i] : 0.f;
  }
  const int HD = H * D;
  for (int t = 0; t < q; ++t) {
    const T* row = proj + (int64_t)(q0 + t) * ld + h * D;
    const T* wrow = wl + (int64_t)(q0 + t) * ld_wl + h * D;
    float kk[MAXR], ksq = 0.f;
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int i = ks + kKS * r;
      kk[r] = i < D ? ldf(row + off_k + i) : 0.f;
      ksq += kk[r] * kk[r];
    }
    ksq += __shfl_xor(ksq, 1, 64);
    ksq += __shfl_xor(ksq, 2, 64);
    const float inv = 1.f / sqrtf(ksq + 1e-6f);
    float uS = 0.f;
#pragma unroll
    for (int r = 0; r < MAXR; ++r) uS += kk[r] * inv * S[r];
    uS += __shfl_xor(uS, 1, 64);
    uS += __shfl_xor(uS, 2, 64);
    const float v = ldf(row + off_v + cc);
    float ot = 0.f;
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int i = ks + kKS * r;
      if (i < D) {
        const float u = kk[r] * inv;
        const float w = expf(-0.6065306597126334f * sigmoidf(ldf(wrow + i) + wb[r]));
        const float a = sigmoidf(ldf(row + off_a + i) + ab[r]);
        S[r] = w * S[r] - a * u * uS + kk[r] * v;
        ot += S[r] * ldf(row + off_r + i);
      }
    }
    ot += __shfl_xor(ot, 1, 64);
    ot += __shfl_xor(ot, 2, 64);
    if (live && ks == 0) o[(int64_t)(q0 + t) * HD + h * D + col] = ot;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int i = ks + kKS * r;
      if (i < D) st[(int64_t)i * D + col] = S[r];
    }
  }
}

// ---- two-pass form: everything that does not depend on the state (decay, removal rate,
// unit key) is computed once per (token, head) by a parallel kernel; the sequential scan
// is then FMAs only, reads its per-token rows as 16-byte loads one token ahead, and each
// thread owns RPT = D / 4 CONSECUTIVE rows of its column.
// prep[t][h][5][D] fp32 = (w, a * u, u, k, r)
template <typename T>
__global__ void delta_prep_kernel(const T* __restrict__ proj, int64_t ld, int off_r, int off_k, int off_a,
                                  const T* __restrict__ wl, int64_t ld_wl, const float* __restrict__ a_bias,
                                  const float* __restrict__ w0, float* __restrict__ prep, int H, int D) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const T* row = proj + (int64_t)t * ld + h * D;
  const T* wrow = wl + (int64_t)t * ld_wl + h * D;
  float ksq = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float k = ldf(row + off_k + d);
    ksq += k * k;
  }
  ksq = wave_sum(ksq);
  const float inv = 1.f / sqrtf(ksq + 1e-6f);
  float* dst = prep + ((int64_t)t * H + h) * 5 * D;
  for (int d = lane; d < D; d += 64) {
    const float k = ldf(row + off_k + d), u = k * inv;
    const float w = expf(-0.6065306597126334f * sigmoidf(ldf(wrow + d) + w0[h * D + d]));
    const float a = sigmoidf(ldf(row + off_a + d) + a_bias[h * D + d]);
    dst[d] = w;
    dst[D + d] = a * u;
    dst[2 * D + d] = u;
    dst[3 * D + d] = k;
    dst[4 * D + d] = ldf(row + off_r + d);
  }
}

// sum over the 4 lanes of a quad by DPP lane permutes (no LDS crossbar on the recurrence's critical path)
__device__ __forceinline__ float quad_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));  // lane ^ 1
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));  // lane ^ 2
  return v;
}

template <typename T, int RPT>
__global__ __launch_bounds__(16 * RPT) void delta_scan2_kernel(const float* __restrict__ prep, const T* __restrict__ proj,
                                                               int64_t ld, int off_v, float* __restrict__ state,
                                                               const int32_t* __restrict__ qsl,
                                                               const int32_t* __restrict__ seq_lens,
                                                               const int32_t* __restrict__ slots, float* __restrict__ o,
                                                               int H) {
  constexpr int D = kKS * RPT, NT = kKS * D, CT = 16, ROW4 = 5 * D / 4, NV = RPT / 4;
  // the per-token rows of CT tokens at a time, through LDS in two buffers: the next chunk's global
  // loads are in flight while this chunk's CT sequential steps run
  __shared__ float4 rows[2][CT][ROW4];
  __shared__ float vals[2][CT][D];
  const int h = blockIdx.x, s = blockIdx.y;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int ctx = seq_lens[s] - q;
  const int tid = threadIdx.x, col = tid / kKS, ks = tid % kKS;
  const int r0 = ks * RPT;
  float S[RPT];
  float* st = state + ((int64_t)slot * H + h) * D * D;
#pragma unroll
  for (int r = 0; r < RPT; ++r) S[r] = ctx > 0 ? st[(int64_t)(r0 + r) * D + col] : 0.f;
  float4 g[5];
  float gv[4];
  auto load_chunk = [&](int c) {
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const int idx = tid + NT * j, tt = idx / ROW4, off = idx - tt * ROW4, t = c * CT + tt;
      g[j] = t < q ? *reinterpret_cast<const float4*>(prep + ((int64_t)(q0 + t) * H + h) * 5 * D + 4 * off)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int idx = tid + NT * j, tt = idx / D, cc = idx - tt * D, t = c * CT + tt;
      gv[j] = t < q ? ldf(proj + (int64_t)(q0 + t) * ld + off_v + h * D + cc) : 0.f;
    }
  };
  auto store_chunk = [&](int b) {
#pragma unroll
    for (int j = 0; j < 5; ++j) {
      const int idx = tid + NT * j, tt = idx / ROW4;
      rows[b][tt][idx - tt * ROW4] = g[j];
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int idx = tid + NT * j, tt = idx / D;
      vals[b][tt][idx - tt * D] = gv[j];
    }
  };
  const int HD = H * D, nchunks = (q + CT - 1) / CT;
  load_chunk(0);
  store_chunk(0);
  __syncthreads();
  for (int c = 0; c < nchunks; ++c) {
    const int b = c & 1;
    if (c + 1 < nchunks) load_chunk(c + 1);
    const int n = min(CT, q - c * CT);
    for (int tt = 0; tt < n; ++tt) {
      float4 in[5][NV];
#pragma unroll
      for (int a = 0; a < 5; ++a)
#pragma unroll
        for (int i = 0; i < NV; ++i) in[a][i] = rows[b][tt][a * (D / 4) + r0 / 4 + i];
      const float v = vals[b][tt][col];
      const float* w = reinterpret_cast<const float*>(in[0]);
      const float* au = reinterpret_cast<const float*>(in[1]);
      const float* u = reinterpret_cast<const float*>(in[2]);
      const float* k = reinterpret_cast<const float*>(in[3]);
      const float* rr = reinterpret_cast<const float*>(in[4]);
      float p[4] = {0.f, 0.f, 0.f, 0.f};  // four chains instead of one of RPT dependent FMAs
#pragma unroll
      for (int r = 0; r < RPT; ++r) p[r & 3] += u[r] * S[r];
      const float uS = quad_sum((p[0] + p[1]) + (p[2] + p[3]));
      float a4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < RPT; ++r) {
        S[r] = w[r] * S[r] - au[r] * uS + k[r] * v;
        a4[r & 3] += S[r] * rr[r];
      }
      const float ot = quad_sum((a4[0] + a4[1]) + (a4[2] + a4[3]));
      if (ks == 0) o[(int64_t)(q0 + c * CT + tt) * HD + h * D + col] = ot;
    }
    if (c + 1 < nchunks) store_chunk(b ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < RPT; ++r) st[(int64_t)(r0 + r) * D + col] = S[r];
}

template <typename T>
__global__ void delta_out_kernel(const float* __restrict__ o, const float* __restrict__ nw, const T* __restrict__ gate,
                                 int64_t gate_stride, float eps, T* __restrict__ out, int H, int D) {
  const int t = blockIdx.x, h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;  // a wave per head
  if (h >= H) return;
  const float* row = o + ((int64_t)t * H + h) * D;
  float ss = 0.f;
  for (int d = lane; d < D; d += 64) ss += row[d] * row[d];
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / (float)D + eps);
  for (int d = lane; d < D; d += 64)
    stf(out + ((int64_t)t * H + h) * D + d,
        row[d] * r * nw[h * D + d] * sigmoidf(ldf(gate + (int64_t)t * gate_stride + h * D + d)));
}

// ------------------------------------------------------------------ activations
// xIELU with sp = softplus(p), cn = 1/2 + softplus(q):
//   z > 0: sp z^2 + z/2 ;  z <= 0: cn (exp(z) - 1 - z) + z/2
template <typename T>
__global__ void xielu_kernel(const T* __restrict__ in, const float* __restrict__ bias, float sp, float cn,
                             T* __restrict__ out, int64_t n, int F) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float z = ldf(in + i);
    if (bias) z += bias[i % F];
    const float y = z > 0.f ? sp * z * z + 0.5f * z : cn * (expm1f(z) - z) + 0.5f * z;
    stf(out + i, y);
  }
}

// F % 4 == 0: 4 elements per access
template <typename T>
__global__ void xielu_vec_kernel(const T* __restrict__ in, const float* __restrict__ bias, float sp, float cn,
                                 T* __restrict__ out, int64_t n4, int F) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    float z[4], b[4] = {0.f, 0.f, 0.f, 0.f}, y[4];
    ld4(in + 4 * i, z);
    if (bias) ld4(bias + (4 * i) % F, b);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v = z[e] + b[e];
      y[e] = v > 0.f ? sp * v * v + 0.5f * v : cn * (expm1f(v) - v) + 0.5f * v;
    }
    st4(out + 4 * i, y);
  }
}

template <typename T>
__global__ void tanh_cols_kernel(const T* __restrict__ in, int64_t ld, T* __restrict__ out, int n, int64_t total) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x)
    stf(out + i, tanhf(ldf(in + (i / n) * ld + i % n)));
}

// [H, T, n] -> [T, H * n]
template <typename T>
__global__ void heads_to_rows_kernel(const T* __restrict__ in, T* __restrict__ out, int Ttot, int H, int n) {
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < H * n; i += blockDim.x) {
    const int h = i / n, d = i % n;
    out[(int64_t)t * H * n + i] = in[((int64_t)h * Ttot + t) * n + d];
  }
}

// ================================================================== host launchers
void embed_rows(const int32_t* ids, const void* table, bool f32, float* out, int T_, int W, int V, const void* pos_table,
                const int32_t* positions, int P, float scale, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, embed_rows_kernel<T><<<T_, 256, 0, st>>>(ids, (const T*)table, out, W, V, (const T*)pos_table,
                                                                positions, P, scale);)
}

void causal_conv(const void* x, bool in_f32, int64_t ld_in, const float* w, const float* bias, float* state,
                 const int32_t* qsl, const int32_t* seq_lens, const int32_t* slots, void* out, bool out_f32, int ns,
                 int max_q, int W, int taps, bool residual, bool act, hipStream_t st) {
  if (ns <= 0 || max_q <= 0) return;
  const int tile = 64;
  const int ntiles = (max_q + tile - 1) / tile;
  dim3 grid((W + 255) / 256, ntiles, ns);
  const int ws = ntiles == 1 ? 1 : 0;
#define XGM_CC(TI, TO)                                                                                                 \
  canon_conv_kernel<TI, TO><<<grid, 256, 0, st>>>((const TI*)x, ld_in, w, bias, state, qsl, seq_lens, slots, (TO*)out, \
                                                  W, taps, tile, ws, residual ? 1 : 0, act ? 1 : 0);
  if (in_f32) {
    if (out_f32) { XGM_CC(float, float) } else { XGM_CC(float, bf16) }
  } else {
    if (out_f32) { XGM_CC(bf16, float) } else { XGM_CC(bf16, bf16) }
  }
#undef XGM_CC
  if (!ws) {
    XGM_DISPATCH_T(in_f32, canon_state_kernel<T><<<dim3((W + 255) / 256, ns), 256, 0, st>>>((const T*)x, ld_in, state, qsl,
                                                                                           seq_lens, slots, W, taps);)
  }
}

// the carried inputs of a convolution whose outputs another kernel formed: state <- last taps - 1 inputs per sequence
void conv_state_update(const void* x, bool in_f32, int64_t ld_in, float* state, const int32_t* qsl,
                       const int32_t* seq_lens, const int32_t* slots, int ns, int W, int taps, hipStream_t st) {
  if (ns <= 0 || taps <= 1) return;
  XGM_DISPATCH_T(in_f32, canon_state_kernel<T><<<dim3((W + 255) / 256, ns), 256, 0, st>>>((const T*)x, ld_in, state, qsl,
                                                                                         seq_lens, slots, W, taps);)
}

void canon_conv(const float* x, const float* w, float* state, const int32_t* qsl, const int32_t* seq_lens,
                const int32_t* slots, void* out, bool out_f32, int ns, int max_q, int W, int taps, hipStream_t st) {
  causal_conv(x, true, W, w, nullptr, state, qsl, seq_lens, slots, out, out_f32, ns, max_q, W, taps, true, false, st);
}

void scaled_add_rmsnorm(const float* x, const void* y, bool y_f32, int64_t y_stride, const float* bias, float alpha,
                        const float* w, float w_offset, float eps, float* x_out, void* out, bool out_f32, int T_, int W,
                        hipStream_t st) {
  if (T_ <= 0) return;
  const int ysz = y_f32 ? 4 : 2;
  const bool vec = W % 4 == 0 && W <= 8192 && (y == nullptr || ((uintptr_t)y % 16 == 0 && (y_stride * ysz) % 16 == 0));
#define XGM_SAR(TY, TO)                                                                                                  \
  {                                                                                                                      \
    if (vec && W <= 2048)                                                                                                \
      scaled_add_rmsnorm_vec_kernel<TY, TO, 2><<<T_, 256, 0, st>>>(x, (const TY*)y, y_stride, bias, alpha, w, w_offset, \
                                                                    eps, x_out, (TO*)out, W);                            \
    else if (vec)                                                                                                        \
      scaled_add_rmsnorm_vec_kernel<TY, TO, 8><<<T_, 256, 0, st>>>(x, (const TY*)y, y_stride, bias, alpha, w, w_offset, \
                                                                    eps, x_out, (TO*)out, W);                            \
    else                                                                                                                 \
      scaled_add_rmsnorm_kernel<TY, TO><<<T_, 256, 0, st>>>(x, (const TY*)y, y_stride, bias, alpha, w, w_offset, eps,    \
                                                            x_out, (TO*)out, W);                                         \
  }
  if (y_f32) {
    if (out_f32) XGM_SAR(float, float) else XGM_SAR(float, bf16)
  } else {
    if (out_f32) XGM_SAR(bf16, float) else XGM_SAR(bf16, bf16)
  }
#undef XGM_SAR
}

void latent_prep(const void* proj, bool f32, int64_t ld, int off_q, int Rq, int off_kv, int R, int rd, const float* wq,
                 const float* wkv, float eps, const int32_t* positions, const int32_t* slot_mapping, const float* rot,
                 int rot_dims, void* cq, void* cache, int T_, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, latent_prep_kernel<T><<<T_, 256, 0, st>>>((const T*)proj, ld, off_q, Rq, off_kv, R, rd, wq, wkv, eps,
                                                                 positions, slot_mapping, rot, rot_dims, (T*)cq,
                                                                 (T*)cache);)
}

template <typename T, int NR>
static int launch_latent_attention(const void* qabs, const void* q, int64_t q_stride, int dq, int dn, const void* gate,
                                   int64_t gate_stride, const void* cache, const int32_t* bt, int bt_width, int bs,
                                   const int32_t* positions, const int32_t* token_seq, const float* rot, int rot_dims,
                                   void* out, int Ttot, int H, int R, int rd, int window, float scale, hipStream_t st) {
  const int Dk = R + rd;
  int KT = 64;
  auto bytes = [&](int kt) { return ((size_t)kt * (Dk + 1) + (size_t)kHPB * Dk) * sizeof(float); };
  while (KT > 16 && bytes(KT) > 96 * 1024) KT >>= 1;
  if (bytes(KT) > 150 * 1024) return -1;
  while (KT > 16 && KT / 2 >= window) KT >>= 1;  // short windows: no idle key lanes
  auto kern = latent_attention_kernel<T, NR>;
  if (bytes(KT) > 48 * 1024) {
    static size_t set_bytes = 0;
    if (bytes(KT) > set_bytes) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess)
        return -2;
      set_bytes = 150 * 1024;
    }
  }
  dim3 grid(Ttot, (H + kHPB - 1) / kHPB);
  kern<<<grid, 256, bytes(KT), st>>>((const T*)qabs, (const T*)q, q_stride, dq, dn, (const T*)gate, gate_stride,
                                     (const T*)cache, bt, bt_width, bs, positions, token_seq, rot, rot_dims, (T*)out, Ttot,
                                     H, R, rd, window, scale, KT);
  return 0;
}

int latent_attention(const void* qabs, const void* q, bool f32, int64_t q_stride, int dq, int dn, const void* gate,
                     int64_t gate_stride, const void* cache, const int32_t* bt, int bt_width, int bs,
                     const int32_t* positions, const int32_t* token_seq, const float* rot, int rot_dims, void* out,
                     int Ttot, int H, int R, int rd, int window, float scale, hipStream_t st) {
  if (Ttot <= 0) return 0;
#define XGM_LA(NR)                                                                                                  \
  XGM_DISPATCH_T(f32, return (launch_latent_attention<T, NR>(qabs, q, q_stride, dq, dn, gate, gate_stride, cache, bt, \
                                                              bt_width, bs, positions, token_seq, rot, rot_dims, out, \
                                                              Ttot, H, R, rd, window, scale, st));)
  if (R <= 128) { XGM_LA(2) }
  if (R <= 256) { XGM_LA(4) }
  if (R <= 512) { XGM_LA(8) }
  if (R <= 1024) { XGM_LA(16) }
#undef XGM_LA
  return -3;
}

template <int NMT_MAX>
static int launch_latent_mfma(const void* qabs, const void* q, int dq, int dn, const void* gate, int64_t gate_stride,
                              const void* cache, const int32_t* bt, int bt_width, int bs, const int32_t* qsl,
                              const int32_t* seq_lens, const int32_t* slots, const float* rot, int rot_dims, void* out,
                              int Ttot, int ns, int max_q, int H, int R, int rd, int window, float scale, int nsplit,
                              float* part_o, float* part_ml, hipStream_t st) {
  const int nkk = (R + rd + 31) / 32;
  const size_t bytes = (size_t)kKT * (nkk * 32 + 8) * sizeof(uint16_t);
  // single-token steps walk one or two tiles per key share, at two waves per SIMD where the registers allow
  auto kern = max_q == 1 ? latent_attention_mfma_kernel<NMT_MAX, true, (NMT_MAX <= 16 ? 2 : 1)>
                         : latent_attention_mfma_kernel<NMT_MAX, false, 1>;
  if (bytes > 48 * 1024) {
    static bool set[2] = {false, false};
    if (!set[max_q == 1]) {
      if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024) != hipSuccess)
        return -2;
      set[max_q == 1] = true;
    }
  }
  const int TPT = max_q == 1 ? 1 : 16, HPT = max_q == 1 ? std::min(16, H) : 1;
  if (max_q != 1 || part_o == nullptr || part_ml == nullptr) nsplit = 1;
  dim3 grid(nsplit > 1 ? nsplit : (max_q + TPT - 1) / TPT, ns, (H + 4 * HPT - 1) / (4 * HPT));
  kern<<<grid, 256, bytes, st>>>((const bf16*)qabs, (const bf16*)q, dq, dn, (const bf16*)gate, gate_stride,
                                 (const bf16*)cache, bt, bt_width, bs, qsl, seq_lens, slots, rot, rot_dims, (bf16*)out,
                                 Ttot, H, R, rd, window, scale, TPT, HPT, nsplit, part_o, part_ml);
  if (nsplit > 1)
    latent_attention_combine_kernel<<<dim3(Ttot, H), 64, 0, st>>>(part_o, part_ml, (const bf16*)gate, gate_stride, slots,
                                                                  (bf16*)out, Ttot, H, R, nsplit);
  return 0;
}

// bf16 only; R % 16 == 0, R <= 512, rd % 8 == 0, rd <= 128 (checked by the caller)
int latent_attention_mfma(const void* qabs, const void* q, int dq, int dn, const void* gate, int64_t gate_stride,
                          const void* cache, const int32_t* bt, int bt_width, int bs, const int32_t* qsl,
                          const int32_t* seq_lens, const int32_t* slots, const float* rot, int rot_dims, void* out,
                          int Ttot, int ns, int max_q, int H, int R, int rd, int window, float scale, int nsplit,
                          float* part_o, float* part_ml, hipStream_t st) {
  if (Ttot <= 0 || ns <= 0 || max_q <= 0) return 0;
  if (nsplit > 1 && Ttot != ns) return -4;  // key shares are for steps of one token per sequence
  if (R % 16 || rd % 8 || R > 512 || rd > 128 || R < 16) return -1;
#define XGM_LM(N)                                                                                                     \
  return launch_latent_mfma<N>(qabs, q, dq, dn, gate, gate_stride, cache, bt, bt_width, bs, qsl, seq_lens, slots, rot, \
                               rot_dims, out, Ttot, ns, max_q, H, R, rd, window, scale, nsplit, part_o, part_ml, st);
  if (R <= 128) { XGM_LM(8) }
  if (R <= 256) { XGM_LM(16) }
  XGM_LM(32)
#undef XGM_LM
}

// prep: fp32 scratch of Ttot * H * 5 * D floats, or null for the one-pass kernel
int delta_scan(const void* proj, bool f32, int64_t ld, int off_r, int off_k, int off_v, int off_a, const void* wl,
               int64_t ld_wl, const float* a_bias, const float* w0, float* state, const int32_t* qsl,
               const int32_t* seq_lens, const int32_t* slots, float* o, int ns, int H, int D, float* prep, int Ttot,
               hipStream_t st) {
  if (ns <= 0) return 0;
  const int threads = ((kKS * D + 63) / 64) * 64;
  if (threads > 1024) return -1;
  dim3 grid(H, ns);
  if (prep != nullptr && (D == 16 || D == 32 || D == 64)) {
    XGM_DISPATCH_T(f32, delta_prep_kernel<T><<<dim3(Ttot, H), 64, 0, st>>>((const T*)proj, ld, off_r, off_k, off_a,
                                                                           (const T*)wl, ld_wl, a_bias, w0, prep, H, D);)
#define XGM_DS2(RPT)                                                                                               \
  XGM_DISPATCH_T(f32, delta_scan2_kernel<T, RPT><<<grid, threads, 0, st>>>(prep, (const T*)proj, ld, off_v, state, \
                                                                            qsl, seq_lens, slots, o, H);)          \
  return 0;
    if (D == 16) { XGM_DS2(4) }
    if (D == 32) { XGM_DS2(8) }
    if (D == 64) { XGM_DS2(16) }
#undef XGM_DS2
  }
#define XGM_DS(MAXR)                                                                                                  \
  XGM_DISPATCH_T(f32, delta_scan_kernel<T, MAXR><<<grid, threads, 0, st>>>((const T*)proj, ld, off_r, off_k, off_v,  \
                                                                            off_a, (const T*)wl, ld_wl, a_bias, w0,   \
                                                                            state, qsl, seq_lens, slots, o, H, D);)  \
  return 0;
  if (D <= 32) { XGM_DS(8) }
  if (D <= 64) { XGM_DS(16) }
  if (D <= 128) { XGM_DS(32) }
  if (D <= 256) { XGM_DS(64) }
#undef XGM_DS
  return -1;
}

void delta_out(const float* o, const float* nw, const void* gate, bool f32, int64_t gate_stride, float eps, void* out,
               int T_, int H, int D, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, delta_out_kernel<T><<<dim3(T_, (H + 3) / 4), 256, 0, st>>>(o, nw, (const T*)gate, gate_stride, eps, (T*)out, H, D);)
}

void xielu(const void* in, bool f32, const float* bias, float sp, float cn, void* out, int64_t n, int F, hipStream_t st) {
  if (n <= 0) return;
  if (F % 4 == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const int blocks4 = (int)std::min<int64_t>((n / 4 + 255) / 256, 1 << 20);
    XGM_DISPATCH_T(f32, xielu_vec_kernel<T><<<blocks4, 256, 0, st>>>((const T*)in, bias, sp, cn, (T*)out, n / 4, F);)
    return;
  }
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, 65535);
  XGM_DISPATCH_T(f32, xielu_kernel<T><<<blocks, 256, 0, st>>>((const T*)in, bias, sp, cn, (T*)out, n, F);)
}

void tanh_cols(const void* in, bool f32, int64_t ld, void* out, int T_, int n, hipStream_t st) {
  const int64_t total = (int64_t)T_ * n;
  if (total <= 0) return;
  const int blocks = (int)std::min<int64_t>((total + 255) / 256, 65535);
  XGM_DISPATCH_T(f32, tanh_cols_kernel<T><<<blocks, 256, 0, st>>>((const T*)in, ld, (T*)out, n, total);)
}

void heads_to_rows(const void* in, bool f32, void* out, int T_, int H, int n, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, heads_to_rows_kernel<T><<<T_, 256, 0, st>>>((const T*)in, (T*)out, T_, H, n);)
}

}  // namespace xgm
