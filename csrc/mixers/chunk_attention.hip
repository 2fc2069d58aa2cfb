// Grouped-query softmax attention over a paged K / V cache with a configurable visibility rule,
// per-head temperature and an optional "sink" term in the softmax denominator.
//
//   qk_norm_cache     from a fused projection row [q | k | v]: RMS norm over the WHOLE q vector and the
//                     WHOLE k vector (all heads at once, weights wq / wk; nullptr = no norm), q to a
//                     dense tensor, k and v to the cache rows slot_mapping[t]
//   masked_attention  token at position i of its sequence sees keys j in [lo(i), i]:
//                       kMaskCausal  lo = 0
//                       kMaskWindow  lo = max(0, i - size + 1)
//                       kMaskChunk   lo = floor(i / size) * size   (chunks counted from the sequence's start)
//                     score = (q . k) * scale * temp[h];  p_j = exp(score_j) / (sum_j' exp(score_j') + exp(sink[h]))
//                     (the sink adds to the denominator only: no key, no value, not scaled). Positions enter
//                     the scores only through an optional distance penalty: with r1 / r2 the score of key j
//                     loses r1[h] * ln(1 + r2[h] * (i - j)). With `gate` head h's output is multiplied by
//                     sigmoid(gate[t][h]). `vmode` chooses the values a query head weighs: kValuesOwn its own
//                     key/value head's (output [T][H][dv]), kValuesAll the concatenated values of all G heads
//                     (output [T][H][G dv]: what mixing the heads' weight maps after the softmax needs),
//                     c >= 0 head c's for every query head.
//                     `gate_elem`: the gate has one logit per output entry, out[t][h][d] *= sigmoid(gate[t][h dv + d]).
//                     `wfn` = kWeightsSigmoid: no softmax; the weight of a visible key is sigmoid(score + hbias[h]),
//                     not normalised over the keys (no sink).
//   talk_mix          out[t][h] = sigmoid(gate[t][h]) * sum_g talk[h][g] * o_all[t][g][c(h)], c(h) = h / (H / G)
//   head_norm_rope_cache  per-head RMS norm of q and k (one weight of a head's size for all heads), pairwise
//                     rotation of each head's first entries by a (cos, sin) table row of the token's position,
//                     q to a dense tensor, k / v to the cache rows slot_mapping[t]
//
// Activations / caches are T = float or bf16; norms, scores, probabilities and the accumulators are fp32.
#include "mixers_common.h"

namespace xgm {

constexpr int kMaskCausal = 0, kMaskWindow = 1, kMaskChunk = 2;
constexpr int kValuesOwn = -1, kValuesAll = -2;
constexpr int kWeightsSoftmax = 0, kWeightsSigmoid = 1;

__device__ __forceinline__ int first_visible(int mask, int size, int pos) {
  if (mask == kMaskWindow) return max(0, pos - size + 1);
  if (mask == kMaskChunk) return (pos / size) * size;
  return 0;
}

// ------------------------------------------------------------------ projections -> normed q, cache rows
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(const T* __restrict__ proj, int64_t ld, int nq, int nk, int nv,
                                                            const float* __restrict__ wq, const float* __restrict__ wk,
                                                            float eps, const int32_t* __restrict__ slot_mapping,
                                                            T* __restrict__ q_out, T* __restrict__ kcache,
                                                            T* __restrict__ vcache) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = proj + (int64_t)t * ld;
  float rq = 1.f, rk = 1.f;
  if (wq) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < nq; c += blockDim.x) {
      const float v = ldf(row + c);
      ss += v * v;
    }
    rq = 1.f / sqrtf(block_sum(ss, red) / (float)nq + eps);
  }
  for (int c = threadIdx.x; c < nq; c += blockDim.x)
    stf(q_out + (int64_t)t * nq + c, ldf(row + c) * rq * (wq ? wq[c] : 1.f));
  const int slot = slot_mapping[t];
  if (slot < 0) return;  // padding row: nothing is cached (uniform over the block)
  if (wk) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < nk; c += blockDim.x) {
      const float v = ldf(row + nq + c);
      ss += v * v;
    }
    rk = 1.f / sqrtf(block_sum(ss, red) / (float)nk + eps);
  }
  for (int c = threadIdx.x; c < nk; c += blockDim.x)
    stf(kcache + (int64_t)slot * nk + c, ldf(row + nq + c) * rk * (wk ? wk[c] : 1.f));
  for (int c = threadIdx.x; c < nv; c += blockDim.x) vcache[(int64_t)slot * nv + c] = row[nq + nk + c];
}

// ------------------------------------------------------------------ general kernel (any sizes, float or bf16)
// One workgroup = one token x one key/value head; its query heads (up to 8 per launch row) are spread
// over the 4 waves, 2 per wave. A tile of KT keys (K and V rows) is staged in LDS once for all of them.
constexpr int kQPW = 2;  // query heads per wave

template <typename T, int NR>
__global__ __launch_bounds__(256) void masked_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int32_t* __restrict__ block_tables, int bt_width, int bs, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ token_seq, const float* __restrict__ temp, const float* __restrict__ sink,
    T* __restrict__ out, int H, int G, int dk, int dv_head, int mask, int size, float scale, int KT,
    const T* __restrict__ gate, int64_t ld_gate, const float* __restrict__ r1, const float* __restrict__ r2, int vmode,
    int gate_elem, int wfn, const float* __restrict__ hbias) {
  extern __shared__ float smem[];
  // dv: value columns per query head; voff: where they start in a cached row of G * dv_head values
  const int dv = vmode == kValuesAll ? G * dv_head : dv_head;
  const int voff = vmode == kValuesAll ? 0 : (vmode >= 0 ? vmode : (int)blockIdx.y) * dv_head;
  const int ldk = dk + 1, ldv = dv + 1;
  float* ktile = smem;                           // [KT][dk + 1]
  float* vtile = ktile + (size_t)KT * ldk;       // [KT][dv + 1]
  float* qs = vtile + (size_t)KT * ldv;          // [4 * kQPW][dk]
  const int t = blockIdx.x, g = blockIdx.y;
  const int rep = H / G;
  const int r0 = blockIdx.z * (4 * kQPW);        // first of this workgroup's query heads within the group
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int s = token_seq[t];
  if (s < 0) {
    for (int a = 0; a < kQPW; ++a) {
      const int r = r0 + wave + 4 * a;
      if (r < rep)
        for (int d = lane; d < dv; d += 64) stf(out + ((int64_t)t * H + g * rep + r) * dv + d, 0.f);
    }
    return;
  }
  const int pos = positions[t];
  const int j0 = first_visible(mask, size, pos);
  float m[kQPW], l[kQPW], acc[kQPW][NR], pen1[kQPW], pen2[kQPW], hb[kQPW];
#pragma unroll
  for (int a = 0; a < kQPW; ++a) {
    const int r = r0 + wave + 4 * a;
    const int h = g * rep + min(r, rep - 1);
    pen1[a] = r1 ? r1[h] : 0.f;
    pen2[a] = r1 ? r2[h] : 0.f;
    hb[a] = hbias ? hbias[h] : 0.f;
    float* qh = qs + (wave + 4 * a) * dk;
    const float sc = scale * (temp ? temp[h] : 1.f);
    for (int d = lane; d < dk; d += 64) qh[d] = r < rep ? ldf(q + ((int64_t)t * H + h) * dk + d) * sc : 0.f;
    // the sink starts the running softmax: weight exp(sink - m) = 1 with no value behind it
    m[a] = sink ? sink[h] : -INFINITY;
    l[a] = sink ? 1.f : 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[a][i] = 0.f;
  }
  const int LPK = 64 / KT;  // lanes per key in the score phase
  const int kj = lane / LPK, part = lane % LPK;
  const int32_t* bt = block_tables + (int64_t)s * bt_width;
  for (int k0 = j0; k0 <= pos; k0 += KT) {
    const int n = min(KT, pos - k0 + 1);
    __syncthreads();  // the previous tile is consumed (and qs is written, on the first pass)
    for (int jj = wave; jj < n; jj += 4) {
      const int key = k0 + jj;
      const int64_t row = (int64_t)bt[key / bs] * bs + key % bs;
      const T* ks = kcache + (row * G + g) * dk;
      const T* vs = vcache + row * G * dv_head + voff;
      for (int d = lane; d < dk; d += 64) ktile[jj * ldk + d] = ldf(ks + d);
      for (int d = lane; d < dv; d += 64) vtile[jj * ldv + d] = ldf(vs + d);
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < kQPW; ++a) {
      if (r0 + wave + 4 * a >= rep) continue;
      const float* qh = qs + (wave + 4 * a) * dk;
      float sc = 0.f;
      if (kj < n) {
        const float* kr = ktile + kj * ldk;
        for (int d = part; d < dk; d += LPK) sc += qh[d] * kr[d];
      }
      for (int o = 1; o < LPK; o <<= 1) sc += __shfl_xor(sc, o, 64);
      if (r1 && kj < n) sc -= pen1[a] * log1pf(pen2[a] * (float)(pos - (k0 + kj)));
      float p;
      if (wfn == kWeightsSigmoid) {   // every visible key weighs sigmoid(score + bias), whatever the others do
        p = kj < n ? sigmoidf(sc + hb[a]) : 0.f;
      } else {
        if (kj >= n) sc = -INFINITY;
        const float mn = fmaxf(m[a], wave_max(sc));
        p = kj < n ? expf(sc - mn) : 0.f;
        const float corr = m[a] == -INFINITY ? 0.f : expf(m[a] - mn);
        l[a] = l[a] * corr + wave_sum(part == 0 ? p : 0.f);
        m[a] = mn;
#pragma unroll
        for (int i = 0; i < NR; ++i) acc[a][i] *= corr;
      }
      for (int j = 0; j < n; ++j) {
        const float pj = __shfl(p, j * LPK, 64);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int d = lane + 64 * i;
          if (d < dv) acc[a][i] += pj * vtile[j * ldv + d];
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < kQPW; ++a) {
    const int r = r0 + wave + 4 * a;
    if (r >= rep) continue;
    float inv = wfn == kWeightsSigmoid ? 1.f : 1.f / l[a];
    if (gate && !gate_elem) inv *= sigmoidf(ldf(gate + (int64_t)t * ld_gate + g * rep + r));
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = lane + 64 * i;
      if (d >= dv) continue;
      float o = acc[a][i] * inv;
      if (gate && gate_elem) o *= sigmoidf(ldf(gate + (int64_t)t * ld_gate + (int64_t)(g * rep + r) * dv + d));
      stf(out + ((int64_t)t * H + g * rep + r) * dv + d, o);
    }
  }
}


// ------------------------------------------------------------------ matrix-core form (bf16, dk % 32 == 0, dv % 16 == 0)
// A wave owns 16 query slots. Prompt portions: 16 consecutive tokens of one sequence x one query head; the 4 waves
// of a workgroup are RH query heads of one key/value head x 4 / RH token tiles, so a tile of 64 keys (K rows and
// V rows, staged once in LDS) serves all of them. Steps of single tokens: the slots are the (up to 64) query heads
// of one key/value head at the sequence's one token, one workgroup per (sequence, key/value head). S^T = K Q^T on v_mfma_f32_16x16x32_bf16: the accumulator
// holds, per lane, 16 keys of ONE slot, and packed to bf16 it is the B operand of O^T += V^T P^T, whose A
// operand (V^T) is a transposed LDS read of the staged V rows.
constexpr int kKT = 64;

__device__ __forceinline__ float exp2_fast(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_exp2f(x);
#else
  return exp2f(x);
#endif
}

__device__ __forceinline__ float rcp_fast(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_rcpf(x);
#else
  return 1.f / x;
#endif
}

template <int NKK_MAX, int NMT_MAX, int NW, int WFN>
__global__ __launch_bounds__(64 * NW) void masked_attention_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ kcache, const bf16* __restrict__ vcache,
    const int32_t* __restrict__ block_tables, int bt_width, int bs, const int32_t* __restrict__ qsl,
    const int32_t* __restrict__ seq_lens, const int32_t* __restrict__ slots, const float* __restrict__ temp,
    const float* __restrict__ sink, bf16* __restrict__ out, int H, int G, int dk, int dv_head, int mask, int size,
    float scale, int RH, int head_slots, float* __restrict__ part_o, float* __restrict__ part_ml, int Ttot,
    const bf16* __restrict__ gate, int64_t ld_gate, const float* __restrict__ r1, const float* __restrict__ r2, int vmode,
    int gate_elem, const float* __restrict__ hbias) {
  extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
  // dv: value columns per query head; voff: where they start in a cached row of G * dv_head values
  const int dv = vmode == kValuesAll ? G * dv_head : dv_head;
  const int LDK = dk + 8, LDV = dv + 8;
  uint16_t* ktile = lds;                 // [kKT][LDK]
  uint16_t* vtile = lds + kKT * LDK;     // [kKT][LDV]
  const int s = blockIdx.z;
  const int q0 = qsl[s], qn = qsl[s + 1] - q0;
  const int rep = H / G;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, kg = lane >> 4;
  if (slots[s] < 0 || qn <= 0) {
    // a padding row of a single-token step still gets a defined output row
    if (head_slots && qn == 1)
      for (int d = threadIdx.x; d < rep * dv; d += blockDim.x) out[((int64_t)q0 * H + blockIdx.y * rep) * dv + d] = 0;
    return;
  }
  // prompt portions: slots = 16 tokens of one head; single-token steps (head_slots): slots = 16 heads of the token
  const int tpb = head_slots ? 1 : NW / RH;  // token tiles per workgroup
  // late token tiles see the most keys: they are dispatched first
  const int t0 = head_slots ? 0 : ((int)gridDim.x - 1 - (int)blockIdx.x) * 16 * tpb;
  if (t0 >= qn) return;
  const int hblocks = (rep + RH - 1) / RH;
  const int g = head_slots ? blockIdx.y : blockIdx.y / hblocks, hb = blockIdx.y % hblocks;
  const int hr = head_slots ? wave * 16 + li : hb * RH + wave % RH;   // head within the group
  const int tok = head_slots ? 0 : t0 + (wave / RH) * 16 + li;         // token within the sequence's rows
  const bool wave_on = head_slots ? wave * 16 < rep : (hr < rep && t0 + (wave / RH) * 16 < qn);
  const bool valid = wave_on && hr < rep && tok < qn;
  const int head = g * rep + min(hr, rep - 1);
  const int voff = vmode == kValuesAll ? 0 : (vmode >= 0 ? vmode : g) * dv_head;
  const float pen1 = r1 ? r1[head] : 0.f, pen2 = r1 ? r2[head] : 0.f;
  const int ctx = seq_lens[s] - qn;
  const int pos_q = ctx + min(tok, qn - 1);
  const int lo_q = first_visible(mask, size, pos_q);
  // a key tile [k0, k0 + 63] needs no per-key test when every slot of the wave sees all of it (wave-uniform)
  const int tw = head_slots ? 0 : t0 + (wave / RH) * 16;               // the wave's first token
  const bool slots_full = head_slots || tw + 16 <= qn;
  const int pos_w0 = ctx + min(tw, qn - 1);
  const int lo_w1 = first_visible(mask, size, ctx + min(head_slots ? 0 : tw + 15, qn - 1));
  const int nkk = dk / 32, nmt = dv / 16;
  // keys any slot of this workgroup can see
  int kmin = first_visible(mask, size, ctx + t0);
  int pos_last = ctx + (head_slots ? 1 : min(qn, t0 + 16 * tpb)) - 1;
  // single-token steps divide the visible key tiles over gridDim.x workgroups (merged by a second launch)
  const int nsplit = head_slots ? gridDim.x : 1;
  if (nsplit > 1) {
    const int tiles = (pos_last - kmin + kKT) / kKT, per = (tiles + nsplit - 1) / nsplit;
    kmin += blockIdx.x * per * kKT;
    pos_last = min(pos_last, kmin + per * kKT - 1);  // may leave this share empty
  }
  const int32_t* bt = block_tables + (int64_t)s * bt_width;

  xgk::bf16x8_t qf[NKK_MAX];
#pragma unroll
  for (int kk = 0; kk < NKK_MAX; ++kk) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (kk < nkk && valid) v = xgk::ld16(q + ((int64_t)(q0 + tok) * H + head) * dk + kk * 32 + kg * 8);
    qf[kk] = xgk::as_frag(v);
  }
  // scores are kept in units of ln 2 (exp2 is one instruction): score * log2(e)
  constexpr float kLog2e = 1.4426950408889634f;
  const float sc_h = scale * (temp ? temp[head] : 1.f) * kLog2e;
  xgk::f32x4_t o[NMT_MAX];
#pragma unroll
  for (int mt = 0; mt < NMT_MAX; ++mt) o[mt] = xgk::f32x4_t{0.f, 0.f, 0.f, 0.f};
  // the sink starts the running softmax: weight exp(sink - m) = 1 with no value behind it
  const bool with_sink = sink && (nsplit == 1 || blockIdx.x == 0);  // the sink enters the first share only
  float m = with_sink ? sink[head] * kLog2e : -INFINITY, l = with_sink ? 1.f : 0.f;
  constexpr bool sig = WFN == kWeightsSigmoid;
  const float sbias = (sig && hbias) ? hbias[head] * kLog2e : 0.f;   // the per-head score bias, in units of ln 2

  // staging: thread -> (row = tid / NW, 16-byte chunks tid % NW, + NW, ..) of the K row and of the V row. The next
  // tile's rows are loaded into registers before the current tile's products and stored after them.
  const int srow = threadIdx.x / NW, squad = threadIdx.x % NW;
  constexpr int NKC = (NKK_MAX * 4 + NW - 1) / NW, NVC = (NMT_MAX * 2 + NW - 1) / NW;
  uint4 sk[NKC], sv[NVC];
  auto fetch = [&](int k0) {
    const int kabs = k0 + srow;
    const bool ok = kabs <= pos_last;
    const int64_t row = ok ? (int64_t)bt[kabs / bs] * bs + kabs % bs : 0;
    const bf16* ks = kcache + (row * G + g) * dk;
    const bf16* vs = vcache + row * G * dv_head + voff;
#pragma unroll
    for (int it = 0; it < NKC; ++it) {
      const int ch = squad + NW * it;
      sk[it] = (ok && ch * 8 < dk) ? xgk::ld16(ks + ch * 8) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < NVC; ++it) {
      const int ch = squad + NW * it;
      sv[it] = (ok && ch * 8 < dv) ? xgk::ld16(vs + ch * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int it = 0; it < NKC; ++it) {
      const int ch = squad + NW * it;
      if (ch * 8 < dk) xgk::st16(ktile + srow * LDK + ch * 8, sk[it]);
    }
#pragma unroll
    for (int it = 0; it < NVC; ++it) {
      const int ch = squad + NW * it;
      if (ch * 8 < dv) xgk::st16(vtile + srow * LDV + ch * 8, sv[it]);
    }
  };
  if (kmin <= pos_last) fetch(kmin);
  for (int k0 = kmin; k0 <= pos_last; k0 += kKT) {
    __syncthreads();  // the previous tile is consumed
    commit();
    __syncthreads();
    if (k0 + kKT <= pos_last) fetch(k0 + kKT);
    if (!wave_on) continue;
    xgk::f32x4_t sacc[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      sacc[n] = xgk::f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < NKK_MAX; ++kk)
        if (kk < nkk)
          sacc[n] = xgk::mfma16x16x32(xgk::as_frag(xgk::ld16(ktile + (n * 16 + li) * LDK + kk * 32 + kg * 8)), qf[kk],
                                      sacc[n]);
    }
    float mx = -INFINITY;
    const bool full = slots_full && k0 + kKT - 1 <= pos_w0 && k0 >= lo_w1;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kabs = k0 + n * 16 + kg * 4 + r;
        float v = sacc[n][r] * sc_h;
        // r1 ln(1 + r2 d) in units of ln 2 is r1 log2(1 + r2 d)
        if (r1) v -= pen1 * __log2f(1.f + pen2 * (float)max(pos_q - kabs, 0));
        if (!full && (!valid || kabs > pos_q || kabs < lo_q)) v = -INFINITY;
        sacc[n][r] = v;
        mx = fmaxf(mx, v);
      }
    if constexpr (sig) {
      // weight = sigmoid(score + bias) = 1 / (1 + 2^-(s + b)) with s, b in units of ln 2; an unseen key (-inf) weighs 0
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) sacc[n][r] = rcp_fast(1.f + exp2_fast(-(sacc[n][r] + sbias)));
    } else {
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m, mx);
      const float alpha = (m_new == -INFINITY || m == -INFINITY) ? (m == -INFINITY ? 0.f : 1.f) : exp2_fast(m - m_new);
      float rs = 0.f;
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = m_new == -INFINITY ? 0.f : exp2_fast(sacc[n][r] - m_new);
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
    }
    // O^T += V^T . P^T over two 32-key halves (keys in the order the score accumulator holds them)
#pragma unroll
    for (int sc = 0; sc < 2; ++sc) {
      uint4 pb;
      pb.x = xgk::pack2(sacc[2 * sc][0], sacc[2 * sc][1]);
      pb.y = xgk::pack2(sacc[2 * sc][2], sacc[2 * sc][3]);
      pb.z = xgk::pack2(sacc[2 * sc + 1][0], sacc[2 * sc + 1][1]);
      pb.w = xgk::pack2(sacc[2 * sc + 1][2], sacc[2 * sc + 1][3]);
      const xgk::bf16x8_t pfrag = xgk::as_frag(pb);
      const int qq = li >> 2, pp = li & 3;
      const int r0 = sc * 32 + 4 * kg + qq, r1 = r0 + 16;
#pragma unroll
      for (int mt = 0; mt < NMT_MAX; ++mt)
        if (mt < nmt) {
          const xgk::bf16x4_t a0 = xgk::lds_read_tr16(vtile + r0 * LDV + mt * 16 + 4 * pp);
          const xgk::bf16x4_t a1 = xgk::lds_read_tr16(vtile + r1 * LDV + mt * 16 + 4 * pp);
          const xgk::bf16x8_t vfrag = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
          o[mt] = xgk::mfma16x16x32(vfrag, pfrag, o[mt]);
        }
    }
  }
  if (valid && nsplit > 1) {  // unnormalised share: (m, l) and the weighted value sum
    const int64_t row = ((int64_t)blockIdx.x * Ttot + q0 + tok) * H + head;
    if (kg == 0) {
      part_ml[2 * row] = m;
      part_ml[2 * row + 1] = l;
    }
#pragma unroll
    for (int mt = 0; mt < NMT_MAX; ++mt)
      if (mt < nmt)
        *reinterpret_cast<float4*>(part_o + row * dv + mt * 16 + 4 * kg) = make_float4(o[mt][0], o[mt][1], o[mt][2], o[mt][3]);
  } else if (valid) {
    float inv = sig ? 1.f : (l > 0.f ? 1.f / l : 0.f);
    if (gate && !gate_elem) inv *= sigmoidf(bf2f(gate[(int64_t)(q0 + tok) * ld_gate + head]));
    bf16* op = out + ((int64_t)(q0 + tok) * H + head) * dv;
    const bf16* ge = gate_elem ? gate + (int64_t)(q0 + tok) * ld_gate + (int64_t)head * dv : nullptr;
#pragma unroll
    for (int mt = 0; mt < NMT_MAX; ++mt)
      if (mt < nmt) {
        float e[4] = {o[mt][0] * inv, o[mt][1] * inv, o[mt][2] * inv, o[mt][3] * inv};
        if (ge) {
#pragma unroll
          for (int r = 0; r < 4; ++r) e[r] *= sigmoidf(bf2f(ge[mt * 16 + 4 * kg + r]));
        }
        uint2 w;
        w.x = xgk::pack2(e[0], e[1]);
        w.y = xgk::pack2(e[2], e[3]);
        *reinterpret_cast<uint2*>(op + mt * 16 + 4 * kg) = w;
      }
  }
}

// merge the key shares of a single-token step: out = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s (m in units of ln 2)
__global__ void masked_attention_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                const int32_t* __restrict__ slots, bf16* __restrict__ out, int Ttot, int H,
                                                int dv, int nsplit, const bf16* __restrict__ gate, int64_t ld_gate,
                                                int gate_elem, int wfn) {
  const int t = blockIdx.x, h = blockIdx.y;
  if (slots[t] < 0) return;  // single-token steps: row t is sequence t (its output row was zeroed)
  if (wfn == kWeightsSigmoid) {   // unnormalised weights: the shares simply add up
    const float gh = (gate && !gate_elem) ? sigmoidf(bf2f(gate[(int64_t)t * ld_gate + h])) : 1.f;
    for (int d = threadIdx.x; d < dv; d += blockDim.x) {
      float acc = 0.f;
      for (int sp = 0; sp < nsplit; ++sp) acc += part_o[(((int64_t)sp * Ttot + t) * H + h) * dv + d];
      if (gate && gate_elem) acc *= sigmoidf(bf2f(gate[(int64_t)t * ld_gate + (int64_t)h * dv + d]));
      out[((int64_t)t * H + h) * dv + d] = f2bf(acc * gh);
    }
    return;
  }
  float M = -INFINITY;
  for (int sp = 0; sp < nsplit; ++sp) M = fmaxf(M, part_ml[2 * (((int64_t)sp * Ttot + t) * H + h)]);
  float L = 0.f;
  for (int sp = 0; sp < nsplit; ++sp) {
    const int64_t row = ((int64_t)sp * Ttot + t) * H + h;
    const float ms = part_ml[2 * row];
    if (ms != -INFINITY) L += exp2_fast(ms - M) * part_ml[2 * row + 1];
  }
  float inv = L > 0.f ? 1.f / L : 0.f;
  if (gate && !gate_elem) inv *= sigmoidf(bf2f(gate[(int64_t)t * ld_gate + h]));
  for (int d = threadIdx.x; d < dv; d += blockDim.x) {
    float acc = 0.f;
    for (int sp = 0; sp < nsplit; ++sp) {
      const int64_t row = ((int64_t)sp * Ttot + t) * H + h;
      const float ms = part_ml[2 * row];
      if (ms != -INFINITY) acc += exp2_fast(ms - M) * part_o[row * dv + d];
    }
    acc *= inv;
    if (gate && gate_elem) acc *= sigmoidf(bf2f(gate[(int64_t)t * ld_gate + (int64_t)h * dv + d]));
    out[((int64_t)t * H + h) * dv + d] = f2bf(acc);
  }
}

// ------------------------------------------------------------------ heads' weight maps mixed after the softmax
// o_all[t][g][c][:] = p_g V_c for every query head g and key/value head c; head h's mixed weights
// sum_g talk[h][g] p_g applied to the values of its own key/value head c(h) are sum_g talk[h][g] o_all[t][g][c(h)].
template <typename T>
__global__ __launch_bounds__(256) void talk_mix_kernel(const T* __restrict__ o_all, const float* __restrict__ talk,
                                                       const T* __restrict__ gate, int64_t ld_gate, T* __restrict__ out,
                                                       int H, int G, int dv) {
  const int t = blockIdx.x;
  const int rep = H / G;
  const T* row = o_all + (int64_t)t * H * G * dv;
  if ((dv & 3) == 0) {  // four value columns per thread
    for (int e = threadIdx.x; e < H * dv / 4; e += blockDim.x) {
      const int h = e / (dv / 4), d = 4 * (e % (dv / 4));
      const int c = h / rep;
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      for (int g = 0; g < H; ++g) {
        float v[4];
        ld4(row + ((int64_t)g * G + c) * dv + d, v);
        const float w = talk[h * H + g];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += w * v[i];
      }
      if (gate) {
        const float sg = sigmoidf(ldf(gate + (int64_t)t * ld_gate + h));
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] *= sg;
      }
      st4(out + (int64_t)t * H * dv + h * dv + d, acc);
    }
    return;
  }
  for (int e = threadIdx.x; e < H * dv; e += blockDim.x) {
    const int h = e / dv, d = e % dv;
    const int c = h / rep;
    float acc = 0.f;
    for (int g = 0; g < H; ++g) acc += talk[h * H + g] * ldf(row + ((int64_t)g * G + c) * dv + d);
    if (gate) acc *= sigmoidf(ldf(gate + (int64_t)t * ld_gate + h));
    stf(out + (int64_t)t * H * dv + e, acc);
  }
}

// ------------------------------------------------------------------ q / k norm + rotation -> q, cache rows
// One workgroup per token; a wave takes the heads (H query heads, then G key heads) round robin. A lane owns the
// entries d = lane, lane + 64, ... of a head; the partner of a rotated entry is re-read (it is in the same row).
// whole: q and k are normed over all their entries at once (weights of size H dk / G dk) instead of head by head.
// half: the rotation pairs entry i with i + rot_dims / 2 instead of 2i with 2i + 1.
// v_first / v_mix: the cached values are (1 - lambda) v + lambda v_first, lambda = *v_mix.
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void head_norm_rope_cache_kernel(
    const TI* __restrict__ src, int64_t ld, int H, int G, int dk, int dv, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ rot, int rot_rows, int rot_dims,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slot_mapping, TO* __restrict__ q_out,
    TO* __restrict__ kcache, TO* __restrict__ vcache, int whole, int half, const TI* __restrict__ v_first,
    int64_t ld_vf, const float* __restrict__ v_mix, int vec) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const TI* row = src + (int64_t)t * ld;
  const int slot = slot_mapping[t];
  const int nq = H * dk, nk = G * dk, nv = G * dv;
  const float* cs = nullptr;
  if (rot && rot_dims > 0) cs = rot + (int64_t)min(max(positions[t], 0), rot_rows - 1) * rot_dims;  // [rot_dims / 2][2]
  float rq = 1.f, rk = 1.f;
  if (whole) {
    if (wq) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < nq; c += blockDim.x) {
        const float a = ldf(row + c);
        ss += a * a;
      }
      rq = 1.f / sqrtf(block_sum(ss, red) / (float)nq + eps);
    }
    if (wk) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < nk; c += blockDim.x) {
        const float a = ldf(row + nq + c);
        ss += a * a;
      }
      rk = 1.f / sqrtf(block_sum(ss, red) / (float)nk + eps);
    }
  }
  const int hr = rot_dims / 2;
  if (vec) {
    // four consecutive entries per thread (no per-head statistic to wait for): a pair lies inside the quad
    // (2i, 2i + 1) or in the quad rot_dims / 2 further on / back (i, i + rot_dims / 2)
    const int qpd = dk / 4;   // quads per head
    for (int e = threadIdx.x; e < (H + G) * qpd; e += blockDim.x) {
      const int hd = e / qpd, d0 = 4 * (e % qpd);
      const bool is_q = hd < H;
      if (!is_q && slot < 0) continue;
      const int hh = is_q ? hd : hd - H;
      const TI* v = row + (is_q ? hd * dk : nq + hh * dk);
      const float* w = is_q ? wq : wk;
      const float* wh = w ? w + hh * dk : nullptr;   // whole-vector weights
      const float r = is_q ? rq : rk;
      float a[4], g[4] = {1.f, 1.f, 1.f, 1.f};
      ld4(v + d0, a);
      if (wh) ld4(wh + d0, g);
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] *= r * g[i];
      if (cs && d0 < rot_dims) {
        if (half) {
          const bool second = d0 >= hr;
          const int pd0 = second ? d0 - hr : d0 + hr, pi = second ? d0 - hr : d0;
          float b[4], cs0[4], cs1[4];
          ld4(v + pd0, b);
          if (wh) ld4(wh + pd0, g);
          ld4(cs + 2 * pi, cs0);        // (c, s) of pairs pi, pi + 1
          ld4(cs + 2 * pi + 4, cs1);    // ... pi + 2, pi + 3
          const float c[4] = {cs0[0], cs0[2], cs1[0], cs1[2]}, sn[4] = {cs0[1], cs0[3], cs1[1], cs1[3]};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float bb = b[i] * r * g[i];
            a[i] = second ? a[i] * c[i] + bb * sn[i] : a[i] * c[i] - bb * sn[i];
          }
        } else {
          float cq[4];
          ld4(cs + d0, cq);             // (c, s) of pairs d0 / 2, d0 / 2 + 1
          const float u0 = a[0], v0 = a[1], u1 = a[2], v1 = a[3];
          a[0] = u0 * cq[0] - v0 * cq[1];
          a[1] = v0 * cq[0] + u0 * cq[1];
          a[2] = u1 * cq[2] - v1 * cq[3];
          a[3] = v1 * cq[2] + u1 * cq[3];
        }
      }
      st4((is_q ? q_out + (int64_t)t * nq + hd * dk : kcache + (int64_t)slot * nk + hh * dk) + d0, a);
    }
    if (slot >= 0) {
      const float lam = v_first ? *v_mix : 0.f;
      for (int c = 4 * threadIdx.x; c < nv; c += 4 * blockDim.x) {
        float a[4];
        ld4(row + nq + nk + c, a);
        if (v_first) {
          float b[4];
          ld4(v_first + (int64_t)t * ld_vf + c, b);
#pragma unroll
          for (int i = 0; i < 4; ++i) a[i] = (1.f - lam) * a[i] + lam * b[i];
        }
        st4(vcache + (int64_t)slot * nv + c, a);
      }
    }
    return;
  }
  for (int hd = wave; hd < H + G; hd += nw) {
    const bool is_q = hd < H;
    if (!is_q && slot < 0) continue;   // padding row: nothing is cached
    const int hh = is_q ? hd : hd - H;
    const TI* v = row + (is_q ? hd * dk : nq + hh * dk);
    const float* w = is_q ? wq : wk;
    const float* wh = (w && whole) ? w + hh * dk : w;   // this head's weights
    TO* dst = is_q ? q_out + (int64_t)t * nq + hd * dk : kcache + (int64_t)slot * nk + hh * dk;
    float r = is_q ? rq : rk;
    if (w && !whole) {
      float ss = 0.f;
      for (int d = lane; d < dk; d += 64) {
        const float a = ldf(v + d);
        ss += a * a;
      }
      r = 1.f / sqrtf(wave_sum(ss) / (float)dk + eps);
    }
    for (int d = lane; d < dk; d += 64) {
      float a = ldf(v + d) * r * (w ? wh[d] : 1.f);
      if (cs && d < rot_dims) {
        const int pd = half ? (d < hr ? d + hr : d - hr) : (d ^ 1);     // the other entry of the pair
        const bool second = half ? d >= hr : (d & 1);
        const int pi = half ? (d < hr ? d : d - hr) : (d >> 1);         // the pair's index
        const float b = ldf(v + pd) * r * (w ? wh[pd] : 1.f);
        const float c = cs[2 * pi], sn = cs[2 * pi + 1];
        a = second ? a * c + b * sn : a * c - b * sn;   // (u, v) -> (u c - v s, v c + u s)
      }
      stf(dst + d, a);
    }
  }
  if (slot >= 0) {
    if (v_first) {
      const float lam = *v_mix;
      for (int c = threadIdx.x; c < nv; c += blockDim.x)
        stf(vcache + (int64_t)slot * nv + c,
            (1.f - lam) * ldf(row + nq + nk + c) + lam * ldf(v_first + (int64_t)t * ld_vf + c));
    } else {
      for (int c = threadIdx.x; c < nv; c += blockDim.x) stf(vcache + (int64_t)slot * nv + c, ldf(row + nq + nk + c));
    }
  }
}

// ------------------------------------------------------------------ short convolution + per-head norm + rotation
// The same as head_norm_rope_cache on the outputs of a causal depthwise convolution over time of the projected row
// [q | k | v] (taps <= 8, weights conv_w[channel][tap], no bias), formed here: channel c of the token at local index i
// of its sequence's rows reads rows i - taps + 1 .. i of this step, or, before the step's first row, the sequence's
// carried inputs state[slot][taps - 1 + index][c] (zero before the sequence's start). A lane owns the entries
// d = lane + 64 n (n < NR) of a head, a wave one head, further workgroups the value channels; rotation partners are
// neighbouring lanes. Steps of single tokens shift the
// carried inputs here (each thread reads and writes only its own channels); longer steps leave that to a second launch.
constexpr int kConvMaxTaps = 8;

template <typename TI, typename TO, int NR>
__global__ __launch_bounds__(256) void conv_head_norm_rope_cache_kernel(
    const TI* __restrict__ proj, int64_t ld, const float* __restrict__ conv_w, int taps, float* __restrict__ state,
    const int32_t* __restrict__ qsl, const int32_t* __restrict__ seq_lens, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ token_seq, int H, int G, int dk, int dv, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const float* __restrict__ rot, int rot_rows, int rot_dims,
    const int32_t* __restrict__ slot_mapping, TO* __restrict__ q_out, TO* __restrict__ kcache, TO* __restrict__ vcache,
    int single) {
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int nq = H * dk, nk = G * dk, nv = G * dv, C = nq + nk + nv;
  // blockIdx.y < nhb: one head per wave (H query heads, then G key heads); beyond: 256 value channels per workgroup
  const int nhb = (H + G + nw - 1) / nw;
  const int s = token_seq[t];
  const int slot = s >= 0 ? slots[s] : -1;
  if (slot < 0) {  // padding row: a defined q row, nothing cached, no state touched
    const int hd = blockIdx.y * nw + wave;
    if ((int)blockIdx.y < nhb && hd < H)
      for (int d = lane; d < dk; d += 64) stf(q_out + (int64_t)t * nq + hd * dk + d, 0.f);
    return;
  }
  const int q0 = qsl[s], qn = qsl[s + 1] - q0;
  const int ctx = seq_lens[s] - qn, li = t - q0, nh = taps - 1;
  const int crow = slot_mapping[t];
  const float* st = state + (int64_t)slot * nh * C;
  // the convolution of channel c at this token; a single-token step also shifts the channel's carried inputs
  auto conv = [&](int c) -> float {
    float u[kConvMaxTaps];
#pragma unroll
    for (int j = 0; j < kConvMaxTaps; ++j) {
      u[j] = 0.f;
      if (j < taps) {
        const int idx = li - nh + j;   // local index of the input under tap j
        if (idx >= 0) u[j] = ldf(proj + (int64_t)(q0 + idx) * ld + c);
        else if (ctx + idx >= 0) u[j] = st[(int64_t)(nh + idx) * C + c];
      }
    }
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < kConvMaxTaps; ++j)
      if (j < taps) acc += conv_w[(int64_t)c * taps + j] * u[j];
    if (single) {   // carried inputs after this token: u[1 .. taps - 1] (already zero before the sequence's start)
      float* sw = state + (int64_t)slot * nh * C + c;
#pragma unroll
      for (int j = 1; j < kConvMaxTaps; ++j)
        if (j < taps) sw[(int64_t)(j - 1) * C] = u[j];
    }
    return acc;
  };
  const float* cs = nullptr;
  if (rot && rot_dims > 0) cs = rot + (int64_t)min(max(ctx + li, 0), rot_rows - 1) * rot_dims;  // [rot_dims / 2][2]
  if ((int)blockIdx.y >= nhb) {
    const int c = ((int)blockIdx.y - nhb) * blockDim.x + threadIdx.x;
    if (c < nv && (crow >= 0 || single)) {
      const float v = conv(nq + nk + c);
      if (crow >= 0) stf(vcache + (int64_t)crow * nv + c, v);
    }
    return;
  }
  for (int hd = blockIdx.y * nw + wave; hd < H + G; hd += H + G) {   // one pass
    const bool is_q = hd < H;
    if (!is_q && crow < 0 && !single) continue;
    const int c0 = is_q ? hd * dk : nq + (hd - H) * dk;
    const float* w = is_q ? wq : wk;
    float a[NR], ss = 0.f;
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int d = lane + 64 * n;
      a[n] = d < dk ? conv(c0 + d) : 0.f;
      ss += a[n] * a[n];
    }
    if (!is_q && crow < 0) continue;
    const float r = w ? 1.f / sqrtf(wave_sum(ss) / (float)dk + eps) : 1.f;
    TO* dst = is_q ? q_out + (int64_t)t * nq + hd * dk : kcache + (int64_t)crow * nk + (hd - H) * dk;
#pragma unroll
    for (int n = 0; n < NR; ++n) {
      const int d = lane + 64 * n;
      float v = d < dk ? a[n] * r * (w ? w[d] : 1.f) : 0.f;
      const float b = __shfl_xor(v, 1, 64);   // the other entry of the pair (2i, 2i + 1)
      if (cs && d < rot_dims) {
        const float c = cs[d & ~1], sn = cs[(d & ~1) + 1];
        v = (d & 1) ? v * c + b * sn : v * c - b * sn;   // (u, v) -> (u c - v s, v c + u s)
      }
      if (d < dk) stf(dst + d, v);
    }
  }
}

// ================================================================== host launchers
void qk_norm_cache(const void* proj, bool f32, int64_t ld, int nq, int nk, int nv, const float* wq, const float* wk,
                   float eps, const int32_t* slot_mapping, void* q_out, void* kcache, void* vcache, int T_,
                   hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, qk_norm_cache_kernel<T><<<T_, 256, 0, st>>>((const T*)proj, ld, nq, nk, nv, wq, wk, eps, slot_mapping,
                                                                   (T*)q_out, (T*)kcache, (T*)vcache);)
}

template <typename T, int NR>
static int launch_masked_attention(const void* q, const void* kcache, const void* vcache, const int32_t* block_tables,
                                   int bt_width, int bs, const int32_t* positions, const int32_t* token_seq,
                                   const float* temp, const float* sink, void* out, int T_, int H, int G, int dk,
                                   int dv_head, int mask, int size, float scale, const void* gate, int64_t ld_gate,
                                   const float* r1, const float* r2, int vmode, int gate_elem, int wfn,
                                   const float* hbias, hipStream_t st) {
  const int dv = vmode == kValuesAll ? G * dv_head : dv_head;
  int KT = 64;
  auto bytes = [&](int kt) { return ((size_t)kt * (dk + dv + 2) + (size_t)4 * kQPW * dk) * sizeof(float); };
  while (KT > 4 && bytes(KT) > 60 * 1024) KT >>= 1;
  if (bytes(KT) > 64 * 1024) return -2;
  const int rep = H / G;
  dim3 grid(T_, G, (rep + 4 * kQPW - 1) / (4 * kQPW));
  masked_attention_kernel<T, NR><<<grid, 256, bytes(KT), st>>>((const T*)q, (const T*)kcache, (const T*)vcache,
                                                               block_tables, bt_width, bs, positions, token_seq, temp,
                                                               sink, (T*)out, H, G, dk, dv_head, mask, size, scale, KT,
                                                               (const T*)gate, ld_gate, r1, r2, vmode, gate_elem, wfn,
                                                               hbias);
  return 0;
}

int masked_attention(const void* q, bool f32, const void* kcache, const void* vcache, const int32_t* block_tables,
                     int bt_width, int bs, const int32_t* positions, const int32_t* token_seq, const float* temp,
                     const float* sink, void* out, int T_, int H, int G, int dk, int dv_head, int mask, int size,
                     float scale, const void* gate, int64_t ld_gate, const float* r1, const float* r2, int vmode,
                     bool gate_elem, int wfn, const float* hbias, hipStream_t st) {
  if (T_ <= 0) return 0;
  const int dv = vmode == kValuesAll ? G * dv_head : dv_head;
  if (G <= 0 || H % G != 0 || dk <= 0 || dv <= 0 || dv > 512 || mask < 0 || mask > 2 ||
      (mask != kMaskCausal && size < 1) || vmode < kValuesAll || vmode >= G || (r1 && !r2) ||
      (gate_elem && vmode != kValuesOwn) || wfn < 0 || wfn > 1 || (wfn == kWeightsSigmoid && sink))
    return -1;
#define XGM_MA(NR)                                                                                                     \
  XGM_DISPATCH_T(f32, return (launch_masked_attention<T, NR>(q, kcache, vcache, block_tables, bt_width, bs, positions, \
                                                             token_seq, temp, sink, out, T_, H, G, dk, dv_head, mask,  \
                                                             size, scale, gate, ld_gate, r1, r2, vmode,             \
                                                             gate_elem ? 1 : 0, wfn, hbias, st));)
  if (dv <= 64) { XGM_MA(1) }
  if (dv <= 128) { XGM_MA(2) }
  if (dv <= 256) { XGM_MA(4) }
  XGM_MA(8)
#undef XGM_MA
}


int masked_attention_mfma(const void* q, const void* kcache, const void* vcache, const int32_t* block_tables, int bt_width,
                          int bs, const int32_t* qsl, const int32_t* seq_lens, const int32_t* slots, const float* temp,
                          const float* sink, void* out, int T_, int ns, int max_q, int H, int G, int dk, int dv_head,
                          int mask, int size, float scale, int nsplit, float* part_o, float* part_ml, const void* gate,
                          int64_t ld_gate, const float* r1, const float* r2, int vmode, int nw_hint, bool gate_elem,
                          int wfn, const float* hbias, hipStream_t st) {
  if (T_ <= 0 || ns <= 0 || max_q <= 0) return 0;
  const int dv = vmode == kValuesAll ? G * dv_head : dv_head;
  if (G <= 0 || H % G != 0 || dk % 32 != 0 || dv % 16 != 0 || dk > 128 || dv > 256 || mask < 0 || mask > 2 ||
      (mask != kMaskCausal && size < 1) || vmode < kValuesAll || vmode >= G || (r1 && !r2) ||
      (gate_elem && vmode != kValuesOwn) || wfn < 0 || wfn > 1 || (wfn == kWeightsSigmoid && sink))
    return -1;
  const int ge = gate_elem ? 1 : 0;
  const int rep = H / G;
  const int RH = rep >= 4 ? 4 : rep >= 2 ? 2 : 1;
  // a step of single tokens: one workgroup per (sequence, key/value head), its query heads as the slots
  const int head_slots = (max_q == 1 && T_ == ns) ? 1 : 0;
  if (head_slots && rep > 64) return -3;
  // waves per workgroup: 4 for single tokens and short portions, 8 for long portions (twice the token tiles of the same
  // heads on every staged key tile; 16 waves measured slower: the early tiles of a 64-token span idle at the late keys)
  int nw = (head_slots || max_q <= 32) ? 4 : 8;
  if (!head_slots && (nw_hint == 4 || nw_hint == 8 || (nw_hint == 16 && dv <= 128))) nw = nw_hint;
  const int tpb = nw / RH;
  dim3 grid((max_q + 16 * tpb - 1) / (16 * tpb), G * ((rep + RH - 1) / RH), ns);
  if (!head_slots || nsplit < 1 || (nsplit > 1 && (!part_o || !part_ml))) nsplit = 1;
  if (head_slots) grid = dim3(nsplit, G, ns);
  const size_t lds = (size_t)kKT * (dk + 8 + dv + 8) * sizeof(uint16_t);
#define XGM_MK2(NKK, NMT, NW, WFN)                                                                                    \
  masked_attention_mfma_kernel<NKK, NMT, NW, WFN><<<grid, 64 * NW, lds, st>>>(                                        \
      (const bf16*)q, (const bf16*)kcache, (const bf16*)vcache, block_tables, bt_width, bs, qsl, seq_lens, slots, temp, \
      sink, (bf16*)out, H, G, dk, dv_head, mask, size, scale, RH, head_slots, part_o, part_ml, T_, (const bf16*)gate,  \
      ld_gate, r1, r2, vmode, ge, hbias);
#define XGM_MK(NKK, NMT, NW)                  \
  if (wfn == kWeightsSigmoid) {               \
    XGM_MK2(NKK, NMT, NW, kWeightsSigmoid)    \
  } else {                                    \
    XGM_MK2(NKK, NMT, NW, kWeightsSoftmax)    \
  }
#define XGM_MM(NKK, NMT)                                                                                              \
  if (nw == 16 && NMT <= 8) {                                                                                         \
    XGM_MK(NKK, NMT, (NMT <= 8 ? 16 : 8))                                                                             \
  } else if (nw >= 8) {                                                                                               \
    XGM_MK(NKK, NMT, 8)                                                                                               \
  } else {                                                                                                            \
    XGM_MK(NKK, NMT, 4)                                                                                               \
  }                                                                                                                   \
  if (nsplit > 1)                                                                                                     \
    masked_attention_combine_kernel<<<dim3(T_, H), 64, 0, st>>>(part_o, part_ml, slots, (bf16*)out, T_, H, dv, nsplit, \
                                                                (const bf16*)gate, ld_gate, ge, wfn);                 \
  return 0;
  if (dk <= 64 && dv <= 64) { XGM_MM(2, 4) }
  if (dk <= 128 && dv <= 128) { XGM_MM(4, 8) }
  if (dk <= 128 && dv <= 256) { XGM_MM(4, 16) }
  return -2;
#undef XGM_MM
#undef XGM_MK
#undef XGM_MK2
}

void talk_mix(const void* o_all, bool f32, const float* talk, const void* gate, int64_t ld_gate, void* out, int T_, int H,
              int G, int dv, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, talk_mix_kernel<T><<<T_, 256, 0, st>>>((const T*)o_all, talk, (const T*)gate, ld_gate, (T*)out, H, G,
                                                              dv);)
}

void head_norm_rope_cache(const void* src, bool src_f32, int64_t ld, int H, int G, int dk, int dv, const float* wq,
                          const float* wk, float eps, const float* rot, int rot_rows, int rot_dims,
                          const int32_t* positions, const int32_t* slot_mapping, void* q_out, void* kcache, void* vcache,
                          bool out_f32, int T_, bool whole, bool half, const void* v_first, int64_t ld_vf,
                          const float* v_mix, hipStream_t st) {
  if (T_ <= 0) return;
  // four entries per thread where no per-head statistic is needed (no norm, or norms over the whole vectors) and
  // quads stay whole: head sizes, value rows and strides multiples of 4, rotated pairs inside a quad (2i, 2i + 1) or
  // a whole number of quads apart (i, i + n / 2), rows aligned to 16 (float) / 8 (bf16) bytes
  const int isz = src_f32 ? 4 : 2, osz = out_f32 ? 4 : 2;
  const bool use_rot = rot && rot_dims > 0;
  const int vec = ((!wq && !wk) || whole) && dk % 4 == 0 && (G * dv) % 4 == 0 && ld % 4 == 0 &&
                  (uintptr_t)src % (4 * isz) == 0 && (uintptr_t)q_out % (4 * osz) == 0 &&
                  (uintptr_t)kcache % (4 * osz) == 0 && (uintptr_t)vcache % (4 * osz) == 0 &&
                  (!use_rot || (half ? rot_dims % 8 == 0 : rot_dims % 4 == 0)) &&
                  (!v_first || (ld_vf % 4 == 0 && (uintptr_t)v_first % (4 * isz) == 0));
#define XGM_HN(TI, TO)                                                                                               \
  head_norm_rope_cache_kernel<TI, TO><<<T_, 256, 0, st>>>((const TI*)src, ld, H, G, dk, dv, wq, wk, eps, rot, rot_rows, \
                                                          rot_dims, positions, slot_mapping, (TO*)q_out, (TO*)kcache,  \
                                                          (TO*)vcache, whole ? 1 : 0, half ? 1 : 0, (const TI*)v_first, \
                                                          ld_vf, v_mix, vec);
  if (src_f32) {
    if (out_f32) { XGM_HN(float, float) } else { XGM_HN(float, bf16) }
  } else {
    if (out_f32) { XGM_HN(bf16, float) } else { XGM_HN(bf16, bf16) }
  }
#undef XGM_HN
}

void conv_state_update(const void* x, bool in_f32, int64_t ld_in, float* state, const int32_t* qsl,
                       const int32_t* seq_lens, const int32_t* slots, int ns, int W, int taps, hipStream_t st);

int conv_head_norm_rope_cache(const void* proj, bool in_f32, int64_t ld, const float* conv_w, int taps, float* state,
                              const int32_t* qsl, const int32_t* seq_lens, const int32_t* slots, const int32_t* token_seq,
                              int ns, int max_q, int H, int G, int dk, int dv, const float* wq, const float* wk, float eps,
                              const float* rot, int rot_rows, int rot_dims, const int32_t* slot_mapping, void* q_out,
                              void* kcache, void* vcache, bool out_f32, int T_, hipStream_t st) {
  if (T_ <= 0) return 0;
  if (taps < 1 || taps > kConvMaxTaps || dk > 256 || dk < 1) return -1;
  const int single = (max_q == 1 && taps > 1) ? 1 : 0;
  dim3 grid(T_, (H + G + 3) / 4 + (G * dv + 255) / 256);
#define XGM_CH2(TI, TO, NR)                                                                                          \
  conv_head_norm_rope_cache_kernel<TI, TO, NR><<<grid, 256, 0, st>>>(                                                \
      (const TI*)proj, ld, conv_w, taps, state, qsl, seq_lens, slots, token_seq, H, G, dk, dv, wq, wk, eps, rot,     \
      rot_rows, rot_dims, slot_mapping, (TO*)q_out, (TO*)kcache, (TO*)vcache, single);
#define XGM_CH(TI, TO)                                                                                               \
  if (dk <= 64) {                                                                                                    \
    XGM_CH2(TI, TO, 1)                                                                                               \
  } else if (dk <= 128) {                                                                                            \
    XGM_CH2(TI, TO, 2)                                                                                               \
  } else {                                                                                                           \
    XGM_CH2(TI, TO, 4)                                                                                               \
  }
  if (in_f32) {
    if (out_f32) { XGM_CH(float, float) } else { XGM_CH(float, bf16) }
  } else {
    if (out_f32) { XGM_CH(bf16, float) } else { XGM_CH(bf16, bf16) }
  }
#undef XGM_CH
#undef XGM_CH2
  if (!single) conv_state_update(proj, in_f32, ld, state, qsl, seq_lens, slots, ns, (H + G) * dk + G * dv, taps, st);
  return 0;
}

}  // namespace xgm
