// pybind11 entry points of xgserve._mixers: raw device pointers + the caller's hipStream_t
// (graph-capturable, no dependence on torch's C++ ABI). Shapes are checked here, before launch.
#include <hip/hip_runtime.h>
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

namespace py = pybind11;

namespace xgm {
void embed_rows(const int32_t*, const void*, bool, float*, int, int, int, const void*, const int32_t*, int, float,
                hipStream_t);
void causal_conv(const void*, bool, int64_t, const float*, const float*, float*, const int32_t*, const int32_t*,
                 const int32_t*, void*, bool, int, int, int, int, bool, bool, hipStream_t);
int residual_norm(float*, const void*, int64_t, const float*, const void*, int64_t, const float*, const float*, bool,
                  const float*, float, float*, void*, bool, int, int, int, const float*, const float*, const int32_t*,
                  const float*, int, hipStream_t);
void qk_norm_cache(const void*, bool, int64_t, int, int, int, const float*, const float*, float, const int32_t*, void*,
                   void*, void*, int, hipStream_t);
int masked_attention(const void*, bool, const void*, const void*, const int32_t*, int, int, const int32_t*,
                     const int32_t*, const float*, const float*, void*, int, int, int, int, int, int, int, float,
                     const void*, int64_t, const float*, const float*, int, bool, int, const float*, hipStream_t);
int masked_attention_mfma(const void*, const void*, const void*, const int32_t*, int, int, const int32_t*, const int32_t*,
                          const int32_t*, const float*, const float*, void*, int, int, int, int, int, int, int, int, int,
                          float, int, float*, float*, const void*, int64_t, const float*, const float*, int, int, bool, int,
                          const float*, hipStream_t);
void talk_mix(const void*, bool, const float*, const void*, int64_t, void*, int, int, int, int, hipStream_t);
void head_norm_rope_cache(const void*, bool, int64_t, int, int, int, int, const float*, const float*, float, const float*,
                          int, int, const int32_t*, const int32_t*, void*, void*, void*, bool, int, bool, bool, const void*,
                          int64_t, const float*, hipStream_t);
int conv_head_norm_rope_cache(const void*, bool, int64_t, const float*, int, float*, const int32_t*, const int32_t*,
                              const int32_t*, const int32_t*, int, int, int, int, int, int, const float*, const float*,
                              float, const float*, int, int, const int32_t*, void*, void*, void*, bool, int, hipStream_t);
int post_norm_residual(float*, const void*, bool, int64_t, const float*, const void*, int64_t, const float*, const float*,
                       const float*, float, const float*, const float*, float, float, void*, bool, int, int, hipStream_t);
void relu2(const void*, bool, const float*, void*, int64_t, int, hipStream_t);
void lower_bound_gates(const void*, bool, int64_t, int, int, int, const float*, const float*, float*, float*, int,
                       hipStream_t);
int gated_linear_scan(const float*, const float*, const float*, const void*, int64_t, int, int, const float*, const float*,
                      const void*, bool, int64_t, float*, const int32_t*, const int32_t*, const int32_t*, float*, int, int,
                      int, int, int, float*, int, int, hipStream_t);
int64_t gated_linear_scan_scratch_floats(int, int, int, int, int);
int ssm_scan(const void*, bool, int64_t, const void*, int64_t, const float*, const float*, const float*, float*,
             const int32_t*, const int32_t*, const int32_t*, float*, int, int, int, int, int, hipStream_t);
void gated_group_norm(const float*, const void*, bool, int64_t, const float*, int, float, void*, int, int, int, bool,
                      hipStream_t);
void glu_act(const void*, bool, int64_t, void*, int, int, int, float, float, hipStream_t);
int grouped_router(const float*, const float*, int, int, int, int, int, float, int32_t*, float*, const float*,
                   const float*, int, hipStream_t);
int moe_align(const int32_t*, int, int, int, int, int32_t*, int32_t*, int32_t*, hipStream_t);
int grouped_gemm(const void*, bool, int64_t, const void*, const int32_t*, const int32_t*, int, int, int, int, int, int, void*,
                 int, float, float, const float*, bool, hipStream_t);
int mingru_scan(const void*, bool, int64_t, int, int, int, int, const float*, const float*, float*, const int32_t*,
                const int32_t*, const int32_t*, void*, bool, int, int, float*, int, hipStream_t);
int64_t mingru_scratch_floats(int, int, int);
void decay_gates(const void*, bool, int64_t, int, int, int, float, const void*, int64_t, const float*, float, float*, float*,
                 float*, int, hipStream_t);
void moe_combine(const float*, const int32_t*, const float*, int, int, int, float*, hipStream_t);
void canon_conv(const float*, const float*, float*, const int32_t*, const int32_t*, const int32_t*, void*, bool, int, int,
                int, int, hipStream_t);
void scaled_add_rmsnorm(const float*, const void*, bool, int64_t, const float*, float, const float*, float, float, float*,
                        void*, bool, int, int, hipStream_t);
void latent_prep(const void*, bool, int64_t, int, int, int, int, int, const float*, const float*, float, const int32_t*,
                 const int32_t*, const float*, int, void*, void*, int, hipStream_t);
int latent_attention(const void*, const void*, bool, int64_t, int, int, const void*, int64_t, const void*, const int32_t*,
                     int, int, const int32_t*, const int32_t*, const float*, int, void*, int, int, int, int, int, float,
                     hipStream_t);
int latent_attention_mfma(const void*, const void*, int, int, const void*, int64_t, const void*, const int32_t*, int, int,
                          const int32_t*, const int32_t*, const int32_t*, const float*, int, void*, int, int, int, int, int,
                          int, int, float, int, float*, float*, hipStream_t);
int delta_scan(const void*, bool, int64_t, int, int, int, int, const void*, int64_t, const float*, const float*, float*,
               const int32_t*, const int32_t*, const int32_t*, float*, int, int, int, float*, int, hipStream_t);
void delta_out(const float*, const float*, const void*, bool, int64_t, float, void*, int, int, int, hipStream_t);
void xielu(const void*, bool, const float*, float, float, void*, int64_t, int, hipStream_t);
void tanh_cols(const void*, bool, int64_t, void*, int, int, hipStream_t);
void heads_to_rows(const void*, bool, void*, int, int, int, hipStream_t);
}  // namespace xgm

template <typename T> static T* P(uintptr_t p) { return reinterpret_cast<T*>(p); }
static hipStream_t S(uintptr_t s) { return reinterpret_cast<hipStream_t>(s); }

static void check(int rc, const char* what) {
  if (rc != 0) throw std::invalid_argument(std::string(what) + ": unsupported shape (code " + std::to_string(rc) + ")");
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

PYBIND11_MODULE(_mixers, m) {
  m.def("embed_rows", [](uintptr_t ids, uintptr_t table, bool f32, uintptr_t out, int T, int W, int V, uintptr_t pos_table,
                         uintptr_t positions, int Pn, float scale, uintptr_t st) {
    if (pos_table && !positions) throw std::invalid_argument("embed_rows: a position table needs positions");
    xgm::embed_rows(P<const int32_t>(ids), P<const void>(table), f32, P<float>(out), T, W, V, P<const void>(pos_table),
                    P<const int32_t>(positions), Pn, scale, S(st));
    check(0, "embed_rows");
  });
  m.def("causal_conv", [](uintptr_t x, bool in_f32, int64_t ld_in, uintptr_t w, uintptr_t bias, uintptr_t state,
                          uintptr_t qsl, uintptr_t sl, uintptr_t slots, uintptr_t out, bool out_f32, int ns, int max_q,
                          int C, int taps, bool residual, bool act, uintptr_t st) {
    if (taps < 1 || taps > 8) throw std::invalid_argument("causal_conv: taps must be in [1, 8]");
    if (ld_in < C) throw std::invalid_argument("causal_conv: row stride smaller than the channel count");
    xgm::causal_conv(P<const void>(x), in_f32, ld_in, P<const float>(w), P<const float>(bias), P<float>(state),
                     P<const int32_t>(qsl), P<const int32_t>(sl), P<const int32_t>(slots), P<void>(out), out_f32, ns,
                     max_q, C, taps, residual, act, S(st));
    check(0, "causal_conv");
  });
  m.def("residual_norm", [](uintptr_t x, uintptr_t y1, int64_t ld1, uintptr_t a1, uintptr_t y2, int64_t ld2, uintptr_t y3,
                            uintptr_t a2, bool y_f32, uintptr_t g, float eps, uintptr_t n32, uintptr_t nact,
                            bool nact_f32, int T, int W, int groups, uintptr_t bw1, uintptr_t bw2, uintptr_t dest,
                            uintptr_t cw, int top, uintptr_t st) {
    if ((y1 && ld1 < W) || (y2 && ld2 < W)) throw std::invalid_argument("residual_norm: row stride smaller than the width");
    int rc = xgm::residual_norm(P<float>(x), P<const void>(y1), ld1, P<const float>(a1), P<const void>(y2), ld2,
                                P<const float>(y3), P<const float>(a2), y_f32, P<const float>(g), eps, P<float>(n32),
                                P<void>(nact), nact_f32, T, W, groups, P<const float>(bw1), P<const float>(bw2),
                                P<const int32_t>(dest), P<const float>(cw), top, S(st));
    check(rc, "residual_norm");
  });
  m.def("qk_norm_cache", [](uintptr_t proj, bool f32, int64_t ld, int nq, int nk, int nv, uintptr_t wq, uintptr_t wk,
                            float eps, uintptr_t slot_mapping, uintptr_t q_out, uintptr_t kcache, uintptr_t vcache, int T,
                            uintptr_t st) {
    if (nq < 1 || nk < 1 || nv < 1 || ld < nq + nk + nv) throw std::invalid_argument("qk_norm_cache: inconsistent sizes");
    xgm::qk_norm_cache(P<const void>(proj), f32, ld, nq, nk, nv, P<const float>(wq), P<const float>(wk), eps,
                       P<const int32_t>(slot_mapping), P<void>(q_out), P<void>(kcache), P<void>(vcache), T, S(st));
    check(0, "qk_norm_cache");
  });
  m.def("masked_attention", [](uintptr_t q, bool f32, uintptr_t kc, uintptr_t vc, uintptr_t bt, int bt_width, int bs,
                               uintptr_t pos, uintptr_t token_seq, uintptr_t temp, uintptr_t sink, uintptr_t out, int T,
                               int H, int G, int dk, int dv, int mask, int size, float scale, uintptr_t gate,
                               int64_t ld_gate, uintptr_t r1, uintptr_t r2, int vmode, bool gate_elem, int wfn,
                               uintptr_t hbias, uintptr_t st) {
    if (bs < 1 || bt_width < 1 || (gate && ld_gate < (gate_elem ? (int64_t)H * dv : H)))
      throw std::invalid_argument("masked_attention: inconsistent sizes");
    int rc = xgm::masked_attention(P<const void>(q), f32, P<const void>(kc), P<const void>(vc), P<const int32_t>(bt),
                                   bt_width, bs, P<const int32_t>(pos), P<const int32_t>(token_seq), P<const float>(temp),
                                   P<const float>(sink), P<void>(out), T, H, G, dk, dv, mask, size, scale,
                                   P<const void>(gate), ld_gate, P<const float>(r1), P<const float>(r2), vmode, gate_elem,
                                   wfn, P<const float>(hbias), S(st));
    check(rc, "masked_attention");
  });
  m.def("masked_attention_mfma", [](uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t bt, int bt_width, int bs,
                                    uintptr_t qsl, uintptr_t sl, uintptr_t slots, uintptr_t temp, uintptr_t sink,
                                    uintptr_t out, int T, int ns, int max_q, int H, int G, int dk, int dv, int mask,
                                    int size, float scale, int nsplit, uintptr_t part_o, uintptr_t part_ml,
                                    uintptr_t gate, int64_t ld_gate, uintptr_t r1, uintptr_t r2, int vmode, int nw_hint,
                                    bool gate_elem, int wfn, uintptr_t hbias, uintptr_t st) {
    if (bs < 1 || bt_width < 1 || nsplit < 1 || (gate && ld_gate < (gate_elem ? (int64_t)H * dv : H)))
      throw std::invalid_argument("masked_attention_mfma: inconsistent sizes");
    int rc = xgm::masked_attention_mfma(P<const void>(q), P<const void>(kc), P<const void>(vc), P<const int32_t>(bt),
                                        bt_width, bs, P<const int32_t>(qsl), P<const int32_t>(sl), P<const int32_t>(slots),
                                        P<const float>(temp), P<const float>(sink), P<void>(out), T, ns, max_q, H, G, dk,
                                        dv, mask, size, scale, nsplit, P<float>(part_o), P<float>(part_ml),
                                        P<const void>(gate), ld_gate, P<const float>(r1), P<const float>(r2), vmode,
                                        nw_hint, gate_elem, wfn, P<const float>(hbias), S(st));
    check(rc, "masked_attention_mfma");
  });
  m.def("talk_mix", [](uintptr_t o_all, bool f32, uintptr_t talk, uintptr_t gate, int64_t ld_gate, uintptr_t out, int T,
                       int H, int G, int dv, uintptr_t st) {
    if (H < 1 || G < 1 || H % G || dv < 1 || (gate && ld_gate < H))
      throw std::invalid_argument("talk_mix: inconsistent sizes");
    xgm::talk_mix(P<const void>(o_all), f32, P<const float>(talk), P<const void>(gate), ld_gate, P<void>(out), T, H, G, dv,
                  S(st));
    check(0, "talk_mix");
  });
  m.def("head_norm_rope_cache", [](uintptr_t src, bool src_f32, int64_t ld, int H, int G, int dk, int dv, uintptr_t wq,
                                   uintptr_t wk, float eps, uintptr_t rot, int rot_rows, int rot_dims, uintptr_t pos,
                                   uintptr_t slot_mapping, uintptr_t q_out, uintptr_t kc, uintptr_t vc, bool out_f32, int T,
                                   bool whole, bool half, uintptr_t v_first, int64_t ld_vf, uintptr_t v_mix, uintptr_t st) {
    if (H < 1 || G < 1 || dk < 1 || dv < 1 || ld < (int64_t)(H + G) * dk + (int64_t)G * dv || rot_dims < 0 ||
        rot_dims > dk || (rot_dims & 1) || (rot && rot_dims > 0 && rot_rows < 1) ||
        (v_first && (!v_mix || ld_vf < (int64_t)G * dv)))
      throw std::invalid_argument("head_norm_rope_cache: inconsistent sizes");
    xgm::head_norm_rope_cache(P<const void>(src), src_f32, ld, H, G, dk, dv, P<const float>(wq), P<const float>(wk), eps,
                              P<const float>(rot), rot_rows, rot_dims, P<const int32_t>(pos),
                              P<const int32_t>(slot_mapping), P<void>(q_out), P<void>(kc), P<void>(vc), out_f32, T, whole, half,
                              P<const void>(v_first), ld_vf, P<const float>(v_mix), S(st));
    check(0, "head_norm_rope_cache");
  });
  m.def("conv_head_norm_rope_cache", [](uintptr_t proj, bool in_f32, int64_t ld, uintptr_t conv_w, int taps,
                                        uintptr_t state, uintptr_t qsl, uintptr_t sl, uintptr_t slots, uintptr_t token_seq,
                                        int ns, int max_q, int H, int G, int dk, int dv, uintptr_t wq, uintptr_t wk,
                                        float eps, uintptr_t rot, int rot_rows, int rot_dims, uintptr_t slot_mapping,
                                        uintptr_t q_out, uintptr_t kc, uintptr_t vc, bool out_f32, int T, uintptr_t st) {
    if (H < 1 || G < 1 || dk < 1 || dv < 1 || ld < (int64_t)(H + G) * dk + (int64_t)G * dv || rot_dims < 0 ||
        rot_dims > dk || (rot_dims & 1) || (rot && rot_dims > 0 && rot_rows < 1) || (taps > 1 && !state))
      throw std::invalid_argument("conv_head_norm_rope_cache: inconsistent sizes");
    int rc = xgm::conv_head_norm_rope_cache(
        P<const void>(proj), in_f32, ld, P<const float>(conv_w), taps, P<float>(state), P<const int32_t>(qsl),
        P<const int32_t>(sl), P<const int32_t>(slots), P<const int32_t>(token_seq), ns, max_q, H, G, dk, dv,
        P<const float>(wq), P<const float>(wk), eps, P<const float>(rot), rot_rows, rot_dims,
        P<const int32_t>(slot_mapping), P<void>(q_out), P<void>(kc), P<void>(vc), out_f32, T, S(st));
    check(rc, "conv_head_norm_rope_cache");
  });
  m.def("post_norm_residual", [](uintptr_t x, uintptr_t y, bool y_f32, int64_t ldy, uintptr_t y_bias, uintptr_t y2,
                                 int64_t ldy2, uintptr_t pw1, uintptr_t pw2, uintptr_t post_w, float mult, uintptr_t extra,
                                 uintptr_t next_w, float off, float eps, uintptr_t out, bool out_f32, int T, int W,
                                 uintptr_t st) {
    if ((y && ldy < W) || (y2 && ldy2 < W)) throw std::invalid_argument("post_norm_residual: row stride below the width");
    int rc = xgm::post_norm_residual(P<float>(x), P<const void>(y), y_f32, ldy, P<const float>(y_bias), P<const void>(y2),
                                     ldy2, P<const float>(pw1), P<const float>(pw2), P<const float>(post_w), mult,
                                     P<const float>(extra), P<const float>(next_w), off, eps, P<void>(out), out_f32, T, W,
                                     S(st));
    check(rc, "post_norm_residual");
  });
  m.def("relu2", [](uintptr_t in, bool f32, uintptr_t bias, uintptr_t out, int64_t n, int cols, uintptr_t st) {
    if (cols < 1 || n % cols) throw std::invalid_argument("relu2: the element count must be whole rows");
    xgm::relu2(P<const void>(in), f32, P<const float>(bias), P<void>(out), n, cols, S(st));
    check(0, "relu2");
  });
  m.def("lower_bound_gates", [](uintptr_t proj, bool f32, int64_t ld, int off_q, int off_f, int n, uintptr_t f_bias,
                                uintptr_t lower, uintptr_t q, uintptr_t f, int T, uintptr_t st) {
    if (n < 1 || off_q < 0 || off_f < 0 || ld < off_q + n || ld < off_f + n)
      throw std::invalid_argument("lower_bound_gates: columns outside the row");
    xgm::lower_bound_gates(P<const void>(proj), f32, ld, off_q, off_f, n, P<const float>(f_bias), P<const float>(lower),
                           P<float>(q), P<float>(f), T, S(st));
    check(0, "lower_bound_gates");
  });
  m.def("gated_linear_scan", [](uintptr_t q, uintptr_t f, uintptr_t k, uintptr_t raw, int64_t ld_raw, int off_q, int off_f,
                                uintptr_t f_bias, uintptr_t lower, uintptr_t v, bool v_f32, int64_t ld_v, uintptr_t state,
                                uintptr_t qsl, uintptr_t sl, uintptr_t slots, uintptr_t o, int ns, int H, int dk, int dv,
                                int cols_hint, uintptr_t scratch, int max_q, int T, uintptr_t st) {
    if (H < 1 || dv < 1 || dk < 1 || ld_v < (int64_t)H * dv ||
        (raw && (off_q < 0 || off_f < 0 || ld_raw < off_q + (int64_t)H * dk || ld_raw < off_f + (int64_t)H * dk)))
      throw std::invalid_argument("gated_linear_scan: inconsistent sizes");
    int rc = xgm::gated_linear_scan(P<const float>(q), P<const float>(f), P<const float>(k), P<const void>(raw), ld_raw,
                                    off_q, off_f, P<const float>(f_bias), P<const float>(lower), P<const void>(v), v_f32,
                                    ld_v, P<float>(state), P<const int32_t>(qsl), P<const int32_t>(sl),
                                    P<const int32_t>(slots), P<float>(o), ns, H, dk, dv, cols_hint, P<float>(scratch),
                                    max_q, T, S(st));
    check(rc, "gated_linear_scan");
  });
  m.def("gated_linear_scan_scratch_floats",
        [](int T, int ns, int H, int dk, int dv) { return xgm::gated_linear_scan_scratch_floats(T, ns, H, dk, dv); });
  m.def("ssm_scan", [](uintptr_t xbc, bool f32, int64_t ld_x, uintptr_t dt, int64_t ld_dt, uintptr_t dt_bias,
                       uintptr_t A_log, uintptr_t D, uintptr_t state, uintptr_t qsl, uintptr_t sl, uintptr_t slots,
                       uintptr_t y, int ns, int H, int G, int N, int Pd, uintptr_t st) {
    if (H < 1 || G < 1 || ld_x < (int64_t)H * Pd + 2 * (int64_t)G * N || ld_dt < H)
      throw std::invalid_argument("ssm_scan: inconsistent sizes");
    int rc = xgm::ssm_scan(P<const void>(xbc), f32, ld_x, P<const void>(dt), ld_dt, P<const float>(dt_bias),
                           P<const float>(A_log), P<const float>(D), P<float>(state), P<const int32_t>(qsl),
                           P<const int32_t>(sl), P<const int32_t>(slots), P<float>(y), ns, H, G, N, Pd, S(st));
    check(rc, "ssm_scan");
  });
  m.def("gated_group_norm", [](uintptr_t y, uintptr_t z, bool f32, int64_t ld_z, uintptr_t w, int wn, float eps,
                               uintptr_t out, int T, int inner, int ng, bool gate_after, uintptr_t st) {
    if (ng < 1 || inner % ng || wn < 1 || inner % wn)
      throw std::invalid_argument("gated_group_norm: the parts and the weight's period must divide the row");
    xgm::gated_group_norm(P<const float>(y), P<const void>(z), f32, ld_z, P<const float>(w), wn, eps, P<void>(out), T,
                          inner, ng, gate_after, S(st));
    check(0, "gated_group_norm");
  });
  m.def("glu_act", [](uintptr_t in, bool f32, int64_t ld, uintptr_t out, int T, int F, int kind, float limit, float alpha,
                      uintptr_t st) {
    if (kind < 0 || kind > 1 || ld < 2 * (int64_t)F) throw std::invalid_argument("glu_act: inconsistent arguments");
    xgm::glu_act(P<const void>(in), f32, ld, P<void>(out), T, F, kind, limit, alpha, S(st));
    check(0, "glu_act");
  });
  m.def("grouped_router", [](uintptr_t logits, uintptr_t corr, int T, int E, int count, int keep, int top, float scale,
                             uintptr_t ids, uintptr_t wts, uintptr_t x, uintptr_t rw, int W, uintptr_t st) {
    int rc = xgm::grouped_router(P<const float>(logits), P<const float>(corr), T, E, count, keep, top, scale,
                                 P<int32_t>(ids), P<float>(wts), P<const float>(x), P<const float>(rw), W, S(st));
    check(rc, "grouped_router");
  });
  m.def("moe_align", [](uintptr_t ids, int pairs, int E, int cap, int tm, uintptr_t rows, uintptr_t tile_expert,
                        uintptr_t dest, uintptr_t st) {
    int rc = xgm::moe_align(P<const int32_t>(ids), pairs, E, cap, tm, P<int32_t>(rows), P<int32_t>(tile_expert),
                            P<int32_t>(dest), S(st));
    check(rc, "moe_align");
  });
  m.def("grouped_gemm", [](uintptr_t A, bool f32, int64_t lda, uintptr_t Wt, uintptr_t rows, uintptr_t tile_expert, int cap,
                           int tm, int top, int Nout, int K, int mode, uintptr_t out, int kind, float limit, float alpha,
                           uintptr_t row_scale, bool mfma, uintptr_t st) {
    if (top < 1 || lda < K) throw std::invalid_argument("grouped_gemm: inconsistent sizes");
    int rc = xgm::grouped_gemm(P<const void>(A), f32, lda, P<const void>(Wt), P<const int32_t>(rows),
                               P<const int32_t>(tile_expert), cap, tm, top, Nout, K, mode, P<void>(out), kind, limit, alpha,
                               P<const float>(row_scale), mfma, S(st));
    check(rc, "grouped_gemm");
  });
  m.def("moe_combine", [](uintptr_t y, uintptr_t dest, uintptr_t wts, int T, int top, int W, uintptr_t out, uintptr_t st) {
    xgm::moe_combine(P<const float>(y), P<const int32_t>(dest), P<const float>(wts), T, top, W, P<float>(out), S(st));
    check(0, "moe_combine");
  });

  m.def("mingru_scan", [](uintptr_t proj, bool f32, int64_t ld, int off_z, int off_x, int off_g, int n, uintptr_t bz,
                          uintptr_t bx, uintptr_t state, uintptr_t qsl, uintptr_t sl, uintptr_t slots, uintptr_t out,
                          bool out_f32, int ns, int max_q, uintptr_t scratch, int T, uintptr_t st) {
    if (n < 1 || off_z < 0 || off_x < 0 || off_g < 0 || ld < off_z + n || ld < off_x + n || ld < off_g + n || !state)
      throw std::invalid_argument("mingru_scan: columns outside the row");
    int rc = xgm::mingru_scan(P<const void>(proj), f32, ld, off_z, off_x, off_g, n, P<const float>(bz), P<const float>(bx),
                              P<float>(state), P<const int32_t>(qsl), P<const int32_t>(sl), P<const int32_t>(slots),
                              P<void>(out), out_f32, ns, max_q, P<float>(scratch), T, S(st));
    check(rc, "mingru_scan");
  });
  m.def("mingru_scratch_floats", [](int T, int ns, int n) { return xgm::mingru_scratch_floats(T, ns, n); });
  m.def("decay_gates", [](uintptr_t proj, bool f32, int64_t ld, int off_q, int off_k, int n, float q_scale, uintptr_t z,
                          int64_t ld_z, uintptr_t zb, float inv_tau, uintptr_t q, uintptr_t f, uintptr_t k, int T,
                          uintptr_t st) {
    if (n < 1 || off_q < 0 || off_k < 0 || ld < off_q + n || ld < off_k + n || ld_z < n || !(inv_tau > 0.f))
      throw std::invalid_argument("decay_gates: inconsistent arguments");
    xgm::decay_gates(P<const void>(proj), f32, ld, off_q, off_k, n, q_scale, P<const void>(z), ld_z, P<const float>(zb),
                     inv_tau, P<float>(q), P<float>(f), P<float>(k), T, S(st));
    check(0, "decay_gates");
  });

  m.def("canon_conv", [](uintptr_t x, uintptr_t w, uintptr_t state, uintptr_t qsl, uintptr_t sl, uintptr_t slots,
                         uintptr_t out, bool out_f32, int ns, int max_q, int W, int taps, uintptr_t st) {
    if (taps < 1 || taps > 8) throw std::invalid_argument("canon_conv: taps must be in [1, 8]");
    xgm::canon_conv(P<const float>(x), P<const float>(w), P<float>(state), P<const int32_t>(qsl), P<const int32_t>(sl),
                    P<const int32_t>(slots), P<void>(out), out_f32, ns, max_q, W, taps, S(st));
    check(0, "canon_conv");
  });
  m.def("scaled_add_rmsnorm", [](uintptr_t x, uintptr_t y, bool y_f32, int64_t y_stride, uintptr_t bias, float alpha,
                                 uintptr_t w, float w_offset, float eps, uintptr_t x_out, uintptr_t out, bool out_f32,
                                 int T, int W, uintptr_t st) {
    xgm::scaled_add_rmsnorm(P<const float>(x), P<const void>(y), y_f32, y_stride, P<const float>(bias), alpha,
                            P<const float>(w), w_offset, eps, P<float>(x_out), P<void>(out), out_f32, T, W, S(st));
    check(0, "scaled_add_rmsnorm");
  });
  m.def("latent_prep", [](uintptr_t proj, bool f32, int64_t ld, int off_q, int Rq, int off_kv, int R, int rd, uintptr_t wq,
                          uintptr_t wkv, float eps, uintptr_t pos, uintptr_t slot_mapping, uintptr_t rot, int rot_dims,
                          uintptr_t cq, uintptr_t cache, int T, uintptr_t st) {
    if (rot_dims % 2 || rot_dims > rd) throw std::invalid_argument("latent_prep: rot_dims must be even and <= rd");
    xgm::latent_prep(P<const void>(proj), f32, ld, off_q, Rq, off_kv, R, rd, P<const float>(wq), P<const float>(wkv), eps,
                     P<const int32_t>(pos), P<const int32_t>(slot_mapping), P<const float>(rot), rot_dims, P<void>(cq),
                     P<void>(cache), T, S(st));
    check(0, "latent_prep");
  });
  m.def("latent_attention", [](uintptr_t qabs, uintptr_t q, bool f32, int64_t q_stride, int dq, int dn, uintptr_t gate,
                               int64_t gate_stride, uintptr_t cache, uintptr_t bt, int bt_width, int bs, uintptr_t pos,
                               uintptr_t token_seq, uintptr_t rot, int rot_dims, uintptr_t out, int T, int H, int R, int rd,
                               int window, float scale, uintptr_t st) {
    if (rot_dims % 2 || rot_dims > rd || dn + rd != dq || window < 1 || bs < 1)
      throw std::invalid_argument("latent_attention: inconsistent sizes");
    int rc = xgm::latent_attention(P<const void>(qabs), P<const void>(q), f32, q_stride, dq, dn, P<const void>(gate),
                                   gate_stride, P<const void>(cache), P<const int32_t>(bt), bt_width, bs,
                                   P<const int32_t>(pos), P<const int32_t>(token_seq), P<const float>(rot), rot_dims,
                                   P<void>(out), T, H, R, rd, window, scale, S(st));
    check(rc, "latent_attention");
  });
  m.def("latent_attention_mfma", [](uintptr_t qabs, uintptr_t q, int dq, int dn, uintptr_t gate, int64_t gate_stride,
                                    uintptr_t cache, uintptr_t bt, int bt_width, int bs, uintptr_t qsl, uintptr_t sl,
                                    uintptr_t slots, uintptr_t rot, int rot_dims, uintptr_t out, int T, int ns, int max_q,
                                    int H, int R, int rd, int window, float scale, int nsplit, uintptr_t part_o,
                                    uintptr_t part_ml, uintptr_t st) {
    if (rot_dims % 2 || rot_dims > rd || dn + rd != dq || window < 1 || bs < 1 || nsplit < 1)
      throw std::invalid_argument("latent_attention_mfma: inconsistent sizes");
    int rc = xgm::latent_attention_mfma(P<const void>(qabs), P<const void>(q), dq, dn, P<const void>(gate), gate_stride,
                                        P<const void>(cache), P<const int32_t>(bt), bt_width, bs, P<const int32_t>(qsl),
                                        P<const int32_t>(sl), P<const int32_t>(slots), P<const float>(rot), rot_dims,
                                        P<void>(out), T, ns, max_q, H, R, rd, window, scale, nsplit, P<float>(part_o),
                                        P<float>(part_ml), S(st));
    check(rc, "latent_attention_mfma");
  });
  m.def("delta_scan", [](uintptr_t proj, bool f32, int64_t ld, int off_r, int off_k, int off_v, int off_a, uintptr_t wl,
                         int64_t ld_wl, uintptr_t a_bias, uintptr_t w0, uintptr_t state, uintptr_t qsl, uintptr_t sl,
                         uintptr_t slots, uintptr_t o, int ns, int H, int D, uintptr_t prep, int T, uintptr_t st) {
    int rc = xgm::delta_scan(P<const void>(proj), f32, ld, off_r, off_k, off_v, off_a, P<const void>(wl), ld_wl,
                             P<const float>(a_bias), P<const float>(w0), P<float>(state), P<const int32_t>(qsl),
                             P<const int32_t>(sl), P<const int32_t>(slots), P<float>(o), ns, H, D, P<float>(prep), T,
                             S(st));
    check(rc, "delta_scan");
  });
  m.def("delta_out", [](uintptr_t o, uintptr_t nw, uintptr_t gate, bool f32, int64_t gate_stride, float eps, uintptr_t out,
                        int T, int H, int D, uintptr_t st) {
    xgm::delta_out(P<const float>(o), P<const float>(nw), P<const void>(gate), f32, gate_stride, eps, P<void>(out), T, H, D,
                   S(st));
    check(0, "delta_out");
  });
  m.def("xielu", [](uintptr_t in, bool f32, uintptr_t bias, float sp, float cn, uintptr_t out, int64_t n, int F,
                    uintptr_t st) {
    xgm::xielu(P<const void>(in), f32, P<const float>(bias), sp, cn, P<void>(out), n, F, S(st));
    check(0, "xielu");
  });
  m.def("tanh_cols", [](uintptr_t in, bool f32, int64_t ld, uintptr_t out, int T, int n, uintptr_t st) {
    xgm::tanh_cols(P<const void>(in), f32, ld, P<void>(out), T, n, S(st));
    check(0, "tanh_cols");
  });
  m.def("heads_to_rows", [](uintptr_t in, bool f32, uintptr_t out, int T, int H, int n, uintptr_t st) {
    xgm::heads_to_rows(P<const void>(in), f32, P<void>(out), T, H, n, S(st));
    check(0, "heads_to_rows");
  });
}
