// pybind11 entry points of the layer-listed models' kernels (_C_mixers).
// Raw device pointers (torch.Tensor.data_ptr()) and the HIP stream handle go
// in; launches neither allocate nor synchronise, so they can be captured into
// HIP graphs.  A launcher that rejects its arguments returns nonzero, raised
// here.
#include <hip/hip_runtime.h>
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

namespace py = pybind11;
using u = uintptr_t;

extern "C" {
int dxm_stream_step(float*, const void*, int64_t, const float*, const float*, const float*, const float*, float, void*,
                    int64_t, int, int, int, int, hipStream_t);
int dxm_embed_streams(float*, const void*, const int64_t*, int, int, int, int64_t, const void*, const int64_t*,
                      int64_t, float, int, hipStream_t);
int dxm_section_norm(void*, const void*, int64_t, const float*, int, int, float, int, hipStream_t);
int dxm_depth_mix(float*, float*, int64_t, int, const float*, const int64_t*, int, float, const float*, void*,
                  const void*, int64_t, const float*, int, int, hipStream_t);
int dxm_retention(float*, float*, int, const void*, int64_t, const void*, int64_t, const void*, int64_t, const float*,
                  float, const int64_t*, const int*, const int*, int, int, int, int, int, int, hipStream_t);
int dxm_latent_rope(void*, const void*, const void*, int64_t, int, int, const void*, int64_t, const float*, float,
                    const float*, int, float, const int64_t*, const int64_t*, void*, int, int, int, int, int,
                    hipStream_t);
int dxm_gather_rows(void*, const void*, const int64_t*, int, int, int64_t, int, hipStream_t);
int dxm_residual_step(float*, const void*, int64_t, const void*, int64_t, const void*, int64_t, const float*,
                      const void*, int64_t, const float*, float, int, const float*, const float*, void*, void*, int, int,
                      int, hipStream_t);
int dxm_act_mul(void*, const void*, int64_t, const void*, int64_t, int, int, int64_t, int, float, float, int,
                hipStream_t);
int dxm_delta_rule(float*, float*, int, float*, const void*, int64_t, const void*, int64_t, const void*, int64_t, const void*,
                   int64_t, const void*, int64_t, const float*, const float*, float, float, const int64_t*, const int*,
                   const int*, int, int, int, int, int, int, hipStream_t);
int dxm_conv_rope_cache(void*, const void*, int64_t, const float*, int, const void*, int, const int64_t*,
                        const int64_t*, const int*, const int*, const int*, int, int, int, int, int, int, const float*,
                        int, void*, void*, int, hipStream_t);
int dxm_conv_state_update(void*, int, const void*, int64_t, const int64_t*, const int*, const int*, int, int, int, int,
                          int, hipStream_t);
int dxm_head_norm_gate(void*, const float*, const float*, const void*, int64_t, int, int, int, float, int, int,
                       hipStream_t);
int dxm_headprep_cache(void*, int64_t, const int64_t*, const int64_t*, int, int, int, int, int, const float*,
                       const float*, float, float, double, void*, void*, int, int, int, const void*, int64_t, float,
                       int, hipStream_t);
int dxm_moe_route(int*, float*, const float*, const float*, int, int, int, int, int, int, int, hipStream_t);
int dxm_moe_plan(int*, int*, const int*, int, int, hipStream_t);
int dxm_grouped_gemm(void*, const void*, int64_t, const void*, const int*, const int*, int, int, int, int, int, int,
                     int, int, hipStream_t);
int dxm_moe_combine(void*, const void*, const float*, const void*, int64_t, int, int, int, int, hipStream_t);
int dxm_diff_combine(void*, const float*, int64_t, int, float, float, float, const void*, int64_t, int, int,
                     hipStream_t);
int dxm_row_attention(void*, float*, const void*, int64_t, const void*, const void*, const int64_t*, const int*,
                      const int*, int, int, int, int, int, int, int, int, int, int, float, int, int, float, const float*,
                      const float*, int, const float*, const void*, int64_t, int, const float*, int, int, int,
                      hipStream_t);
int dxm_tile_attention_ok(int, int);
int dxm_tile_attention(void*, const void*, int64_t, const void*, const void*, const int64_t*, const int*, const int*,
                       int, int, const int*, int, int, int, int, int, int, int, int, float, int, int, float, const float*,
                       const float*, int, const float*, const void*, int64_t, int, const float*, int, hipStream_t);
int dxm_group_decode(float*, const void*, int64_t, const void*, const void*, const int64_t*, const int*, const int*, int,
                     int, int, int, int, int, int, int, int, int, float, int, int, float, const float*, const float*, int,
                     const float*, int, int, hipStream_t);
int dxm_merge_parts(void*, const float*, int64_t, int, int, int, const void*, int64_t, int, int, const float*, int,
                    hipStream_t);
}

static void check(int rc, const char* what) {
  if (rc != 0) throw std::runtime_error(std::string(what) + " rejected its arguments (code " + std::to_string(rc) + ")");
}

#define P(x) reinterpret_cast<void*>(x)
#define F(x) reinterpret_cast<float*>(x)
#define S(x) reinterpret_cast<hipStream_t>(x)

PYBIND11_MODULE(_C_mixers, m) {
  m.doc() = "dynamo_exp_amd gfx950 kernels of layer-listed models";
  m.attr("arch") = "gfx950";
  m.def("stream_step", [](u X, u y, int64_t ys, u mix, u gain, u rin, u nw, float eps, u out, int64_t os, int rows,
                          int S_, int W, int f32, u st) {
    check(dxm_stream_step(F(X), P(y), ys, F(mix), F(gain), F(rin), F(nw), eps, P(out), os, rows, S_, W, f32, S(st)),
          "stream_step");
  });
  m.def("embed_streams", [](u X, u table, u ids, int rows, int S_, int W, int64_t vocab, u ptab, u pos, int64_t n_pos,
                            float scale, int f32, u st) {
    check(dxm_embed_streams(F(X), P(table), reinterpret_cast<const int64_t*>(ids), rows, S_, W, vocab, P(ptab),
                            reinterpret_cast<const int64_t*>(pos), n_pos, scale, f32, S(st)),
          "embed_streams");
  });
  m.def("section_norm", [](u out, u x, int64_t xs, u w, int rows, int n, float eps, int f32, u st) {
    check(dxm_section_norm(P(out), P(x), xs, F(w), rows, n, eps, f32, S(st)), "section_norm");
  });
  m.def("depth_mix", [](u dst, u stack, int64_t plane, int n, u w, u rows, int n_rows, float eps, u nw, u out, u c,
                        int64_t cs, u cw, int W, int f32, u st) {
    check(dxm_depth_mix(F(dst), F(stack), plane, n, F(w), reinterpret_cast<const int64_t*>(rows), n_rows, eps, F(nw),
                        P(out), P(c), cs, F(cw), W, f32, S(st)),
          "depth_mix");
  });
  m.def("retention", [](u out, u state, int n_slots, u q, int64_t qs, u k, int64_t ks, u v, int64_t vs, u decay,
                        float k_scale, u pos, u seq_rows, u slots, int n_seq, int T, int H, int dk, int dv, int f32,
                        u st) {
    check(dxm_retention(F(out), F(state), n_slots, P(q), qs, P(k), ks, P(v), vs, F(decay), k_scale,
                        reinterpret_cast<const int64_t*>(pos), reinterpret_cast<const int*>(seq_rows),
                        reinterpret_cast<const int*>(slots), n_seq, T, H, dk, dv, f32, S(st)),
          "retention");
  });
  m.def("latent_rope", [](u q_out, u qa, u q, int64_t qs, int q_head, int q_off, u kv, int64_t kvs, u cn, float eps,
                          u inv_freq, int half, float mag, u pos, u slots, u cache, int T, int H, int r, int dr,
                          int f32, u st) {
    check(dxm_latent_rope(P(q_out), P(qa), P(q), qs, q_head, q_off, P(kv), kvs, F(cn), eps, F(inv_freq), half, mag,
                          reinterpret_cast<const int64_t*>(pos), reinterpret_cast<const int64_t*>(slots), P(cache), T,
                          H, r, dr, f32, S(st)),
          "latent_rope");
  });
  m.def("gather_rows", [](u out, u table, u ids, int rows, int W, int64_t vocab, int f32, u st) {
    check(dxm_gather_rows(P(out), P(table), reinterpret_cast<const int64_t*>(ids), rows, W, vocab, f32, S(st)),
          "gather_rows");
  });
  m.def("residual_step", [](u X, u a, int64_t as, u b, int64_t bs, u c, int64_t cs, u cw, u cg, int64_t cgs, u cgb,
                            float eps, int norm, u nw, u nb, u out, u xc, int rows, int W, int f32, u st) {
    check(dxm_residual_step(F(X), P(a), as, P(b), bs, P(c), cs, F(cw), P(cg), cgs, F(cgb), eps, norm, F(nw), F(nb),
                            P(out), P(xc), rows, W, f32, S(st)),
          "residual_step");
  });
  m.def("act_mul", [](u out, u gate, int64_t gs, u up, int64_t us, int rows, int Fw, int64_t os, int act, float limit,
                      float alpha, int f32, u st) {
    check(dxm_act_mul(P(out), P(gate), gs, P(up), us, rows, Fw, os, act, limit, alpha, f32, S(st)), "act_mul");
  });
  m.def("moe_route", [](u idx, u w, u z, u corr, int T, int E, int top, int n_groups, int keep, int score,
                        int group_max, u st) {
    check(dxm_moe_route(reinterpret_cast<int*>(idx), F(w), F(z), F(corr), T, E, top, n_groups, keep, score, group_max,
                        S(st)),
          "moe_route");
  });
  m.def("delta_rule", [](u out, u state, int n_slots, u prep, u r, int64_t rs, u k, int64_t ks, u v, int64_t vs, u a,
                         int64_t as, u w, int64_t ws, u ab, u wb, float decay_scale, float key_eps, u pos, u seq_rows,
                         u slots, int n_seq, int T, int H, int dk, int dv, int f32, u st) {
    check(dxm_delta_rule(F(out), F(state), n_slots, F(prep), P(r), rs, P(k), ks, P(v), vs, P(a), as, P(w), ws, F(ab), F(wb),
                         decay_scale, key_eps, reinterpret_cast<const int64_t*>(pos),
                         reinterpret_cast<const int*>(seq_rows), reinterpret_cast<const int*>(slots), n_seq, T, H, dk,
                         dv, f32, S(st)),
          "delta_rule");
  });
  m.def("conv_rope_cache", [](u q, u x, int64_t xs, u cw, int taps, u tail, int n_slots, u pos, u kv_slots, u row_seq,
                              u seq_rows, u slots, int n_seq, int T, int n_q, int n_k, int d, int dv, u inv_freq,
                              int half, u kc, u vc, int f32, u st) {
    check(dxm_conv_rope_cache(P(q), P(x), xs, F(cw), taps, P(tail), n_slots, reinterpret_cast<const int64_t*>(pos),
                              reinterpret_cast<const int64_t*>(kv_slots), reinterpret_cast<const int*>(row_seq),
                              reinterpret_cast<const int*>(seq_rows), reinterpret_cast<const int*>(slots), n_seq, T,
                              n_q, n_k, d, dv, F(inv_freq), half, P(kc), P(vc), f32, S(st)),
          "conv_rope_cache");
  });
  m.def("conv_state_update", [](u tail, int n_slots, u x, int64_t xs, u pos, u seq_rows, u slots, int n_seq, int T,
                                int C, int taps, int f32, u st) {
    check(dxm_conv_state_update(P(tail), n_slots, P(x), xs, reinterpret_cast<const int64_t*>(pos),
                                reinterpret_cast<const int*>(seq_rows), reinterpret_cast<const int*>(slots), n_seq, T,
                                C, taps, f32, S(st)),
          "conv_state_update");
  });
  m.def("head_norm_gate", [](u out, u o, u w, u gate, int64_t gs, int rows, int H, int dv, float eps, int gate_act,
                             int f32, u st) {
    check(dxm_head_norm_gate(P(out), F(o), F(w), P(gate), gs, rows, H, dv, eps, gate_act, f32, S(st)),
          "head_norm_gate");
  });
  m.def("moe_plan", [](u order, u offsets, u idx, int R, int E, u st) {
    check(dxm_moe_plan(reinterpret_cast<int*>(order), reinterpret_cast<int*>(offsets),
                       reinterpret_cast<const int*>(idx), R, E, S(st)),
          "moe_plan");
  });
  m.def("grouped_gemm", [](u out, u a, int64_t as, u w, u order, u offsets, int R, int E, int N, int K, int top,
                           int gather, int scatter, int f32, u st) {
    check(dxm_grouped_gemm(P(out), P(a), as, P(w), reinterpret_cast<const int*>(order),
                           reinterpret_cast<const int*>(offsets), R, E, N, K, top, gather, scatter, f32, S(st)),
          "grouped_gemm");
  });
  m.def("moe_combine", [](u out, u y, u w, u shared, int64_t ss, int T, int top, int W, int f32, u st) {
    check(dxm_moe_combine(P(out), P(y), F(w), P(shared), ss, T, top, W, f32, S(st)), "moe_combine");
  });
  m.def("headprep_cache", [](u x, int64_t xs, u pos, u slots, int rows, int n_q, int n_k, int d, int k_off, u qw, u kw,
                             float eps, float coef, double every, u kc, u vc, int v_mode, int v_off, int v_w, u vf,
                             int64_t vfs, float lam, int f32, u st) {
    check(dxm_headprep_cache(P(x), xs, reinterpret_cast<const int64_t*>(pos), reinterpret_cast<const int64_t*>(slots),
                             rows, n_q, n_k, d, k_off, F(qw), F(kw), eps, coef, every, P(kc), P(vc), v_mode, v_off,
                             v_w, P(vf), vfs, lam, f32, S(st)),
          "headprep_cache");
  });
  m.def("diff_combine", [](u out, u a, int64_t n_vec, int dv, float lam, float post, float eps, u gate, int64_t gs,
                           int H, int f32, u st) {
    check(dxm_diff_combine(P(out), F(a), n_vec, dv, lam, post, eps, P(gate), gs, H, f32, S(st)), "diff_combine");
  });
  m.def("tile_attention_ok", &dxm_tile_attention_ok);
  m.def("tile_attention", [](u out, u q, int64_t qs, u kc, u vc, u pos, u seq, u bt, int bts, int bs, u tiles,
                             int n_tiles, int n_qh, int maps, int group, int d, int dv, int Wk, int Wv, float scale,
                             int mask, int size, float cap, u r1, u r2, int wfn, u hbias, u gate, int64_t gs,
                             int keep, u sink, int out_f32, u st) {
    check(dxm_tile_attention(P(out), P(q), qs, P(kc), P(vc), reinterpret_cast<const int64_t*>(pos),
                             reinterpret_cast<const int*>(seq), reinterpret_cast<const int*>(bt), bts, bs,
                             reinterpret_cast<const int*>(tiles), n_tiles, n_qh, maps, group, d, dv, Wk, Wv, scale,
                             mask, size, cap, F(r1), F(r2), wfn, F(hbias), P(gate), gs, keep, F(sink), out_f32, S(st)),
          "tile_attention");
  });
  m.def("group_decode", [](u out, u ws, u q, int64_t qs, u kc, u vc, u pos, u seq, u bt, int bts, int bs, int rows,
                           int n_qh, int maps, int group, int d, int dv, int Wk, int Wv, float scale, int mask,
                           int size, float cap, u r1, u r2, int wfn, u hbias, u gate, int64_t gs, int keep, u sink,
                           int parts, int out_f32, u st) {
    check(dxm_group_decode(F(ws), P(q), qs, P(kc), P(vc), reinterpret_cast<const int64_t*>(pos),
                           reinterpret_cast<const int*>(seq), reinterpret_cast<const int*>(bt), bts, bs, rows, n_qh,
                           maps, group, d, dv, Wk, Wv, scale, mask, size, cap, F(r1), F(r2), wfn, F(hbias), keep,
                           parts, S(st)),
          "group_decode");
    check(dxm_merge_parts(P(out), F(ws), (int64_t)rows * n_qh, parts, dv, wfn, P(gate), gs, n_qh, maps, F(sink),
                          out_f32, S(st)),
          "merge_parts");
  });
  m.def("row_attention", [](u out, u ws, u q, int64_t qs, u kc, u vc, u pos, u seq, u bt, int bts, int bs, int rows,
                            int n_qh, int maps, int group, int d, int dv, int Wk, int Wv, float scale, int mask,
                            int size, float cap, u r1, u r2, int wfn, u hbias, u gate, int64_t gs, int keep, u sink,
                            int parts, int f32, int out_f32, u st) {
    check(dxm_row_attention(P(out), F(ws), P(q), qs, P(kc), P(vc), reinterpret_cast<const int64_t*>(pos),
                            reinterpret_cast<const int*>(seq), reinterpret_cast<const int*>(bt), bts, bs, rows, n_qh,
                            maps, group, d, dv, Wk, Wv, scale, mask, size, cap, F(r1), F(r2), wfn, F(hbias), P(gate), gs,
                            keep, F(sink), parts, f32, out_f32, S(st)),
          "row_attention");
  });
}
