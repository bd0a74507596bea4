// Python bindings for the gfx950 kernels (module llmss_amd._C).
//
// Pointers and the HIP stream are passed as integers: the Python layer (llmss_amd/ops/hip.py)
// owns tensor validation (dtype, contiguity, shapes vs. the grid each kernel assumes) so that a
// malformed call raises in Python instead of faulting the GPU. No torch headers are needed, which
// keeps the build a plain hipcc compile (no hipify step, no CUDA-compat layer).
#include <hip/hip_runtime.h>
#include <pybind11/pybind11.h>
#include <stdint.h>

namespace py = pybind11;

void launch_add_norm(const void* x, int64_t x_stride, const void* res_in, void* res_out, const void* w, const void* b,
                     void* y, int64_t y_stride, int T, int H, float eps, bool rms, hipStream_t st, void* q8,
                     void* s8, int xcw);
void launch_embed(const void* ids, const void* pos, const void* wte, const void* wpe, void* out, int T, int H,
                  int vocab, hipStream_t st);
void launch_rope_cache(void* qkv, int64_t row_stride, const void* pos, const void* cos_t, const void* sin_t, void* kc,
                       void* vc, const void* slot, int T, int nh, int nkv, int D, int rot, int block_size, int k_off,
                       int v_off, int style, bool do_rope, const void* part, int S, int64_t slab, const void* bias,
                       hipStream_t st, bool kv8);
void launch_attn_decode(const void* q, int64_t q_stride, const void* kc, const void* vc, const void* block_tables,
                        int bt_stride, const void* ctx_lens, void* out, int64_t out_stride, void* part_o,
                        void* part_ml, int B, int nh, int nkv, int D, int block_size, int nsplit, int part_size,
                        float scale, hipStream_t st, bool kv8);
void launch_attn_prefill(const void* qkv, int64_t row_stride, int T, const void* cu_seqlens, void* out,
                         int64_t out_stride, int B, int max_seqlen, int nh, int nkv, int D, int k_off, int v_off,
                         float scale, hipStream_t st);
void attn_prefill_set_version(int v);
void attn_prefill_set_waves(int nw);
void gemm_big_set_group(int g);
void launch_cand_topk(const void* logits, int64_t ld, int B, int vl, int lo, int V, const void* temperature,
                      const void* top_k, int K, int KC, void* pack, int64_t ldp, hipStream_t st, int shards);
void launch_sample_cand(const void* pack, int64_t ldp, int B, int groups, int KC, const void* temperature,
                        const void* top_k, const void* top_p, const void* seeds, void* out, void* out2, hipStream_t st);
void launch_ce_loss(const void* logits, int64_t ld, bool fp32, const void* labels, int T, int V, void* loss,
                    hipStream_t st);
void launch_attn_extend(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                        const void* block_tables, int max_blocks, const void* cu_q, const void* ctx_lens, void* out,
                        int64_t out_stride, int B, int max_qlen, int nh, int nkv, int D, int bs, float scale,
                        hipStream_t st, bool kv8, void* q8, void* s8, int window, int nsplit, int split_keys,
                        void* part_o, void* part_ml);
int launch_gemm_qkv_args(const void* x, int64_t ldx, const void* w, int64_t ldw, const void* bias, void* y, int64_t ldy,
                         int M, int N, int K, void* workspace, int64_t ws_bytes, int nt_hint, int split_hint,
                         const void* pos, const void* cos_t, const void* sin_t, void* kc, void* vc, const void* slot,
                         int nh, int nkv, int D, int rot, int block_size, int style, bool do_rope, hipStream_t st);
int launch_gemm(const void* x, int64_t ldx, const void* w, int64_t ldw, bool w_fp8, const void* w_scale,
                const void* bias, void* y, int64_t ldy, int M, int N, int K, int act, bool glu, void* workspace,
                int64_t ws_bytes, int nt_hint, int split_hint, bool partial_out, hipStream_t st);
void gemm_plan(int M, int N, int K, bool w_fp8, int* nt, int* splitk);
void gemm_tuned_set(int M, int N, int K, bool glu, int kind, int nt_hint, int split);
void gemm_tuned_clear();
void gemm_reserve_streamk(int n);
void gemm_set_slot(int s);
int launch_gemm_f8f8(const void* xq, int64_t ldx, const void* xs, const void* wq, int64_t ldw, const void* wsc,
                     const void* bias, void* y, int64_t ldy, int M, int N, int K, int act, bool glu, int tile,
                     int depth, int split, void* workspace, int64_t ws_bytes, hipStream_t st, bool partial_out,
                     bool ilv, void* mxq, void* mxs, const void* asc);
int gemm_f8f8_partial_slabs(int M, int N, int K, bool glu, int act, int tile, int split, int64_t ws_bytes);
int gemm_partial_slabs(int M, int N, int K, bool w_fp8, bool glu, int act, int nt_hint, int split_hint,
                       int64_t ws_bytes);
void attn_decode_set_unroll(int u);
void launch_comm_model(void* buf, int channels, int64_t nbytes, double us, hipStream_t st);
int64_t comm_model_slice(int channels, int64_t nbytes);

bool gemm_tuned_get(int M, int N, int K, bool glu, int kind, int* nt_hint, int* split);
void launch_add_norm_partial(const void* part, int S, int64_t slab, const void* xbias, const void* res_in,
                             void* res_out, const void* w, const void* b, void* y, int64_t y_stride, int T, int H,
                             float eps, bool rms, hipStream_t st, void* q8, void* s8);
void launch_sample(const void* logits, int64_t ld, bool fp32_logits, int B, int V, const void* temperature,
                   const void* top_k, const void* top_p, const void* seeds, void* out, void* out2, hipStream_t st);
void launch_quant_fp8_rows(const void* w, void* q, void* scale, int64_t N, int64_t K, hipStream_t st);
void launch_quant_fp8_rows_ld(const void* x, int64_t ldx, void* q, void* scale, int64_t M, int64_t K, hipStream_t st);
void launch_dequant_fp8_rows(const void* q, const void* scale, void* w, int64_t N, int64_t K, hipStream_t st);

// fp32 residual stream, strided / grouped GEMMs in either storage type, latent attention, mixture of experts
void launch_embed_scaled(const void* ids, const void* table, void* x, int T_, int H, int vocab, float scale, int dt,
                         hipStream_t st);
void launch_resid_add_norm(void* x, const void* a, int64_t lda, const void* b, int64_t ldb, const void* ey,
                           const void* place, const void* wts, int top, const void* shared_, int64_t lds_,
                           const void* w, float woff, float eps, void* y, int64_t ldy, int T_, int H, int dt,
                           hipStream_t st);
void launch_gemm_any(const void* A, const void* B, void* C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                     int64_t sBb, int64_t sBn, int64_t sBk, int64_t sCb, int64_t sCm, int da, int db, int dc,
                     hipStream_t st);
void launch_gemm_tile(const void* A, const void* B, void* C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                      int64_t sBb, int64_t sBn, int64_t sCb, int64_t sCm, int dc, hipStream_t st);
void launch_moe_gate_up_tile(const void* h, int64_t ldh, const void* wg, const void* wu, const void* meta,
                             const void* order, void* act, int E, int maxt, int top, int F, int K, float limit,
                             float alpha, int tile_rows, const void* pw, int silu, hipStream_t st);
void launch_moe_down_tile(const void* act, const void* wd, const void* meta, void* y, int E, int maxt, int N, int F,
                          int tile_rows, hipStream_t st);
void launch_latent_norm_cache(const void* src, int64_t ld, int off, const void* w, float eps, void* cache,
                              const void* slots, int T_, int R, int rot, int rdims, const void* cs, void* qa,
                              int off_q, int H, int qdim, int dt, int dq, hipStream_t st);
void launch_rope_angles(const void* positions, const void* freqs, void* cs, int T_, int half, hipStream_t st);
void launch_latent_attn(const void* qa, int64_t ldq, const void* cache, const void* bt, int maxb, const void* cu_q,
                        const void* ctx_lens, void* out, int64_t ldo, int T_, int B, int H, int R, int bs, int window,
                        float scale, int dt, hipStream_t st);
void launch_moe_route(const void* z, const void* corr, void* idx, void* wts, int T_, int E, int top, int norm,
                      hipStream_t st);
void launch_moe_router(const void* h, int64_t ldh, const void* wr, const void* corr, void* idx, void* wts, int T_,
                       int E, int K, int top, int dt, int norm, hipStream_t st);
void launch_moe_group(const void* idx, int P, int E, int maxt, void* meta, void* order, void* place, int tile_rows,
                      hipStream_t st);
void launch_moe_gate_up(const void* h, int64_t ldh, const void* wg, const void* wu, const void* meta,
                        const void* order, void* act, int E, int maxt, int top, int F, int K, float limit,
                        float alpha, int dt, const void* pw, int silu, hipStream_t st);
void launch_moe_down(const void* act, const void* wd, const void* meta, void* y, int E, int maxt, int N, int F,
                     int dt, hipStream_t st);
void launch_moe_combine(const void* y, const void* place, const void* wts, const void* shared_, int64_t lds_,
                        void* out, int T_, int N, int top, int dt, hipStream_t st);
void launch_glu_clamp(const void* gu, int64_t ldg, void* out, int64_t ldo, int T_, int F, float limit, float alpha,
                      int dt, hipStream_t st);

// residual streams, causal convolutions with a per-sequence tail, matrix-state recurrences, sink attention
void launch_embed_streams(const void* ids, const void* positions, const void* table, const void* ptab, void* x, int S,
                          int T_, int W, int vocab, int npos, int dt, hipStream_t st);
void launch_stream_add_norm(void* x, const void* y, int64_t ldy, const void* mix, const void* outw, float c,
                            const void* inw, const void* w, float eps, int rms, void* h, int64_t ldh, int S, int T_,
                            int W, int dt, int h_f32, hipStream_t st);
void launch_causal_conv(const void* in, int64_t ldi, const void* w, void* state, const void* cu, const void* ctx,
                        const void* sslots, void* out, int64_t ldo, int T_, int B, int C, int taps, int res, int silu,
                        int di, int dw, int dout, const void* bias, hipStream_t st);
void launch_gated_group_norm(const void* o, int64_t ldo, const void* gate, int64_t ldg, const void* w, float eps,
                             int act, float c, void* out, int64_t ldout, int T_, int groups, int n, int dt, int wfull,
                             int first, hipStream_t st);
void launch_glu_act(const void* gu, int64_t ldg, void* out, int64_t ldo, int T_, int F, int act, int dt,
                    hipStream_t st);
void launch_recurrence(int mode, const void* q, const void* k, const void* v, int64_t ldq, int64_t ldk, int64_t ldv,
                       const void* ab, int64_t ldab, int off_a, int off_b, const void* decay, const void* dt_bias,
                       void* state, const void* cu, const void* ctx, const void* sslots, void* out, int64_t ldo, int B,
                       int H, int G, int dim, int vdim, int silu_in, int gates_ready, int dq, int dp, const void* skip,
                       hipStream_t st);
// blocks normed on both sides, token input, windowed sigmoid attention with pooled blocks
void launch_sandwich_add_norm(void* x, const void* y, int64_t ldy, const void* ey, const void* place, const void* wts,
                              int top, const void* shared_, int64_t lds_, const void* r, int64_t ldr, const void* rb,
                              const void* wpost, const void* add, const void* wnext, void* h, int64_t ldh, float eps,
                              int T_, int W, int dt, hipStream_t st);
void launch_token_side_add(void* x, const void* ids, const void* table, int64_t ldt, int vocab, int col0, int d,
                           const void* wg, const void* wp, const void* wn, const void* add, const void* wnext, void* h,
                           int64_t ldh, float eps, int T_, int W, int dt, hipStream_t st);
void launch_rope_pairs_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* cs, int rdims,
                             void* qout, void* kc, void* vc, const void* slots, int T_, int H, int G, int dim, int vdim,
                             int dt, hipStream_t st);
void launch_pool_update(const void* kc, const void* vc, void* kp, void* vp, const void* bt, int maxb, const void* cu,
                        const void* ctx, int B, int max_qlen, int nk, int nv, int bs, int pool, int per, int dt,
                        hipStream_t st);
bool pool_attn_mfma_ok(int dim, int vdim);
void launch_pool_window_attn_mfma(const void* q, const void* kc, const void* vc, const void* kp, const void* vp,
                                  const void* bt, int maxb, const void* cu, const void* ctx, const void* pb, void* out,
                                  int out_f32, void* part, int nsplit, int64_t row0, int64_t rows, int B, int max_qlen,
                                  int H, int G, int dim, int vdim, int bs, float scale, int window, int pool, int per,
                                  hipStream_t st);
void launch_pool_window_attn(const void* q, const void* kc, const void* vc, const void* kp, const void* vp,
                             const void* bt, int maxb, const void* cu, const void* ctx, const void* pb, void* out,
                             int out_f32, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                             int window, int pool, int per, int dt, hipStream_t st);
void launch_silu_f32(const void* in, int64_t ldi, void* out, int64_t ldo, int T_, int n, int dt, hipStream_t st);
void launch_delta_gates(const void* a, const void* b, int64_t ld, const void* A_log, const void* dt_bias, void* gates,
                        int T_, int H, int dt, hipStream_t st);
void launch_rope_bias_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* bias,
                            const void* positions, const void* cs, int npos, int rot, void* qout, void* kc, void* vc,
                            const void* slots, int T_, int H, int G, int dim, int vdim, int dt, hipStream_t st);
void launch_sink_attn(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                      const void* ctx, void* out, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                      float cap, int all, int sink, int chunk, int vshare, int dt, hipStream_t st);
bool sink_attn_mfma_ok(int dim, int vdim);
void launch_sink_attn_mfma(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                           const void* ctx, void* out, int B, int max_qlen, int H, int G, int dim, int vdim, int bs,
                           float scale, float cap, int all, int sink, int chunk, int vshare, int precise,
                           hipStream_t st);
void launch_talk_mix(const void* O, const void* talk, float c, void* y, int64_t ldy, int T_, int H, int G, int vdim,
                     int dt, hipStream_t st);

// blocks normed on the sublayer's output, depth average, bigram embedding, ungated activations, differential attention
void launch_embed_bigram(const void* ids, const void* positions, const void* table, float scale, const void* bigram,
                         int64_t buckets, int64_t mul_prev, int64_t mul_cur, void* prev, const void* cu,
                         const void* ctx, const void* sslots, int B, void* h0, void* h1, int T_, int W, int vocab,
                         int dt, hipStream_t st);
void launch_resid_norm_add(void* hist, int64_t ldh, int n, const void* y, int64_t ldy, const void* w, float eps,
                           const void* dwa, int T_, int W, int dt, hipStream_t st);
void launch_gate_mul(void* y, int64_t ldy, const void* src, int64_t lds_, int T_, int N, int dt, hipStream_t st);
void launch_act_fn(const void* x, int64_t ldx, void* out, int64_t ldo, int T_, int F, int act, float a, float b,
                   int dt, hipStream_t st);
void launch_qk_norm_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* qw,
                          const void* kw, float eps, void* qout, void* kc, void* vc, const void* slots, int T_, int H,
                          int G, int maps, int dim, int vdim, int dt, hipStream_t st);
void launch_diff_combine(const void* O, float lam, float eps, float mult, void* y, int64_t ldy, int T_, int H, int G,
                         int vdim, int dt, hipStream_t st);

void register_runtime(py::module_& m);  // host-side C++ runtime (runtime.cpp)
void register_comm(py::module_& m);     // RCCL communicator (comm.cpp)
void register_ctrl(py::module_& m);     // shared-memory control ring (ctrl.cpp)

#define P(x) reinterpret_cast<void*>(static_cast<uintptr_t>(x))
#define CP(x) reinterpret_cast<const void*>(static_cast<uintptr_t>(x))
#define S(x) reinterpret_cast<hipStream_t>(static_cast<uintptr_t>(x))

PYBIND11_MODULE(_C, m) {
  m.doc() = "llmss_amd gfx950 HIP kernels + native runtime";
  m.def("add_norm", [](uintptr_t x, int64_t xs, uintptr_t ri, uintptr_t ro, uintptr_t w, uintptr_t b, uintptr_t y,
                       int64_t ys, int T, int H, float eps, bool rms, uintptr_t st, uintptr_t q8, uintptr_t s8, int xcw) {
    launch_add_norm(CP(x), xs, CP(ri), P(ro), CP(w), CP(b), P(y), ys, T, H, eps, rms, S(st), P(q8), P(s8), xcw);
  }, pybind11::arg("x"), pybind11::arg("xs"), pybind11::arg("ri"), pybind11::arg("ro"), pybind11::arg("w"),
     pybind11::arg("b"), pybind11::arg("y"), pybind11::arg("ys"), pybind11::arg("T"), pybind11::arg("H"),
     pybind11::arg("eps"), pybind11::arg("rms"), pybind11::arg("st"), pybind11::arg("q8") = 0,
     pybind11::arg("s8") = 0, pybind11::arg("xcw") = 0);
  m.def("embed", [](uintptr_t ids, uintptr_t pos, uintptr_t wte, uintptr_t wpe, uintptr_t out, int T, int H, int V,
                    uintptr_t st) { launch_embed(CP(ids), CP(pos), CP(wte), CP(wpe), P(out), T, H, V, S(st)); });
  m.def("rope_cache", [](uintptr_t qkv, int64_t rs, uintptr_t pos, uintptr_t cos_t, uintptr_t sin_t, uintptr_t kc,
                         uintptr_t vc, uintptr_t slot, int T, int nh, int nkv, int D, int rot, int bs, int k_off,
                         int v_off, int style, bool do_rope, uintptr_t part, int nslab, int64_t slab, uintptr_t bias,
                         uintptr_t st, bool kv8) {
    launch_rope_cache(P(qkv), rs, CP(pos), CP(cos_t), CP(sin_t), P(kc), P(vc), CP(slot), T, nh, nkv, D, rot, bs, k_off,
                      v_off, style, do_rope, CP(part), nslab, slab, CP(bias), S(st), kv8);
  });
  m.def("attn_decode", [](uintptr_t q, int64_t qs, uintptr_t kc, uintptr_t vc, uintptr_t bt, int bts, uintptr_t cl,
                          uintptr_t out, int64_t os, uintptr_t po, uintptr_t pml, int B, int nh, int nkv, int D, int bs,
                          int nsplit, int psize, float scale, uintptr_t st, bool kv8) {
    launch_attn_decode(CP(q), qs, CP(kc), CP(vc), CP(bt), bts, CP(cl), P(out), os, P(po), P(pml), B, nh, nkv, D, bs,
                       nsplit, psize, scale, S(st), kv8);
  });
  m.def("attn_prefill", [](uintptr_t qkv, int64_t rs, int T, uintptr_t cu, uintptr_t out, int64_t os, int B,
                           int maxlen, int nh, int nkv, int D, int k_off, int v_off, float scale, uintptr_t st) {
    launch_attn_prefill(CP(qkv), rs, T, CP(cu), P(out), os, B, maxlen, nh, nkv, D, k_off, v_off, scale, S(st));
  });
  m.def("attn_prefill_set_version", &attn_prefill_set_version);
  m.def("attn_prefill_set_waves", &attn_prefill_set_waves);
  m.def("gemm_big_set_group", &gemm_big_set_group);
  m.def("cand_topk", [](uintptr_t lg, int64_t ld, int B, int vl, int lo, int V, uintptr_t temp, uintptr_t topk, int K,
                        int KC, uintptr_t pack, int64_t ldp, uintptr_t st, int shards) {
    launch_cand_topk(CP(lg), ld, B, vl, lo, V, CP(temp), CP(topk), K, KC, P(pack), ldp, S(st), shards);
  }, pybind11::arg("lg"), pybind11::arg("ld"), pybind11::arg("B"), pybind11::arg("vl"), pybind11::arg("lo"),
     pybind11::arg("V"), pybind11::arg("temp"), pybind11::arg("topk"), pybind11::arg("K"), pybind11::arg("KC"),
     pybind11::arg("pack"), pybind11::arg("ldp"), pybind11::arg("st"), pybind11::arg("shards") = 1);
  m.def("sample_cand", [](uintptr_t pack, int64_t ldp, int B, int groups, int KC, uintptr_t temp, uintptr_t topk,
                          uintptr_t topp, uintptr_t seeds, uintptr_t out, uintptr_t out2, uintptr_t st) {
    launch_sample_cand(CP(pack), ldp, B, groups, KC, CP(temp), CP(topk), CP(topp), CP(seeds), P(out), P(out2), S(st));
  });
  m.def("ce_loss", [](uintptr_t lg, int64_t ld, bool fp32, uintptr_t lab, int T, int V, uintptr_t loss, uintptr_t st) {
    launch_ce_loss(CP(lg), ld, fp32, CP(lab), T, V, P(loss), S(st));
  });
  m.def("attn_extend", [](uintptr_t q, int64_t qs, uintptr_t kc, uintptr_t vc, uintptr_t bt, int maxb, uintptr_t cu,
                          uintptr_t cl, uintptr_t out, int64_t os, int B, int maxq, int nh, int nkv, int D, int bs,
                          float scale, uintptr_t st, bool kv8, uintptr_t q8, uintptr_t s8, int window, int nsplit,
                          int split_keys, uintptr_t po, uintptr_t pml) {
    launch_attn_extend(CP(q), qs, CP(kc), CP(vc), CP(bt), maxb, CP(cu), CP(cl), P(out), os, B, maxq, nh, nkv, D, bs,
                       scale, S(st), kv8, P(q8), P(s8), window, nsplit, split_keys, P(po), P(pml));
  }, pybind11::arg("q"), pybind11::arg("qs"), pybind11::arg("kc"), pybind11::arg("vc"), pybind11::arg("bt"),
     pybind11::arg("maxb"), pybind11::arg("cu"), pybind11::arg("cl"), pybind11::arg("out"), pybind11::arg("os"),
     pybind11::arg("B"), pybind11::arg("maxq"), pybind11::arg("nh"), pybind11::arg("nkv"), pybind11::arg("D"),
     pybind11::arg("bs"), pybind11::arg("scale"), pybind11::arg("st"), pybind11::arg("kv8"), pybind11::arg("q8") = 0,
     pybind11::arg("s8") = 0, pybind11::arg("window") = 0, pybind11::arg("nsplit") = 1,
     pybind11::arg("split_keys") = 0, pybind11::arg("po") = 0, pybind11::arg("pml") = 0);
  m.def("gemm", [](uintptr_t x, int64_t ldx, uintptr_t w, int64_t ldw, bool fp8, uintptr_t ws, uintptr_t bias,
                   uintptr_t y, int64_t ldy, int M, int N, int K, int act, bool glu, uintptr_t work, int64_t wbytes,
                   int nt_hint, int split_hint, bool partial_out, uintptr_t st) {
    return launch_gemm(CP(x), ldx, CP(w), ldw, fp8, CP(ws), CP(bias), P(y), ldy, M, N, K, act, glu, P(work), wbytes,
                       nt_hint, split_hint, partial_out, S(st));
  });
  m.def("gemm_qkv", [](uintptr_t x, int64_t ldx, uintptr_t w, int64_t ldw, uintptr_t bias, uintptr_t y, int64_t ldy,
                       int M, int N, int K, uintptr_t work, int64_t wbytes, int nt_hint, int split_hint, uintptr_t pos,
                       uintptr_t cos_t, uintptr_t sin_t, uintptr_t kc, uintptr_t vc, uintptr_t slot, int nh, int nkv,
                       int D, int rot, int bs, int style, bool do_rope, uintptr_t st) {
    return launch_gemm_qkv_args(CP(x), ldx, CP(w), ldw, CP(bias), P(y), ldy, M, N, K, P(work), wbytes, nt_hint,
                                split_hint, CP(pos), CP(cos_t), CP(sin_t), P(kc), P(vc), CP(slot), nh, nkv, D, rot, bs,
                                style, do_rope, S(st));
  }, pybind11::arg("x"), pybind11::arg("ldx"), pybind11::arg("w"), pybind11::arg("ldw"), pybind11::arg("bias"),
     pybind11::arg("y"), pybind11::arg("ldy"), pybind11::arg("M"), pybind11::arg("N"), pybind11::arg("K"),
     pybind11::arg("work"), pybind11::arg("wbytes"), pybind11::arg("nt_hint"), pybind11::arg("split_hint"),
     pybind11::arg("pos"), pybind11::arg("cos_t"), pybind11::arg("sin_t"), pybind11::arg("kc"), pybind11::arg("vc"),
     pybind11::arg("slot"), pybind11::arg("nh"), pybind11::arg("nkv"), pybind11::arg("D"), pybind11::arg("rot"),
     pybind11::arg("bs"), pybind11::arg("style"), pybind11::arg("do_rope"), pybind11::arg("st"));
  m.def("gemm_plan", [](int M, int N, int K, bool fp8) {
    int nt, s;
    gemm_plan(M, N, K, fp8, &nt, &s);
    return py::make_tuple(nt, s);
  });
  m.def("gemm_tuned_set", &gemm_tuned_set);
  m.def("gemm_tuned_clear", &gemm_tuned_clear);
  m.def("gemm_reserve_streamk", &gemm_reserve_streamk);
  m.def("gemm_set_slot", &gemm_set_slot);
  m.def("gemm_f8f8", [](uintptr_t xq, int64_t ldx, uintptr_t xs, uintptr_t wq, int64_t ldw, uintptr_t wsc,
                        uintptr_t bias, uintptr_t y, int64_t ldy, int M, int N, int K, int act, bool glu, int tile,
                        int depth, int split, uintptr_t work, int64_t wbytes, uintptr_t st, bool partial_out, bool ilv,
                        uintptr_t mxq, uintptr_t mxs, uintptr_t asc) {
    return launch_gemm_f8f8(CP(xq), ldx, CP(xs), CP(wq), ldw, CP(wsc), CP(bias), P(y), ldy, M, N, K, act, glu, tile,
                            depth, split, P(work), wbytes, S(st), partial_out, ilv, P(mxq), P(mxs), CP(asc));
  }, pybind11::arg("xq"), pybind11::arg("ldx"), pybind11::arg("xs"), pybind11::arg("wq"), pybind11::arg("ldw"),
     pybind11::arg("wsc"), pybind11::arg("bias"), pybind11::arg("y"), pybind11::arg("ldy"), pybind11::arg("M"),
     pybind11::arg("N"), pybind11::arg("K"), pybind11::arg("act"), pybind11::arg("glu"), pybind11::arg("tile"),
     pybind11::arg("depth"), pybind11::arg("split"), pybind11::arg("work"), pybind11::arg("wbytes"),
     pybind11::arg("st"), pybind11::arg("partial_out") = false, pybind11::arg("ilv") = false,
     pybind11::arg("mxq") = 0, pybind11::arg("mxs") = 0, pybind11::arg("asc") = 0);
  m.def("gemm_f8f8_partial_slabs", &gemm_f8f8_partial_slabs);
  m.def("gemm_partial_slabs", &gemm_partial_slabs);
  m.def("attn_decode_set_unroll", &attn_decode_set_unroll);
  m.def("comm_model", [](uintptr_t buf, int channels, int64_t nbytes, double us, uintptr_t st) {
    launch_comm_model(P(buf), channels, nbytes, us, S(st));
  });
  m.def("comm_model_slice", &comm_model_slice);
  m.def("gemm_tuned_get", [](int M, int N, int K, bool glu, int kind) -> py::object {
    int nt, s;
    if (!gemm_tuned_get(M, N, K, glu, kind, &nt, &s)) return py::none();
    return py::make_tuple(nt, s);
  });
  m.def("add_norm_partial", [](uintptr_t part, int S, int64_t slab, uintptr_t xbias, uintptr_t ri, uintptr_t ro,
                               uintptr_t w, uintptr_t b, uintptr_t y, int64_t ys, int T, int H, float eps, bool rms,
                               uintptr_t st, uintptr_t q8, uintptr_t s8) {
    launch_add_norm_partial(CP(part), S, slab, CP(xbias), CP(ri), P(ro), CP(w), CP(b), P(y), ys, T, H, eps, rms, S(st),
                            P(q8), P(s8));
  }, pybind11::arg("part"), pybind11::arg("S"), pybind11::arg("slab"), pybind11::arg("xbias"), pybind11::arg("ri"),
     pybind11::arg("ro"), pybind11::arg("w"), pybind11::arg("b"), pybind11::arg("y"), pybind11::arg("ys"),
     pybind11::arg("T"), pybind11::arg("H"), pybind11::arg("eps"), pybind11::arg("rms"), pybind11::arg("st"),
     pybind11::arg("q8") = 0, pybind11::arg("s8") = 0);
  m.def("sample", [](uintptr_t logits, int64_t ld, bool fp32, int B, int V, uintptr_t temp, uintptr_t topk,
                     uintptr_t topp, uintptr_t seeds, uintptr_t out, uintptr_t out2, uintptr_t st) {
    launch_sample(CP(logits), ld, fp32, B, V, CP(temp), CP(topk), CP(topp), CP(seeds), P(out), P(out2), S(st));
  });
  m.def("quant_fp8_rows", [](uintptr_t w, uintptr_t q, uintptr_t scale, int64_t N, int64_t K, uintptr_t st) {
    launch_quant_fp8_rows(CP(w), P(q), P(scale), N, K, S(st));
  });
  m.def("quant_fp8_rows_ld", [](uintptr_t x, int64_t ldx, uintptr_t q, uintptr_t scale, int64_t M, int64_t K,
                                uintptr_t st) { launch_quant_fp8_rows_ld(CP(x), ldx, P(q), P(scale), M, K, S(st)); });
  m.def("dequant_fp8_rows", [](uintptr_t q, uintptr_t scale, uintptr_t w, int64_t N, int64_t K, uintptr_t st) {
    launch_dequant_fp8_rows(CP(q), CP(scale), P(w), N, K, S(st));
  });
  m.def("embed_scaled", [](uintptr_t ids, uintptr_t table, uintptr_t x, int T, int H, int V, float scale, int dt,
                           uintptr_t st) { launch_embed_scaled(CP(ids), CP(table), P(x), T, H, V, scale, dt, S(st)); });
  m.def("resid_add_norm", [](uintptr_t x, uintptr_t a, int64_t lda, uintptr_t b, int64_t ldb, uintptr_t ey,
                             uintptr_t place, uintptr_t wts, int top, uintptr_t sh, int64_t lds_, uintptr_t w,
                             float woff, float eps, uintptr_t y, int64_t ldy, int T, int H, int dt, uintptr_t st) {
    launch_resid_add_norm(P(x), CP(a), lda, CP(b), ldb, CP(ey), CP(place), CP(wts), top, CP(sh), lds_, CP(w), woff,
                          eps, P(y), ldy, T, H, dt, S(st));
  });
  m.def("gemm_any", [](uintptr_t A, uintptr_t B, uintptr_t C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                       int64_t sBb, int64_t sBn, int64_t sBk, int64_t sCb, int64_t sCm, int da, int db, int dc,
                       uintptr_t st) {
    launch_gemm_any(CP(A), CP(B), P(C), M, N, K, batch, sAb, sAm, sBb, sBn, sBk, sCb, sCm, da, db, dc, S(st));
  });
  m.def("gemm_tile", [](uintptr_t A, uintptr_t B, uintptr_t C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                        int64_t sBb, int64_t sBn, int64_t sCb, int64_t sCm, int dc, uintptr_t st) {
    launch_gemm_tile(CP(A), CP(B), P(C), M, N, K, batch, sAb, sAm, sBb, sBn, sCb, sCm, dc, S(st));
  });
  m.def("moe_gate_up_tile", [](uintptr_t h, int64_t ldh, uintptr_t wg, uintptr_t wu, uintptr_t meta, uintptr_t order,
                               uintptr_t act, int E, int maxt, int top, int F, int K, float limit, float alpha,
                               int tile_rows, uintptr_t pw, int silu, uintptr_t st) {
    launch_moe_gate_up_tile(CP(h), ldh, CP(wg), CP(wu), CP(meta), CP(order), P(act), E, maxt, top, F, K, limit, alpha,
                            tile_rows, CP(pw), silu, S(st));
  });
  m.def("moe_down_tile", [](uintptr_t act, uintptr_t wd, uintptr_t meta, uintptr_t y, int E, int maxt, int N, int F,
                            int tile_rows, uintptr_t st) {
    launch_moe_down_tile(CP(act), CP(wd), CP(meta), P(y), E, maxt, N, F, tile_rows, S(st));
  });
  m.def("latent_norm_cache", [](uintptr_t src, int64_t ld, int off, uintptr_t w, float eps, uintptr_t cache,
                                uintptr_t slots, int T, int R, int rot, int rdims, uintptr_t cs, uintptr_t qa,
                                int off_q, int H, int qdim, int dt, int dq, uintptr_t st) {
    launch_latent_norm_cache(CP(src), ld, off, CP(w), eps, P(cache), CP(slots), T, R, rot, rdims, CP(cs), P(qa), off_q,
                             H, qdim, dt, dq, S(st));
  });
  m.def("rope_angles", [](uintptr_t pos, uintptr_t freqs, uintptr_t cs, int T, int half, uintptr_t st) {
    launch_rope_angles(CP(pos), CP(freqs), P(cs), T, half, S(st));
  });
  m.def("latent_attn", [](uintptr_t qa, int64_t ldq, uintptr_t cache, uintptr_t bt, int maxb, uintptr_t cu,
                          uintptr_t ctx, uintptr_t out, int64_t ldo, int T, int B, int H, int R, int bs, int window,
                          float scale, int dt, uintptr_t st) {
    launch_latent_attn(CP(qa), ldq, CP(cache), CP(bt), maxb, CP(cu), CP(ctx), P(out), ldo, T, B, H, R, bs, window,
                       scale, dt, S(st));
  });
  m.def("moe_route", [](uintptr_t z, uintptr_t corr, uintptr_t idx, uintptr_t wts, int T, int E, int top, int norm,
                        uintptr_t st) { launch_moe_route(CP(z), CP(corr), P(idx), P(wts), T, E, top, norm, S(st)); });
  m.def("moe_router", [](uintptr_t h, int64_t ldh, uintptr_t wr, uintptr_t corr, uintptr_t idx, uintptr_t wts, int T,
                         int E, int K, int top, int dt, int norm, uintptr_t st) {
    launch_moe_router(CP(h), ldh, CP(wr), CP(corr), P(idx), P(wts), T, E, K, top, dt, norm, S(st));
  });
  m.def("moe_group", [](uintptr_t idx, int Pn, int E, int maxt, uintptr_t meta, uintptr_t order, uintptr_t place,
                        int tile_rows, uintptr_t st) {
    launch_moe_group(CP(idx), Pn, E, maxt, P(meta), P(order), P(place), tile_rows, S(st));
  });
  m.def("moe_gate_up", [](uintptr_t h, int64_t ldh, uintptr_t wg, uintptr_t wu, uintptr_t meta, uintptr_t order,
                          uintptr_t act, int E, int maxt, int top, int F, int K, float limit, float alpha, int dt,
                          uintptr_t pw, int silu, uintptr_t st) {
    launch_moe_gate_up(CP(h), ldh, CP(wg), CP(wu), CP(meta), CP(order), P(act), E, maxt, top, F, K, limit, alpha, dt,
                       CP(pw), silu, S(st));
  });
  m.def("moe_down", [](uintptr_t act, uintptr_t wd, uintptr_t meta, uintptr_t y, int E, int maxt, int N, int F, int dt,
                       uintptr_t st) { launch_moe_down(CP(act), CP(wd), CP(meta), P(y), E, maxt, N, F, dt, S(st)); });
  m.def("moe_combine", [](uintptr_t y, uintptr_t place, uintptr_t wts, uintptr_t sh, int64_t lds_, uintptr_t out, int T,
                          int N, int top, int dt, uintptr_t st) {
    launch_moe_combine(CP(y), CP(place), CP(wts), CP(sh), lds_, P(out), T, N, top, dt, S(st));
  });
  m.def("glu_clamp", [](uintptr_t gu, int64_t ldg, uintptr_t out, int64_t ldo, int T, int F, float limit, float alpha,
                        int dt, uintptr_t st) { launch_glu_clamp(CP(gu), ldg, P(out), ldo, T, F, limit, alpha, dt, S(st)); });
  m.def("embed_streams", [](uintptr_t ids, uintptr_t pos, uintptr_t table, uintptr_t ptab, uintptr_t x, int Sn, int T,
                            int W, int V, int npos, int dt, uintptr_t st) {
    launch_embed_streams(CP(ids), CP(pos), CP(table), CP(ptab), P(x), Sn, T, W, V, npos, dt, S(st));
  });
  m.def("stream_add_norm", [](uintptr_t x, uintptr_t y, int64_t ldy, uintptr_t mix, uintptr_t outw, float c,
                              uintptr_t inw, uintptr_t w, float eps, int rms, uintptr_t h, int64_t ldh, int Sn, int T,
                              int W, int dt, int h_f32, uintptr_t st) {
    launch_stream_add_norm(P(x), CP(y), ldy, CP(mix), CP(outw), c, CP(inw), CP(w), eps, rms, P(h), ldh, Sn, T, W, dt,
                           h_f32, S(st));
  });
  m.def("causal_conv", [](uintptr_t in, int64_t ldi, uintptr_t w, uintptr_t state, uintptr_t cu, uintptr_t ctx,
                          uintptr_t ss, uintptr_t out, int64_t ldo, int T, int B, int C, int taps, int res, int silu,
                          int di, int dw, int dout, uintptr_t bias, uintptr_t st) {
    launch_causal_conv(CP(in), ldi, CP(w), P(state), CP(cu), CP(ctx), CP(ss), P(out), ldo, T, B, C, taps, res, silu,
                       di, dw, dout, CP(bias), S(st));
  });
  m.def("gated_group_norm", [](uintptr_t o, int64_t ldo, uintptr_t gate, int64_t ldg, uintptr_t w, float eps, int act,
                               float c, uintptr_t out, int64_t ldout, int T, int groups, int n, int dt, int wfull,
                               int first, uintptr_t st) {
    launch_gated_group_norm(CP(o), ldo, CP(gate), ldg, CP(w), eps, act, c, P(out), ldout, T, groups, n, dt, wfull,
                            first, S(st));
  });
  m.def("glu_act", [](uintptr_t gu, int64_t ldg, uintptr_t out, int64_t ldo, int T, int F, int act, int dt,
                      uintptr_t st) { launch_glu_act(CP(gu), ldg, P(out), ldo, T, F, act, dt, S(st)); });
  m.def("recurrence", [](int mode, uintptr_t q, uintptr_t k, uintptr_t v, int64_t ldq, int64_t ldk, int64_t ldv,
                         uintptr_t ab, int64_t ldab, int off_a, int off_b, uintptr_t decay, uintptr_t dtb,
                         uintptr_t state, uintptr_t cu, uintptr_t ctx, uintptr_t ss, uintptr_t out, int64_t ldo, int B,
                         int H, int G, int dim, int vdim, int silu_in, int gates_ready, int dq, int dp, uintptr_t skip,
                         uintptr_t st) {
    launch_recurrence(mode, CP(q), CP(k), CP(v), ldq, ldk, ldv, CP(ab), ldab, off_a, off_b, CP(decay), CP(dtb),
                      P(state), CP(cu), CP(ctx), CP(ss), P(out), ldo, B, H, G, dim, vdim, silu_in, gates_ready, dq, dp,
                      CP(skip), S(st));
  });
  m.def("silu_f32", [](uintptr_t in, int64_t ldi, uintptr_t out, int64_t ldo, int T, int n, int dt, uintptr_t st) {
    launch_silu_f32(CP(in), ldi, P(out), ldo, T, n, dt, S(st));
  });
  m.def("delta_gates", [](uintptr_t a, uintptr_t b, int64_t ld, uintptr_t A_log, uintptr_t dtb, uintptr_t gates, int T,
                          int H, int dt, uintptr_t st) {
    launch_delta_gates(CP(a), CP(b), ld, CP(A_log), CP(dtb), P(gates), T, H, dt, S(st));
  });
  m.def("rope_bias_cache", [](uintptr_t proj, int64_t ldp, int off_q, int off_k, int off_v, uintptr_t bias,
                              uintptr_t pos, uintptr_t cs, int npos, int rot, uintptr_t qout, uintptr_t kc,
                              uintptr_t vc, uintptr_t slots, int T, int H, int G, int dim, int vdim, int dt,
                              uintptr_t st) {
    launch_rope_bias_cache(CP(proj), ldp, off_q, off_k, off_v, CP(bias), CP(pos), CP(cs), npos, rot, P(qout), P(kc),
                           P(vc), CP(slots), T, H, G, dim, vdim, dt, S(st));
  });
  m.def("sink_attn", [](uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t bt, int maxb, uintptr_t cu, uintptr_t ctx,
                        uintptr_t out, int T, int B, int H, int G, int dim, int vdim, int bs, float scale, float cap,
                        int all, int sink, int chunk, int vshare, int dt, uintptr_t st) {
    launch_sink_attn(CP(q), CP(kc), CP(vc), CP(bt), maxb, CP(cu), CP(ctx), P(out), T, B, H, G, dim, vdim, bs, scale,
                     cap, all, sink, chunk, vshare, dt, S(st));
  });
  m.def("sink_attn_mfma_ok", &sink_attn_mfma_ok);
  m.def("sink_attn_mfma", [](uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t bt, int maxb, uintptr_t cu,
                             uintptr_t ctx, uintptr_t out, int B, int max_qlen, int H, int G, int dim, int vdim, int bs,
                             float scale, float cap, int all, int sink, int chunk, int vshare, int precise,
                             uintptr_t st) {
    launch_sink_attn_mfma(CP(q), CP(kc), CP(vc), CP(bt), maxb, CP(cu), CP(ctx), P(out), B, max_qlen, H, G, dim, vdim,
                          bs, scale, cap, all, sink, chunk, vshare, precise, S(st));
  });
  m.def("talk_mix", [](uintptr_t O, uintptr_t talk, float c, uintptr_t y, int64_t ldy, int T, int H, int G, int vdim,
                       int dt, uintptr_t st) { launch_talk_mix(CP(O), CP(talk), c, P(y), ldy, T, H, G, vdim, dt, S(st)); });
  m.def("embed_bigram", [](uintptr_t ids, uintptr_t pos, uintptr_t table, float scale, uintptr_t bigram,
                           int64_t buckets, int64_t mul_prev, int64_t mul_cur, uintptr_t prev, uintptr_t cu,
                           uintptr_t ctx, uintptr_t ss, int B, uintptr_t h0, uintptr_t h1, int T, int W, int V, int dt,
                           uintptr_t st) {
    launch_embed_bigram(CP(ids), CP(pos), CP(table), scale, CP(bigram), buckets, mul_prev, mul_cur, P(prev), CP(cu),
                        CP(ctx), CP(ss), B, P(h0), P(h1), T, W, V, dt, S(st));
  });
  m.def("resid_norm_add", [](uintptr_t hist, int64_t ldh, int n, uintptr_t y, int64_t ldy, uintptr_t w, float eps,
                             uintptr_t dwa, int T, int W, int dt, uintptr_t st) {
    launch_resid_norm_add(P(hist), ldh, n, CP(y), ldy, CP(w), eps, CP(dwa), T, W, dt, S(st));
  });
  m.def("gate_mul", [](uintptr_t y, int64_t ldy, uintptr_t src, int64_t lds_, int T, int N, int dt, uintptr_t st) {
    launch_gate_mul(P(y), ldy, CP(src), lds_, T, N, dt, S(st));
  });
  m.def("act_fn", [](uintptr_t x, int64_t ldx, uintptr_t out, int64_t ldo, int T, int F, int act, float a, float b,
                     int dt, uintptr_t st) { launch_act_fn(CP(x), ldx, P(out), ldo, T, F, act, a, b, dt, S(st)); });
  m.def("qk_norm_cache", [](uintptr_t proj, int64_t ldp, int off_q, int off_k, int off_v, uintptr_t qw, uintptr_t kw,
                            float eps, uintptr_t qout, uintptr_t kc, uintptr_t vc, uintptr_t slots, int T, int H, int G,
                            int maps, int dim, int vdim, int dt, uintptr_t st) {
    launch_qk_norm_cache(CP(proj), ldp, off_q, off_k, off_v, CP(qw), CP(kw), eps, P(qout), P(kc), P(vc), CP(slots), T,
                         H, G, maps, dim, vdim, dt, S(st));
  });
  m.def("diff_combine", [](uintptr_t O, float lam, float eps, float mult, uintptr_t y, int64_t ldy, int T, int H, int G,
                           int vdim, int dt, uintptr_t st) {
    launch_diff_combine(CP(O), lam, eps, mult, P(y), ldy, T, H, G, vdim, dt, S(st));
  });
  m.def("sandwich_add_norm", [](uintptr_t x, uintptr_t y, int64_t ldy, uintptr_t ey, uintptr_t place, uintptr_t wts,
                                int top, uintptr_t sh, int64_t lds_, uintptr_t r, int64_t ldr, uintptr_t rb,
                                uintptr_t wpost, uintptr_t add, uintptr_t wnext, uintptr_t h, int64_t ldh, float eps,
                                int T, int W, int dt, uintptr_t st) {
    launch_sandwich_add_norm(P(x), CP(y), ldy, CP(ey), CP(place), CP(wts), top, CP(sh), lds_, CP(r), ldr, CP(rb),
                             CP(wpost), CP(add), CP(wnext), P(h), ldh, eps, T, W, dt, S(st));
  });
  m.def("token_side_add", [](uintptr_t x, uintptr_t ids, uintptr_t table, int64_t ldt, int vocab, int col0, int d,
                             uintptr_t wg, uintptr_t wp, uintptr_t wn, uintptr_t add, uintptr_t wnext, uintptr_t h,
                             int64_t ldh, float eps, int T, int W, int dt, uintptr_t st) {
    launch_token_side_add(P(x), CP(ids), CP(table), ldt, vocab, col0, d, CP(wg), CP(wp), CP(wn), CP(add), CP(wnext),
                          P(h), ldh, eps, T, W, dt, S(st));
  });
  m.def("rope_pairs_cache", [](uintptr_t proj, int64_t ldp, int off_q, int off_k, int off_v, uintptr_t cs, int rdims,
                               uintptr_t qout, uintptr_t kc, uintptr_t vc, uintptr_t slots, int T, int H, int G,
                               int dim, int vdim, int dt, uintptr_t st) {
    launch_rope_pairs_cache(CP(proj), ldp, off_q, off_k, off_v, CP(cs), rdims, P(qout), P(kc), P(vc), CP(slots), T, H,
                            G, dim, vdim, dt, S(st));
  });
  m.def("pool_update", [](uintptr_t kc, uintptr_t vc, uintptr_t kp, uintptr_t vp, uintptr_t bt, int maxb, uintptr_t cu,
                          uintptr_t ctx, int B, int max_qlen, int nk, int nv, int bs, int pool, int per, int dt,
                          uintptr_t st) {
    launch_pool_update(CP(kc), CP(vc), P(kp), P(vp), CP(bt), maxb, CP(cu), CP(ctx), B, max_qlen, nk, nv, bs, pool, per,
                       dt, S(st));
  });
  m.def("pool_window_attn", [](uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t kp, uintptr_t vp, uintptr_t bt,
                               int maxb, uintptr_t cu, uintptr_t ctx, uintptr_t pb, uintptr_t out, int out_f32, int T,
                               int B, int H, int G, int dim, int vdim, int bs, float scale, int window, int pool,
                               int per, int dt, uintptr_t st) {
    launch_pool_window_attn(CP(q), CP(kc), CP(vc), CP(kp), CP(vp), CP(bt), maxb, CP(cu), CP(ctx), CP(pb), P(out),
                            out_f32, T, B, H, G, dim, vdim, bs, scale, window, pool, per, dt, S(st));
  });
  m.def("pool_attn_mfma_ok", &pool_attn_mfma_ok);
  m.def("pool_window_attn_mfma", [](uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t kp, uintptr_t vp, uintptr_t bt,
                                    int maxb, uintptr_t cu, uintptr_t ctx, uintptr_t pb, uintptr_t out, int out_f32,
                                    uintptr_t part, int nsplit, int64_t row0, int64_t rows, int B, int max_qlen, int H,
                                    int G, int dim, int vdim, int bs, float scale, int window, int pool, int per,
                                    uintptr_t st) {
    launch_pool_window_attn_mfma(CP(q), CP(kc), CP(vc), CP(kp), CP(vp), CP(bt), maxb, CP(cu), CP(ctx), CP(pb), P(out),
                                 out_f32, P(part), nsplit, row0, rows, B, max_qlen, H, G, dim, vdim, bs, scale, window,
                                 pool, per, S(st));
  });
  register_runtime(m);
  register_comm(m);
  register_ctrl(m);
}
