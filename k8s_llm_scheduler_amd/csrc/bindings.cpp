// pybind11 module `_C`: launchers for the gfx950 kernels + native runtime classes.
//
// Tensors cross the boundary as raw device pointers (Python passes tensor.data_ptr()); shape and
// dtype checks live in the Python wrappers (k8s_llm_scheduler_amd/ops/__init__.py).  Kernels are
// launched on the CURRENT PyTorch HIP stream (queried through c10), so they are captured by
// torch.cuda.CUDAGraph (= hipGraph) like any PyTorch op.
#include <hip/hip_runtime.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <chrono>
#include <cstdint>
#include <cstring>
#include <thread>
#include <stdexcept>
#include <string>

#include "runtime/block_allocator.h"
#ifndef K8S_LEAN
#include "runtime/rccl_comm.h"
#include "runtime/xgmi_comm.h"
#endif

namespace py = pybind11;

extern "C" {
void* k8s_current_stream();
int k8s_rmsnorm(void* out, const void* x, void* residual, const void* w, int rows, int H, float eps, hipStream_t s);
int k8s_rope_kv_write(void* q_out, void* k_cache, void* v_cache, const void* qkv, const float* cos_sin,
                      const int* positions, const int* slot_mapping, const int* context_lens, const int* block_tables,
                      int max_blocks, int block_size, int T, int nq, int nkv, int D, hipStream_t s);
int k8s_paged_decode_attention(void* out, void* part_acc, void* part_ml, const void* q, const void* k_cache,
                               const void* v_cache, const int* block_tables, const int* context_lens, float scale,
                               int B, int nq, int nkv, int D, int block_size, int max_blocks, int part, int pmax,
                               hipStream_t s);
int k8s_paged_prefill_attention(void* out, const void* q, const void* k_cache, const void* v_cache, const int* cu_q,
                                const int* context_lens, const int* block_tables, float scale, int num_seqs,
                                int max_qlen, int nq, int nkv, int D, int block_size, int max_blocks, hipStream_t s);
void k8s_gemv_plan(int M, int N_out, int K, int epi, int mode, int* ks_out, int* splits_out);
int k8s_sgemv(void* out, void* partial, const void* x, const void* W, const float* wscale, const void* res, int M,
              int N, int K, int epi, int norm, float eps, hipStream_t s);
long long k8s_sgemv_workspace(int M, int N, int K, int epi, int fp8);
// checked builds (common.h K8S_CHECKED): every instrumented unit's device record pointer; -1 in release builds
int k8s_check_bind_misc(void* rec);
int k8s_check_bind_rope_kv(void* rec);
int k8s_check_bind_attn_decode_fused(void* rec);
int k8s_check_bind_attn_decode_split(void* rec);
int k8s_check_bind_attn_prefill(void* rec);
int k8s_check_bind_attn_decode(void* rec);
int k8s_gemv_set_loop(int wg_per_cu);
int k8s_gemv_set_wide(int on);
int k8s_pgemm_set_prio(int mode);
int k8s_pgemm_set_row_slabs(int on);
int k8s_gemv_fp8(void* out, void* partial, const void* x, const void* W, const float* wscale, int M, int N_out,
                 int K, int epi, const void* res_in, void* res_out, const void* nw, float eps, hipStream_t s);
int k8s_quantize_fp8_rows(void* q, float* scale, const void* w, int N, int K, hipStream_t s);
int k8s_quantize_act_fp8(void* q, float* scale, const void* x, int T, int K, hipStream_t s);
int k8s_quantize_act_fp8_rms(void* q, float* scale, const void* x, int T, int K, int rms, float eps, hipStream_t s);
int k8s_quantize_act_mx(void* q, void* e8, const void* x, int T, int K, hipStream_t s);
int k8s_dequant_fp8_rows(void* w, const void* q, const float* scale, int N, int K, hipStream_t s);
int k8s_gemv(void* out, void* partial, const void* x, const void* W, int M, int N_out, int K, int epi, hipStream_t s);
int k8s_gemv_rms(void* out, void* partial, const void* x, const void* W, const float* wscale, int M, int N_out, int K,
                 int epi, const void* res_in, void* res_out, float eps, hipStream_t s);
int k8s_gemv_norm(void* out, void* partial, const void* x, const void* W, int M, int N_out, int K, int epi,
                  const void* res_in, void* res_out, const void* nw, float eps, hipStream_t s);
int k8s_decode_attention_fused(void* out, void* part_acc, void* part_ml, const void* qkv, const float* cos_sin,
                               void* k_cache, void* v_cache, const int* block_tables, const int* context_lens,
                               float scale, int B, int nq, int nkv, int D, int block_size, int max_blocks, int pmax, int part,
                               void* oq, void* oe, const int* cas, const float* pre, int ngm, int rec_stride,
                               hipStream_t s);
int k8s_decode_prefix_col_blocks(int B, int nq, int nkv);
int k8s_decode_prefix(void* pre, int rec_stride, const void* qkv, const float* cos_sin, const void* k_cache,
                      const void* v_cache, const int* block_tables, const int* context_lens, const int* cas, float scale,
                      int B, int nq, int nkv, int D, int block_size, int max_blocks, int ngm, hipStream_t s);
long long k8s_decode_split_workspace(int B, int nq, int nkv, int pmax);
int k8s_decode_attention_split(void* out, void* part, uint32_t* counters, const void* qkv, const float* cos_sin,
                               void* k_cache, void* v_cache, const int* block_tables, const int* context_lens,
                               float scale, int B, int nq, int nkv, int D, int block_size, int max_blocks, int pmax,
                               hipStream_t s);
int k8s_sample(int* tokens, const float* logits, int B, int Vs, int shards, const float* temperature,
               const float* top_p, const uint32_t* seeds, const int* counter, int* ctx_inc, int* hist, int hist_stride,
               int* steps, void* scratch, void* nuc_scratch, const int* slots, const int* stop_cls, int* stop_json,
               const int* stop_cfg, const int* stop_forced, const int* stop_forced_len, int stop_fstride,
               int stop_eos_tok, int* stop_done, int id_base, void* keys_out, int nuc_passes, hipStream_t s);
int k8s_sample_nuc_local(int level, const float* logits, int B, int Vs, const float* temperature, const float* top_p,
                         const int* ctx_inc, const int* slots, void* nuc_scratch, void* out, hipStream_t s);
int k8s_sample_nuc_combine(int level, const void* g, int ld, int ranks, int B, const float* temperature,
                           const float* top_p, const int* ctx_inc, const int* slots, void* nuc_scratch, void* mine,
                           hipStream_t s);
int k8s_sample_merge(int* tokens, const void* g, int ld, int ranks, int B, int* ctx_inc, int* hist, int hist_stride,
                     int* steps, const int* slots, const int* stop_cls, int* stop_json, const int* stop_cfg,
                     const int* stop_forced, const int* stop_forced_len, int stop_fstride, int stop_eos_tok,
                     int* stop_done, hipStream_t s);
long long k8s_sample_scratch_bytes(int B);
long long k8s_sample_nucleus_bytes(int B, int shards);
int k8s_embedding(void* out, const int* ids, const void* table, int T, int H, int vocab, void* oq, void* oe,
                  hipStream_t s);
int k8s_silu_mul(void* out, const void* gu, int T, int I, hipStream_t s);
int k8s_prefetch(const void* p, long long bytes, int blocks, void* sink, hipStream_t s);
int k8s_hash_init(void* out, int rows, int cols, long long gcols, long long row0, long long col0, uint32_t seed,
                  uint32_t tensor_id, float scale, float shift, hipStream_t s);
int k8s_mgemm_num_configs();
int k8s_mgemm_lds_bytes(int cfg, int mode);
int k8s_mgemm_config(int cfg, int* bm, int* bn, int* threads, int* lds_bytes, int* swiglu, int* rb);
int k8s_mgemm_plan_info(int M, int N_out, int K, int epi, int fp8, int cfg, int nwg, long long* tiles, int* cmax,
                        long long* ws_elems);
int k8s_mgemm(void* out, float* ws, unsigned* tickets, const void* x, const void* W, const float* xs, const float* wsc,
              int M, int N_out, int K, int epi, int fp8, int cfg, int nwg, int cmax, const void* res, int rms,
              float eps, void* oq, void* oe, int fenced, hipStream_t s);
int k8s_pgemm4_num_configs();
int k8s_pgemm4_config(int cfg, int* bp, int* bq, int* lds_bytes);
int k8s_pgemm4_plan(int M, int N_out, int K, int epi, int cfg, int splits, int* nwg, long long* slab_elems);
int k8s_pgemm4(void* out, float* slab, const void* x, const void* W, int M, int N_out, int K, int epi, int cfg,
               int splits, int group_m, const void* res, int rms, float eps, hipStream_t s);
int k8s_embed_rows(float* out, const int* ids, const void* table, int T, int W, int vocab, float scale, int f32,
                   hipStream_t s);
int k8s_resnorm(float* x, const void* branch, const void* branch2, float mult, const void* rowvec, const void* w,
                float offset, float eps, void* out, int T, int W, int groups, int f32, hipStream_t s);
int k8s_norm_mix(void* out, const void* a, long lda, const void* wa, const void* b, const void* wb, float eps, float ca,
                 float cb, int T, int W, int groups, int in_f32, int out_f32, hipStream_t s);
int k8s_postnorm(float* x, const void* branch, const void* branch2, float alpha, float c1, float c2, float gain,
                 float eps, void* out, int T, int W, int f32, hipStream_t s);
int k8s_gate_mul(void* out, const void* y, long ldy, const void* gate, long ldg, int T, int F, int kind, int y_f32,
                 int f32, hipStream_t s);
int k8s_short_conv(void* out, const float* x, long ldx, const float* w, float* state, const int* cu_q,
                   const int* tok_seq, const int* seq_slots, const int* positions, const float* in_bias,
                   const float* out_bias, int act, int T, int C, int taps, int nseq, int unit_cols, int unit_dim,
                   int scale_cols, float scale, float unit_eps, int residual, int out_f32, hipStream_t s);
int k8s_delta_scan(void* out, const float* qkv, const float* proj, long ld, int cb, int ca, int cg, const float* neg_a,
                   const float* dt_bias, const float* normw, float* state, const int* cu_q, const int* seq_slots,
                   const int* positions, int nseq, int H, int G, int D, int V, float eps, int f32, int T, int Lc,
                   float* ws, hipStream_t s);
int k8s_delta_scan_chunks_ok(int D, int V);
long long k8s_delta_scan_workspace(int T, int nseq, int H, int D, int V, int Lc);
int k8s_rglru_scan(void* out, const float* u, const float* gates, const float* gate_bias, const float* rate,
                   const float* proj, long ld, int ycol, const float* ybias, float* state, const int* cu_q,
                   const int* seq_slots, const int* positions, int nseq, int C, int blocks, int max_qlen, int f32,
                   hipStream_t s);
int k8s_act(void* out, const void* x, int T, int F, int kind, float limit, float alpha, const float* row_scale,
            const int* row_map, int f32, hipStream_t s);
int k8s_gemm_any(void* C, const void* A, const void* W, int M, int N, int K, long lda, long ldw, long ldc, int batch,
                 long sA, long sW, long sC, const int* a_rows, const int* tiles, int ntiles, int in_f32, int out_f32,
                 hipStream_t s);
int k8s_token_shift(void* out, const void* h, const void* mu, const void* state, const int* cu_q, const int* tok_seq,
                    const int* seq_slots, const int* positions, int n, int T, int W, int f32, hipStream_t s);
int k8s_shift_save(void* state, const void* h, const int* cu_q, const int* seq_slots, const int* positions, int nseq,
                   int W, int f32, hipStream_t s);
int k8s_wkv_max_dim();
long long k8s_wkv_workspace(int T, int nseq, int H, int D, int Lc);
int k8s_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, long ld, const float* z,
                 const void* w0, const void* u, const void* lnw, float* state, const int* cu_q, const int* seq_slots,
                 const int* positions, int nseq, int H, int D, float eps, int f32, int T, int Lc, float* ws,
                 hipStream_t s);
int k8s_latent_kv_write(void* cache, const void* dkv, const void* normw, void* q, const float* cos_sin,
                        const int* positions, const int* slot_mapping, int T, int C, int R, int H, int Dn, int dims,
                        float eps, int f32, long ldd, int interleaved, hipStream_t s);
int k8s_latent_attention(void* out, const void* q_abs, const void* q, const void* cache, const int* block_tables,
                         int max_blocks, const int* tok_seq, const int* positions, int T, int C, int R, int H, int Dn,
                         int window, float scale, int bs, int f32, const float* sinks, hipStream_t s);
int k8s_latent_mfma_ok(int C, int R, int Dn);
int k8s_latent_attention_mfma(void* out, float* pacc, float* pml, const void* q_abs, const void* q, const void* cache,
                              const int* block_tables, int max_blocks, const int* tok_seq, const int* positions, int T,
                              int C, int R, int H, int Dn, int window, float scale, int bs, int nsplit, const int* cu_q,
                              int nseq, int max_qlen, const float* sinks, hipStream_t s);
int k8s_moe_route(int* idx, float* w, const float* logits, int ld, int T, int E, int top, float scale, int mode,
                  hipStream_t s);
int k8s_window_kv_write(void* kcache, void* vcache, void* qkv, long ld, int koff, int voff, const void* qb,
                        const void* kb, const void* vb, const float* cos_sin, const int* positions,
                        const int* slot_mapping, const float* vfirst_in, float* vfirst_out, float lam, int T, int H, int G,
                        int D, int V, int dims, float eps, int unit, int half_layout, const void* qnw, const void* knw,
                        const void* hqw, const void* hkw, int f32, hipStream_t s);
int k8s_window_pool(float* kpool, float* vpool, const void* kcache, const void* vcache, const int* block_tables,
                    int max_blocks, const int* tok_seq, const int* positions, int T, int G, int D, int V, int P, int bs,
                    int f32, hipStream_t s);
int k8s_window_tile_rows(int H, int G, int D, int V);
int k8s_window_attention(void* out, float* pacc, float* pml, const void* q, long ldq, const void* gate, long ldg,
                         const void* kcache, const void* vcache, const float* kpool, const float* vpool,
                         const int* block_tables, int max_blocks, const int* tok_seq, const int* positions, int T, int H,
                         int G, int D, int V, int window, int P, float scale, int sink, int bs, int nsplit, int chunk,
                         float softcap, const float* sinkv, int gate_ph, int f32, hipStream_t s);
int k8s_window_mfma_ok(int H, int G, int D, int V);
int k8s_window_attention_mfma(void* out, const void* q, long ldq, const void* gate, long ldg, const void* kcache,
                              const void* vcache, const float* kpool, const float* vpool, const int* block_tables,
                              int max_blocks, const int* cu_q, const int* positions, int nseq, int max_qlen, int H, int G,
                              int D, int V, int window, int P, float scale, int sink, int bs, int chunk, float softcap,
                              const float* sinkv, int gate_ph, hipStream_t s);
int k8s_gated_scan_max_dim();
long long k8s_gated_scan_record(int kind, int D, int V);
int k8s_gated_scan(void* out, const float* proj, long ld, int kind, int cq, int ck, int cv, int ci, int cf, int cg,
                   const void* fbias, const void* ibias, const void* lower, const void* normw, float* state,
                   const int* cu_q, const int* seq_slots, const int* positions, int nseq, int H, int D, int V, float eps,
                   float cap, int f32, int T, int Lc, float* ws, const float* aux, long ldaux, const float* hpar, int R,
                   hipStream_t s);
long long k8s_gated_scan_workspace(int T, int nseq, int H, int D, int V, int Lc);
int k8s_moe_align(int* sorted_tok, int* pos_of_pair, int* seg, int* tiles, int ntiles, const int* topk_idx, int P,
                  int top, int E, int BM, hipStream_t s);
int k8s_moe_combine(void* z, const void* D, const int* pos, const float* w, const void* shared, const float* logits,
                    int ld, int sg_col, int T, int W, int top, int f32, hipStream_t s);
int k8s_pgemm_num_configs();
int k8s_pgemm_config(int cfg, int* bp, int* bq, int* lds_bytes);
int k8s_pgemm_plan(int M, int N_out, int K, int epi, int fp8, int cfg, int splits, int* nwg, long long* ws_elems,
                   int* tickets);
int k8s_pgemm(void* out, float* ws, unsigned* tickets, const void* x, const void* W, const float* xs, const float* wsc,
              int M, int N_out, int K, int epi, int fp8, int cfg, int splits, int group_m, const void* res, int rms,
              float eps, void* oq, void* oe, hipStream_t s);
}

namespace {

template <typename T = void>
inline T* P(uintptr_t p) { return reinterpret_cast<T*>(p); }

inline hipStream_t S(int64_t s) {
  return s < 0 ? reinterpret_cast<hipStream_t>(k8s_current_stream()) : reinterpret_cast<hipStream_t>(s);
}

inline void check(int rc, const char* what) {
  if (rc == 0) return;
  std::string msg = std::string(what) + " failed: ";
  if (rc < 0) msg += "invalid arguments (code " + std::to_string(rc) + ")";
  else msg += hipGetErrorString(static_cast<hipError_t>(rc));
  throw std::runtime_error(msg);
}

}  // namespace

#ifndef K8S_MODULE_NAME
#define K8S_MODULE_NAME _C
#endif
PYBIND11_MODULE(K8S_MODULE_NAME, m) {
#ifdef K8S_CHECKED
  m.attr("checked") = true;
#else
  m.attr("checked") = false;
#endif
  // point every instrumented unit at one device record (ops.check_*); returns 0, or nonzero in release builds
  m.def("check_bind", [](uintptr_t rec) {
    int rc = 0;
#ifdef K8S_LEAN
    rc |= k8s_check_bind_misc(reinterpret_cast<void*>(rec));
#else
    for (auto f : {k8s_check_bind_misc, k8s_check_bind_rope_kv, k8s_check_bind_attn_decode_fused,
                   k8s_check_bind_attn_decode_split, k8s_check_bind_attn_prefill, k8s_check_bind_attn_decode})
      rc |= f(reinterpret_cast<void*>(rec));
#endif
    return rc;
  });
  m.doc() = "gfx950 HIP kernels and native runtime of k8s_llm_scheduler_amd";
  m.attr("ARCH") = "gfx950";
  // The lean module (-DK8S_LEAN: python -m k8s_llm_scheduler_amd._build --lean) holds the runtime, the sampler and the
  // kernels of the fp32-stream models only; the tuned GEMV / GEMM kernels, the Llama attention kernels, fp8 and the
  // communicators are left out, and the any-shape GEMM serves every product.
#ifdef K8S_LEAN
  m.attr("lean") = true;
#else
  m.attr("lean") = false;
#endif

  m.def("rmsnorm", [](uintptr_t out, uintptr_t x, uintptr_t residual, uintptr_t w, int rows, int H, float eps,
                      int64_t s) { check(k8s_rmsnorm(P(out), P(x), P(residual), P(w), rows, H, eps, S(s)), "rmsnorm"); });
#ifndef K8S_LEAN
  m.def("rope_kv_write", [](uintptr_t q_out, uintptr_t kc, uintptr_t vc, uintptr_t qkv, uintptr_t cos_sin,
                            uintptr_t pos, uintptr_t slots, uintptr_t ctx, uintptr_t bt, int max_blocks, int bs, int T,
                            int nq, int nkv, int D, int64_t s) {
    check(k8s_rope_kv_write(P(q_out), P(kc), P(vc), P(qkv), P<float>(cos_sin), P<int>(pos), P<int>(slots),
                            P<int>(ctx), P<int>(bt), max_blocks, bs, T, nq, nkv, D, S(s)),
          "rope_kv_write");
  });
  m.def("paged_decode_attention", [](uintptr_t out, uintptr_t pacc, uintptr_t pml, uintptr_t q, uintptr_t kc,
                                     uintptr_t vc, uintptr_t bt, uintptr_t ctx, float scale, int B, int nq, int nkv,
                                     int D, int bs, int max_blocks, int part, int pmax, int64_t s) {
    check(k8s_paged_decode_attention(P(out), P(pacc), P(pml), P(q), P(kc), P(vc), P<int>(bt), P<int>(ctx), scale, B,
                                     nq, nkv, D, bs, max_blocks, part, pmax, S(s)),
          "paged_decode_attention");
  });
  m.def("paged_prefill_attention", [](uintptr_t out, uintptr_t q, uintptr_t kc, uintptr_t vc, uintptr_t cu_q,
                                      uintptr_t ctx, uintptr_t bt, float scale, int nseq, int max_qlen, int nq,
                                      int nkv, int D, int bs, int max_blocks, int64_t s) {
    check(k8s_paged_prefill_attention(P(out), P(q), P(kc), P(vc), P<int>(cu_q), P<int>(ctx), P<int>(bt), scale, nseq,
                                      max_qlen, nq, nkv, D, bs, max_blocks, S(s)),
          "paged_prefill_attention");
  });
#endif
  // Bounded wait for a recorded hipEvent (torch.cuda.Event.cuda_event) with the GIL released: the engine's per-step
  // device waits must neither block forever (a stalled collective) nor hold the GIL while they poll (the control
  // plane's watch / worker threads run beside the engine loop).  True once the event completed, False at the timeout.
  m.def("event_wait", [](uintptr_t ev, double timeout_s) {
    py::gil_scoped_release nogil;
    const auto e = reinterpret_cast<hipEvent_t>(ev);
    const auto t0 = std::chrono::steady_clock::now();
    for (long spins = 0;; ++spins) {
      const hipError_t r = hipEventQuery(e);
      if (r == hipSuccess) return true;
      if (r != hipErrorNotReady) throw std::runtime_error(std::string("hipEventQuery: ") + hipGetErrorString(r));
      const double waited = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
      if (waited >= timeout_s) return false;
      if (waited < 0.005) std::this_thread::yield();   // decode steps end within milliseconds: stay responsive
      else std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
  }, py::arg("event"), py::arg("timeout_s"));
#ifndef K8S_LEAN
  m.def("pgemm_set_prio", [](int mode) { return k8s_pgemm_set_prio(mode); });
  m.def("pgemm_set_row_slabs", [](int on) { return k8s_pgemm_set_row_slabs(on); });
  m.def("gemv_set_wide", [](int on) { return k8s_gemv_set_wide(on); });
  m.def("gemv_set_loop", [](int wg) { return k8s_gemv_set_loop(wg); });
  m.def("gemv_plan", [](int M, int N, int K, int epi, int mode) {
    int ks, sp;
    k8s_gemv_plan(M, N, K, epi, mode, &ks, &sp);
    return py::make_tuple(ks, sp);
  });
  m.def("gemv_fp8", [](uintptr_t out, uintptr_t partial, uintptr_t x, uintptr_t W, uintptr_t wscale, int M, int N,
                       int K, int epi, uintptr_t res_in, uintptr_t res_out, uintptr_t nw, float eps, int64_t s) {
    check(k8s_gemv_fp8(P(out), P(partial), P(x), P(W), P<float>(wscale), M, N, K, epi, P(res_in), P(res_out), P(nw),
                       eps, S(s)),
          "gemv_fp8");
  });
  m.def("quantize_fp8_rows", [](uintptr_t q, uintptr_t scale, uintptr_t w, int N, int K, int64_t s) {
    check(k8s_quantize_fp8_rows(P(q), P<float>(scale), P(w), N, K, S(s)), "quantize_fp8_rows");
  });
  m.def("quantize_act_fp8", [](uintptr_t q, uintptr_t scale, uintptr_t x, int T, int K, int64_t s) {
    check(k8s_quantize_act_fp8(P(q), P<float>(scale), P(x), T, K, S(s)), "quantize_act_fp8");
  });
  m.def("quantize_act_mx", [](uintptr_t q, uintptr_t e8, uintptr_t x, int T, int K, int64_t s) {
    check(k8s_quantize_act_mx(P(q), P(e8), P(x), T, K, S(s)), "quantize_act_mx");
  });
  m.def("quantize_act_fp8_rms", [](uintptr_t q, uintptr_t scale, uintptr_t x, int T, int K, int rms, float eps,
                                   int64_t s) {
    check(k8s_quantize_act_fp8_rms(P(q), P<float>(scale), P(x), T, K, rms, eps, S(s)), "quantize_act_fp8_rms");
  });
  m.def("dequant_fp8_rows", [](uintptr_t w, uintptr_t q, uintptr_t scale, int N, int K, int64_t s) {
    check(k8s_dequant_fp8_rows(P(w), P(q), P<float>(scale), N, K, S(s)), "dequant_fp8_rows");
  });
  m.def("gemv", [](uintptr_t out, uintptr_t partial, uintptr_t x, uintptr_t W, int M, int N, int K, int epi,
                   int64_t s) { check(k8s_gemv(P(out), P(partial), P(x), P(W), M, N, K, epi, S(s)), "gemv"); });
  m.def("gemv_norm", [](uintptr_t out, uintptr_t partial, uintptr_t x, uintptr_t W, int M, int N, int K, int epi,
                        uintptr_t res_in, uintptr_t res_out, uintptr_t nw, float eps, int64_t s) {
    check(k8s_gemv_norm(P(out), P(partial), P(x), P(W), M, N, K, epi, P(res_in), P(res_out), P(nw), eps, S(s)),
          "gemv_norm");
  });
  // small-batch decode GEMV (3..8 rows, x in registers): returns -5 (nothing launched) for a combination it does not
  // instantiate, so the caller can take another kernel
  m.def("sgemv", [](uintptr_t out, uintptr_t partial, uintptr_t x, uintptr_t W, uintptr_t wscale, uintptr_t res, int M,
                    int N, int K, int epi, int norm, float eps, int64_t s) {
    const int rc = k8s_sgemv(P(out), P(partial), P(x), P(W), P<float>(wscale), P(res), M, N, K, epi, norm, eps, S(s));
    if (rc != -5) check(rc, "sgemv");
    return rc;
  });
  m.def("sgemv_workspace", [](int M, int N, int K, int epi, int fp8) { return k8s_sgemv_workspace(M, N, K, epi, fp8); });
  m.def("gemv_rms", [](uintptr_t out, uintptr_t partial, uintptr_t x, uintptr_t W, uintptr_t wscale, int M, int N,
                       int K, int epi, uintptr_t res_in, uintptr_t res_out, float eps, int64_t s) {
    check(k8s_gemv_rms(P(out), P(partial), P(x), P(W), P<float>(wscale), M, N, K, epi, P(res_in), P(res_out), eps, S(s)),
          "gemv_rms");
  });
  m.def("decode_attention_fused", [](uintptr_t out, uintptr_t pacc, uintptr_t pml, uintptr_t qkv, uintptr_t cos_sin,
                                     uintptr_t kc, uintptr_t vc, uintptr_t bt, uintptr_t ctx, float scale, int B, int nq,
                                     int nkv, int D, int bs, int max_blocks, int pmax, int part, int64_t s,
                                     uintptr_t oq, uintptr_t oe, uintptr_t cas, uintptr_t pre, int ngm, int rec_stride) {
    check(k8s_decode_attention_fused(P(out), P(pacc), P(pml), P(qkv), P<float>(cos_sin), P(kc), P(vc), P<int>(bt),
                                     P<int>(ctx), scale, B, nq, nkv, D, bs, max_blocks, pmax, part, P(oq), P(oe),
                                     P<int>(cas), P<float>(pre), ngm, rec_stride, S(s)),
          "decode_attention_fused");
  }, py::arg("out"), py::arg("pacc"), py::arg("pml"), py::arg("qkv"), py::arg("cos_sin"), py::arg("kc"),
     py::arg("vc"), py::arg("bt"), py::arg("ctx"), py::arg("scale"), py::arg("B"), py::arg("nq"), py::arg("nkv"),
     py::arg("D"), py::arg("bs"), py::arg("max_blocks"), py::arg("pmax"), py::arg("part"), py::arg("s"),
     py::arg("oq") = 0, py::arg("oe") = 0, py::arg("cas") = 0, py::arg("pre") = 0, py::arg("ngm") = 0,
     py::arg("rec_stride") = 0);
  m.def("decode_prefix_col_blocks", [](int B, int nq, int nkv) { return k8s_decode_prefix_col_blocks(B, nq, nkv); });
  m.def("decode_prefix", [](uintptr_t pre, int rec_stride, uintptr_t qkv, uintptr_t cos_sin, uintptr_t kc,
                            uintptr_t vc, uintptr_t bt, uintptr_t ctx, uintptr_t cas, float scale, int B, int nq, int nkv,
                            int D, int bs, int max_blocks, int ngm, int64_t s) {
    check(k8s_decode_prefix(P(pre), rec_stride, P(qkv), P<float>(cos_sin), P(kc), P(vc), P<int>(bt), P<int>(ctx),
                            P<int>(cas), scale, B, nq, nkv, D, bs, max_blocks, ngm, S(s)),
          "decode_prefix");
  });
  m.def("decode_split_workspace", [](int B, int nq, int nkv, int pmax) {
    return k8s_decode_split_workspace(B, nq, nkv, pmax);
  });
  m.def("decode_attention_split", [](uintptr_t out, uintptr_t part, uintptr_t counters, uintptr_t qkv,
                                     uintptr_t cos_sin, uintptr_t kc, uintptr_t vc, uintptr_t bt, uintptr_t ctx,
                                     float scale, int B, int nq, int nkv, int D, int bs, int max_blocks, int pmax,
                                     int64_t s) {
    check(k8s_decode_attention_split(P(out), P(part), P<uint32_t>(counters), P(qkv), P<float>(cos_sin), P(kc), P(vc),
                                     P<int>(bt), P<int>(ctx), scale, B, nq, nkv, D, bs, max_blocks, pmax, S(s)),
          "decode_attention_split");
  });
#endif
  m.def("sample", [](uintptr_t tokens, uintptr_t logits, int B, int Vs, int shards, uintptr_t temp, uintptr_t top_p,
                     uintptr_t seeds, uintptr_t counter, uintptr_t ctx_inc, uintptr_t hist, int hist_stride,
                     uintptr_t steps, uintptr_t scratch, uintptr_t nuc_scratch, uintptr_t slots, uintptr_t cls,
                     uintptr_t json, uintptr_t cfg, uintptr_t forced, uintptr_t forced_len, int fstride, int eos_tok,
                     uintptr_t done, int64_t s, int id_base, uintptr_t keys_out, int nuc_passes) {
    check(k8s_sample(P<int>(tokens), P<float>(logits), B, Vs, shards, P<float>(temp), P<float>(top_p),
                     P<uint32_t>(seeds), P<int>(counter), P<int>(ctx_inc), P<int>(hist), hist_stride, P<int>(steps),
                     P(scratch), P(nuc_scratch), P<int>(slots), P<int>(cls), P<int>(json), P<int>(cfg), P<int>(forced),
                     P<int>(forced_len), fstride, eos_tok, P<int>(done), id_base, P(keys_out), nuc_passes, S(s)),
          "sample");
  }, py::arg("tokens"), py::arg("logits"), py::arg("B"), py::arg("Vs"), py::arg("shards"), py::arg("temp"),
     py::arg("top_p"), py::arg("seeds"), py::arg("counter"), py::arg("ctx_inc"), py::arg("hist"),
     py::arg("hist_stride"), py::arg("steps"), py::arg("scratch"), py::arg("nuc_scratch"), py::arg("slots"),
     py::arg("cls"), py::arg("json"), py::arg("cfg"), py::arg("forced"), py::arg("forced_len"), py::arg("fstride"),
     py::arg("eos_tok"), py::arg("done"), py::arg("stream"), py::arg("id_base") = 0, py::arg("keys_out") = 0,
     py::arg("nuc_passes") = 1);
  // vocab-parallel sampling stages (sampler.hip): the TP ranks exchange row maxima / bin totals / best keys
  m.def("sample_nuc_local", [](int level, uintptr_t logits, int B, int Vs, uintptr_t temp, uintptr_t top_p,
                               uintptr_t ctx_inc, uintptr_t slots, uintptr_t nuc_scratch, uintptr_t out, int64_t s) {
    check(k8s_sample_nuc_local(level, P<float>(logits), B, Vs, P<float>(temp), P<float>(top_p), P<int>(ctx_inc),
                               P<int>(slots), P(nuc_scratch), P(out), S(s)),
          "sample_nuc_local");
  });
  m.def("sample_nuc_combine", [](int level, uintptr_t g, int ld, int ranks, int B, uintptr_t temp, uintptr_t top_p,
                                 uintptr_t ctx_inc, uintptr_t slots, uintptr_t nuc_scratch, uintptr_t mine, int64_t s) {
    check(k8s_sample_nuc_combine(level, P(g), ld, ranks, B, P<float>(temp), P<float>(top_p), P<int>(ctx_inc),
                                 P<int>(slots), P(nuc_scratch), P(mine), S(s)),
          "sample_nuc_combine");
  });
  m.def("sample_merge", [](uintptr_t tokens, uintptr_t g, int ld, int ranks, int B, uintptr_t ctx_inc, uintptr_t hist,
                           int hist_stride, uintptr_t steps, uintptr_t slots, uintptr_t cls, uintptr_t json,
                           uintptr_t cfg, uintptr_t forced, uintptr_t forced_len, int fstride, int eos_tok,
                           uintptr_t done, int64_t s) {
    check(k8s_sample_merge(P<int>(tokens), P(g), ld, ranks, B, P<int>(ctx_inc), P<int>(hist), hist_stride,
                           P<int>(steps), P<int>(slots), P<int>(cls), P<int>(json), P<int>(cfg), P<int>(forced),
                           P<int>(forced_len), fstride, eos_tok, P<int>(done), S(s)),
          "sample_merge");
  });
  // Host memory the GPU can write (fine-grained, coherent): the decode graphs' done flags, polled by the host
  // between replays without a device synchronisation.
  m.def("host_mapped_alloc", [](size_t bytes) {
    void* p = nullptr;
    if (hipHostMalloc(&p, bytes, hipHostMallocMapped | hipHostMallocCoherent) != hipSuccess)
      throw std::runtime_error("hipHostMalloc failed");
    std::memset(p, 0, bytes);
    void* d = nullptr;
    if (hipHostGetDevicePointer(&d, p, 0) != hipSuccess) throw std::runtime_error("hipHostGetDevicePointer failed");
    return py::make_tuple(reinterpret_cast<uintptr_t>(p), reinterpret_cast<uintptr_t>(d));
  });
  m.def("host_mapped_free", [](uintptr_t p) { (void)hipHostFree(reinterpret_cast<void*>(p)); });
  m.def("sample_scratch_bytes", [](int B) { return k8s_sample_scratch_bytes(B); });
  m.def("sample_nucleus_bytes", [](int B, int shards) { return k8s_sample_nucleus_bytes(B, shards); });
  m.def("embedding", [](uintptr_t out, uintptr_t ids, uintptr_t table, int T, int H, int vocab, int64_t s,
                        uintptr_t oq, uintptr_t oe) {
    check(k8s_embedding(P(out), P<int>(ids), P(table), T, H, vocab, P(oq), P(oe), S(s)), "embedding");
  }, py::arg("out"), py::arg("ids"), py::arg("table"), py::arg("T"), py::arg("H"), py::arg("vocab"), py::arg("s"),
     py::arg("oq") = 0, py::arg("oe") = 0);
  m.def("prefetch", [](uintptr_t p, long long bytes, int blocks, uintptr_t sink, int64_t s) {
    check(k8s_prefetch(P(p), bytes, blocks, P(sink), S(s)), "prefetch");
  });
  m.def("silu_mul", [](uintptr_t out, uintptr_t gu, int T, int I, int64_t s) {
    check(k8s_silu_mul(P(out), P(gu), T, I, S(s)), "silu_mul");
  });
  m.def("hash_init", [](uintptr_t out, int rows, int cols, long long gcols, long long row0, long long col0,
                        uint32_t seed, uint32_t tid, float scale, float shift, int64_t s) {
    check(k8s_hash_init(P(out), rows, cols, gcols, row0, col0, seed, tid, scale, shift, S(s)), "hash_init");
  });

  // fp32 residual stream, recurrent / latent mixers, mixture of experts (stream32.hip, mixers.hip, moe.hip)
  m.def("embed_rows", [](uintptr_t out, uintptr_t ids, uintptr_t table, int T, int W, int vocab, float scale, int f32,
                         int64_t s) {
    check(k8s_embed_rows(P<float>(out), P<int>(ids), P(table), T, W, vocab, scale, f32, S(s)), "embed_rows");
  });
  m.def("resnorm", [](uintptr_t x, uintptr_t branch, uintptr_t branch2, float mult, uintptr_t rowvec, uintptr_t w,
                      float offset, float eps, uintptr_t out, int T, int W, int groups, int f32, int64_t s) {
    check(k8s_resnorm(P<float>(x), P(branch), P(branch2), mult, P(rowvec), P(w), offset, eps, P(out), T, W, groups, f32,
                      S(s)), "resnorm");
  });
  m.def("norm_mix", [](uintptr_t out, uintptr_t a, long lda, uintptr_t wa, uintptr_t b, uintptr_t wb, float eps,
                       float ca, float cb, int T, int W, int groups, int in_f32, int out_f32, int64_t s) {
    check(k8s_norm_mix(P(out), P(a), lda, P(wa), P(b), P(wb), eps, ca, cb, T, W, groups, in_f32, out_f32, S(s)),
          "norm_mix");
  });
  m.def("postnorm", [](uintptr_t x, uintptr_t branch, uintptr_t branch2, float alpha, float c1, float c2, float gain,
                       float eps, uintptr_t out, int T, int W, int f32, int64_t s) {
    check(k8s_postnorm(P<float>(x), P(branch), P(branch2), alpha, c1, c2, gain, eps, P(out), T, W, f32, S(s)),
          "postnorm");
  });
  m.def("gate_mul", [](uintptr_t out, uintptr_t y, long ldy, uintptr_t gate, long ldg, int T, int F, int kind,
                       int y_f32, int f32, int64_t s) {
    check(k8s_gate_mul(P(out), P(y), ldy, P(gate), ldg, T, F, kind, y_f32, f32, S(s)), "gate_mul");
  });
  // short convolutions, the gated delta rule, the real-gated linear recurrent unit (delta_scan.hip)
  m.def("short_conv", [](uintptr_t out, uintptr_t x, long ldx, uintptr_t w, uintptr_t state, uintptr_t cu_q,
                         uintptr_t tok_seq, uintptr_t seq_slots, uintptr_t positions, uintptr_t in_bias,
                         uintptr_t out_bias, int act, int T, int C, int taps, int nseq, int unit_cols, int unit_dim,
                         int scale_cols, float scale, float unit_eps, int residual, int out_f32, int64_t s) {
    check(k8s_short_conv(P(out), P<float>(x), ldx, P<float>(w), P<float>(state), P<int>(cu_q), P<int>(tok_seq),
                         P<int>(seq_slots), P<int>(positions), P<float>(in_bias), P<float>(out_bias), act, T, C, taps,
                         nseq, unit_cols, unit_dim, scale_cols, scale, unit_eps, residual, out_f32, S(s)),
          "short_conv");
  });
  m.def("delta_scan", [](uintptr_t out, uintptr_t qkv, uintptr_t proj, long ld, int cb, int ca, int cg, uintptr_t neg_a,
                         uintptr_t dt_bias, uintptr_t normw, uintptr_t state, uintptr_t cu_q, uintptr_t seq_slots,
                         uintptr_t positions, int nseq, int H, int G, int D, int V, float eps, int f32, int T, int Lc,
                         uintptr_t ws, int64_t s) {
    check(k8s_delta_scan(P(out), P<float>(qkv), P<float>(proj), ld, cb, ca, cg, P<float>(neg_a), P<float>(dt_bias),
                         P<float>(normw), P<float>(state), P<int>(cu_q), P<int>(seq_slots), P<int>(positions), nseq, H,
                         G, D, V, eps, f32, T, Lc, P<float>(ws), S(s)), "delta_scan");
  });
  m.def("delta_scan_chunks_ok", [](int D, int V) { return k8s_delta_scan_chunks_ok(D, V) != 0; });
  m.def("delta_scan_workspace", [](int T, int nseq, int H, int D, int V, int Lc) {
    return k8s_delta_scan_workspace(T, nseq, H, D, V, Lc);
  });
  m.def("rglru_scan", [](uintptr_t out, uintptr_t u, uintptr_t gates, uintptr_t gate_bias, uintptr_t rate,
                         uintptr_t proj, long ld, int ycol, uintptr_t ybias, uintptr_t state, uintptr_t cu_q,
                         uintptr_t seq_slots, uintptr_t positions, int nseq, int C, int blocks, int max_qlen, int f32,
                         int64_t s) {
    check(k8s_rglru_scan(P(out), P<float>(u), P<float>(gates), P<float>(gate_bias), P<float>(rate), P<float>(proj), ld,
                         ycol, P<float>(ybias), P<float>(state), P<int>(cu_q), P<int>(seq_slots), P<int>(positions),
                         nseq, C, blocks, max_qlen, f32, S(s)), "rglru_scan");
  });
  m.def("act", [](uintptr_t out, uintptr_t x, int T, int F, int kind, float limit, float alpha, uintptr_t row_scale,
                  uintptr_t row_map, int f32, int64_t s) {
    check(k8s_act(P(out), P(x), T, F, kind, limit, alpha, P<float>(row_scale), P<int>(row_map), f32, S(s)), "act");
  });
  m.def("gemm_any", [](uintptr_t C, uintptr_t A, uintptr_t W, int M, int N, int K, long lda, long ldw, long ldc,
                       int batch, long sA, long sW, long sC, uintptr_t a_rows, uintptr_t tiles, int ntiles, int in_f32,
                       int out_f32, int64_t s) {
    check(k8s_gemm_any(P(C), P(A), P(W), M, N, K, lda, ldw, ldc, batch, sA, sW, sC, P<int>(a_rows), P<int>(tiles),
                       ntiles, in_f32, out_f32, S(s)), "gemm_any");
  });
  m.def("token_shift", [](uintptr_t out, uintptr_t h, uintptr_t mu, uintptr_t state, uintptr_t cu_q, uintptr_t tok_seq,
                          uintptr_t seq_slots, uintptr_t positions, int n, int T, int W, int f32, int64_t s) {
    check(k8s_token_shift(P(out), P(h), P(mu), P(state), P<int>(cu_q), P<int>(tok_seq), P<int>(seq_slots),
                          P<int>(positions), n, T, W, f32, S(s)), "token_shift");
  });
  m.def("shift_save", [](uintptr_t state, uintptr_t h, uintptr_t cu_q, uintptr_t seq_slots, uintptr_t positions,
                         int nseq, int W, int f32, int64_t s) {
    check(k8s_shift_save(P(state), P(h), P<int>(cu_q), P<int>(seq_slots), P<int>(positions), nseq, W, f32, S(s)),
          "shift_save");
  });
  m.def("wkv_max_dim", []() { return k8s_wkv_max_dim(); });
  m.def("wkv_scan", [](uintptr_t out, uintptr_t r, uintptr_t k, uintptr_t v, uintptr_t g, long ld, uintptr_t z,
                       uintptr_t w0, uintptr_t u, uintptr_t lnw, uintptr_t state, uintptr_t cu_q, uintptr_t seq_slots,
                       uintptr_t positions, int nseq, int H, int D, float eps, int f32, int T, int Lc, uintptr_t ws,
                       int64_t s) {
    check(k8s_wkv_scan(P(out), P(r), P(k), P(v), P(g), ld, P<float>(z), P(w0), P(u), P(lnw), P<float>(state),
                       P<int>(cu_q), P<int>(seq_slots), P<int>(positions), nseq, H, D, eps, f32, T, Lc, P<float>(ws),
                       S(s)), "wkv_scan");
  });
  m.def("wkv_workspace", [](int T, int nseq, int H, int D, int Lc) { return k8s_wkv_workspace(T, nseq, H, D, Lc); });
  m.def("latent_kv_write", [](uintptr_t cache, uintptr_t dkv, uintptr_t normw, uintptr_t q, uintptr_t cos_sin,
                              uintptr_t positions, uintptr_t slots, int T, int C, int R, int H, int Dn, int dims,
                              float eps, int f32, long ldd, int interleaved, int64_t s) {
    check(k8s_latent_kv_write(P(cache), P(dkv), P(normw), P(q), P<float>(cos_sin), P<int>(positions), P<int>(slots), T,
                              C, R, H, Dn, dims, eps, f32, ldd, interleaved, S(s)), "latent_kv_write");
  });
  m.def("latent_attention", [](uintptr_t out, uintptr_t q_abs, uintptr_t q, uintptr_t cache, uintptr_t bt,
                               int max_blocks, uintptr_t tok_seq, uintptr_t positions, int T, int C, int R, int H,
                               int Dn, int window, float scale, int bs, int f32, uintptr_t sinks, int64_t s) {
    check(k8s_latent_attention(P(out), P(q_abs), P(q), P(cache), P<int>(bt), max_blocks, P<int>(tok_seq),
                               P<int>(positions), T, C, R, H, Dn, window, scale, bs, f32, P<float>(sinks), S(s)),
          "latent_attention");
  });
  m.def("latent_mfma_ok", [](int C, int R, int Dn) { return k8s_latent_mfma_ok(C, R, Dn) != 0; });
  m.def("latent_attention_mfma", [](uintptr_t out, uintptr_t pacc, uintptr_t pml, uintptr_t q_abs, uintptr_t q,
                                    uintptr_t cache, uintptr_t bt, int max_blocks, uintptr_t tok_seq,
                                    uintptr_t positions, int T, int C, int R, int H, int Dn, int window, float scale,
                                    int bs, int nsplit, uintptr_t cu_q, int nseq, int max_qlen, uintptr_t sinks,
                                    int64_t s) {
    check(k8s_latent_attention_mfma(P(out), P<float>(pacc), P<float>(pml), P(q_abs), P(q), P(cache), P<int>(bt),
                                    max_blocks, P<int>(tok_seq), P<int>(positions), T, C, R, H, Dn, window, scale, bs,
                                    nsplit, P<int>(cu_q), nseq, max_qlen, P<float>(sinks), S(s)),
          "latent_attention_mfma");
  });
  m.def("moe_route", [](uintptr_t idx, uintptr_t w, uintptr_t logits, int ld, int T, int E, int top, float scale,
                        int mode, int64_t s) {
    check(k8s_moe_route(P<int>(idx), P<float>(w), P<float>(logits), ld, T, E, top, scale, mode, S(s)), "moe_route");
  });
  // windowed grouped-query attention with pooled far blocks, gated matrix-state recurrences (window_attn.hip,
  // gated_scan.hip)
  m.def("window_kv_write", [](uintptr_t kcache, uintptr_t vcache, uintptr_t qkv, long ld, int koff, int voff,
                              uintptr_t qb, uintptr_t kb, uintptr_t vb, uintptr_t cos_sin, uintptr_t positions,
                              uintptr_t slots, uintptr_t vfirst_in, uintptr_t vfirst_out, float lam, int T, int H, int G,
                              int D, int V, int dims, float eps, int unit, int half_layout, uintptr_t qnw,
                              uintptr_t knw, uintptr_t hqw, uintptr_t hkw, int f32, int64_t s) {
    check(k8s_window_kv_write(P(kcache), P(vcache), P(qkv), ld, koff, voff, P(qb), P(kb), P(vb), P<float>(cos_sin),
                              P<int>(positions), P<int>(slots), P<float>(vfirst_in), P<float>(vfirst_out), lam, T, H, G,
                              D, V, dims, eps, unit, half_layout, P(qnw), P(knw), P(hqw), P(hkw), f32, S(s)),
          "window_kv_write");
  });
  m.def("window_pool", [](uintptr_t kpool, uintptr_t vpool, uintptr_t kcache, uintptr_t vcache, uintptr_t bt,
                          int max_blocks, uintptr_t tok_seq, uintptr_t positions, int T, int G, int D, int V, int P_,
                          int bs, int f32, int64_t s) {
    check(k8s_window_pool(P<float>(kpool), P<float>(vpool), P(kcache), P(vcache), P<int>(bt), max_blocks,
                          P<int>(tok_seq), P<int>(positions), T, G, D, V, P_, bs, f32, S(s)), "window_pool");
  });
  m.def("window_tile_rows", [](int H, int G, int D, int V) { return k8s_window_tile_rows(H, G, D, V); });
  m.def("window_attention", [](uintptr_t out, uintptr_t pacc, uintptr_t pml, uintptr_t q, long ldq, uintptr_t gate,
                               long ldg, uintptr_t kcache, uintptr_t vcache, uintptr_t kpool, uintptr_t vpool,
                               uintptr_t bt, int max_blocks, uintptr_t tok_seq, uintptr_t positions, int T, int H, int G,
                               int D, int V, int window, int P_, float scale, int sink, int bs, int nsplit, int chunk,
                               float softcap, uintptr_t sinkv, int gate_ph, int f32, int64_t s) {
    check(k8s_window_attention(P(out), P<float>(pacc), P<float>(pml), P(q), ldq, P(gate), ldg, P(kcache), P(vcache),
                               P<float>(kpool), P<float>(vpool), P<int>(bt), max_blocks, P<int>(tok_seq),
                               P<int>(positions), T, H, G, D, V, window, P_, scale, sink, bs, nsplit, chunk, softcap,
                               P<float>(sinkv), gate_ph, f32, S(s)),
          "window_attention");
  });
  m.def("window_mfma_ok", [](int H, int G, int D, int V) { return k8s_window_mfma_ok(H, G, D, V) != 0; });
  m.def("window_attention_mfma", [](uintptr_t out, uintptr_t q, long ldq, uintptr_t gate, long ldg, uintptr_t kcache,
                                    uintptr_t vcache, uintptr_t kpool, uintptr_t vpool, uintptr_t bt, int max_blocks,
                                    uintptr_t cu_q, uintptr_t positions, int nseq, int max_qlen, int H, int G, int D,
                                    int V, int window, int P_, float scale, int sink, int bs, int chunk, float softcap,
                                    uintptr_t sinkv, int gate_ph, int64_t s) {
    check(k8s_window_attention_mfma(P(out), P(q), ldq, P(gate), ldg, P(kcache), P(vcache), P<float>(kpool),
                                    P<float>(vpool), P<int>(bt), max_blocks, P<int>(cu_q), P<int>(positions), nseq,
                                    max_qlen, H, G, D, V, window, P_, scale, sink, bs, chunk, softcap, P<float>(sinkv),
                                    gate_ph, S(s)), "window_attention_mfma");
  });
  m.def("gated_scan_max_dim", []() { return k8s_gated_scan_max_dim(); });
  m.def("gated_scan_record", [](int kind, int D, int V) { return k8s_gated_scan_record(kind, D, V); });
  m.def("gated_scan", [](uintptr_t out, uintptr_t proj, long ld, int kind, int cq, int ck, int cv, int ci, int cf,
                         int cg, uintptr_t fbias, uintptr_t ibias, uintptr_t lower, uintptr_t normw, uintptr_t state,
                         uintptr_t cu_q, uintptr_t seq_slots, uintptr_t positions, int nseq, int H, int D, int V,
                         float eps, float cap, int f32, int T, int Lc, uintptr_t ws, uintptr_t aux, long ldaux,
                         uintptr_t hpar, int R, int64_t s) {
    check(k8s_gated_scan(P(out), P<float>(proj), ld, kind, cq, ck, cv, ci, cf, cg, P(fbias), P(ibias), P(lower),
                         P(normw), P<float>(state), P<int>(cu_q), P<int>(seq_slots), P<int>(positions), nseq, H, D, V,
                         eps, cap, f32, T, Lc, P<float>(ws), P<float>(aux), ldaux, P<float>(hpar), R, S(s)),
          "gated_scan");
  });
  m.def("gated_scan_workspace", [](int T, int nseq, int H, int D, int V, int Lc) {
    return k8s_gated_scan_workspace(T, nseq, H, D, V, Lc);
  });
  m.def("moe_align", [](uintptr_t sorted_tok, uintptr_t pos, uintptr_t seg, uintptr_t tiles, int ntiles,
                        uintptr_t topk_idx, int P_, int top, int E, int BM, int64_t s) {
    check(k8s_moe_align(P<int>(sorted_tok), P<int>(pos), P<int>(seg), P<int>(tiles), ntiles, P<int>(topk_idx), P_, top,
                        E, BM, S(s)), "moe_align");
  });
  m.def("moe_combine", [](uintptr_t z, uintptr_t D, uintptr_t pos, uintptr_t w, uintptr_t shared, uintptr_t logits,
                          int ld, int sg_col, int T, int W, int top, int f32, int64_t s) {
    check(k8s_moe_combine(P(z), P(D), P<int>(pos), P<float>(w), P(shared), P<float>(logits), ld, sg_col, T, W, top,
                          f32, S(s)), "moe_combine");
  });

#ifndef K8S_LEAN
  m.def("mgemm_configs", []() {
    py::list out;
    for (int c = 0; c < k8s_mgemm_num_configs(); ++c) {
      int bm = 0, bn = 0, th = 0, lds = 0, sw = 0, rb = 0;
      k8s_mgemm_config(c, &bm, &bn, &th, &lds, &sw, &rb);
      out.append(py::make_tuple(bm, bn, th, lds, sw != 0, rb));
    }
    return out;
  });
  m.def("mgemm_lds_bytes", [](int cfg, int mode) { return k8s_mgemm_lds_bytes(cfg, mode); });
  m.def("mgemm_plan_info", [](int M, int N, int K, int epi, int fp8, int cfg, int nwg) {
    long long tiles = 0, ws = 0;
    int cmax = 0;
    if (k8s_mgemm_plan_info(M, N, K, epi, fp8, cfg, nwg, &tiles, &cmax, &ws) != 0)
      throw std::invalid_argument("mgemm_plan_info: invalid plan");
    return py::make_tuple(tiles, cmax, ws);
  });
  m.def("mgemm", [](uintptr_t out, uintptr_t ws, uintptr_t tickets, uintptr_t x, uintptr_t W, uintptr_t xs,
                    uintptr_t wsc, int M, int N, int K, int epi, int fp8, int cfg, int nwg, int cmax, uintptr_t res,
                    int rms, float eps, int64_t s, uintptr_t oq, uintptr_t oe, int fenced) {
    check(k8s_mgemm(P(out), P<float>(ws), P<unsigned>(tickets), P(x), P(W), P<float>(xs), P<float>(wsc), M, N, K,
                    epi, fp8, cfg, nwg, cmax, P(res), rms, eps, P(oq), P(oe), fenced, S(s)),
          "mgemm");
  }, py::arg("out"), py::arg("ws"), py::arg("tickets"), py::arg("x"), py::arg("W"), py::arg("xs"), py::arg("wsc"),
     py::arg("M"), py::arg("N"), py::arg("K"), py::arg("epi"), py::arg("fp8"), py::arg("cfg"), py::arg("nwg"),
     py::arg("cmax"), py::arg("res"), py::arg("rms"), py::arg("eps"), py::arg("s"), py::arg("oq") = 0,
     py::arg("oe") = 0, py::arg("fenced") = 0);

  m.def("pgemm4_configs", []() {
    py::list out;
    for (int c = 0; c < k8s_pgemm4_num_configs(); ++c) {
      int bp = 0, bq = 0, lds = 0;
      k8s_pgemm4_config(c, &bp, &bq, &lds);
      out.append(py::make_tuple(bp, bq, lds));
    }
    return out;
  });
  m.def("pgemm4_plan", [](int M, int N, int K, int epi, int cfg, int splits) {
    int nwg = 0;
    long long slab = 0;
    if (k8s_pgemm4_plan(M, N, K, epi, cfg, splits, &nwg, &slab) != 0)
      throw std::invalid_argument("pgemm4_plan: invalid plan");
    return py::make_tuple(nwg, slab);
  });
  m.def("pgemm4", [](uintptr_t out, uintptr_t slab, uintptr_t x, uintptr_t W, int M, int N, int K, int epi, int cfg,
                     int splits, int group_m, uintptr_t res, int rms, float eps, int64_t s) {
    check(k8s_pgemm4(P(out), P<float>(slab), P(x), P(W), M, N, K, epi, cfg, splits, group_m, P(res), rms, eps, S(s)),
          "pgemm4");
  });
  m.def("pgemm_configs", []() {
    py::list out;
    for (int c = 0; c < k8s_pgemm_num_configs(); ++c) {
      int bp = 0, bq = 0, lds = 0;
      k8s_pgemm_config(c, &bp, &bq, &lds);
      out.append(py::make_tuple(bp, bq, lds));
    }
    return out;
  });
  m.def("pgemm_plan", [](int M, int N, int K, int epi, int fp8, int cfg, int splits) {
    int nwg = 0, tickets = 0;
    long long ws = 0;
    if (k8s_pgemm_plan(M, N, K, epi, fp8, cfg, splits, &nwg, &ws, &tickets) != 0)
      throw std::invalid_argument("pgemm_plan: invalid plan");
    return py::make_tuple(nwg, ws, tickets);
  });
  m.def("pgemm", [](uintptr_t out, uintptr_t ws, uintptr_t tickets, uintptr_t x, uintptr_t W, uintptr_t xs,
                    uintptr_t wsc, int M, int N, int K, int epi, int fp8, int cfg, int splits, int group_m,
                    uintptr_t res, int rms, float eps, int64_t s, uintptr_t oq, uintptr_t oe) {
    check(k8s_pgemm(P(out), P<float>(ws), P<unsigned>(tickets), P(x), P(W), P<float>(xs), P<float>(wsc), M, N, K,
                    epi, fp8, cfg, splits, group_m, P(res), rms, eps, P(oq), P(oe), S(s)),
          "pgemm");
  }, py::arg("out"), py::arg("ws"), py::arg("tickets"), py::arg("x"), py::arg("W"), py::arg("xs"), py::arg("wsc"),
     py::arg("M"), py::arg("N"), py::arg("K"), py::arg("epi"), py::arg("fp8"), py::arg("cfg"), py::arg("splits"),
     py::arg("group_m"), py::arg("res"), py::arg("rms"), py::arg("eps"), py::arg("s"), py::arg("oq") = 0,
     py::arg("oe") = 0);

  using k8sllm::RcclComm;
  py::class_<RcclComm>(m, "RcclComm")
      .def_static("unique_id", []() {
        auto v = RcclComm::unique_id();
        return py::bytes(reinterpret_cast<const char*>(v.data()), v.size());
      })
      .def(py::init([](int world, int rank, py::bytes id) {
             std::string s = id;
             return new RcclComm(world, rank, std::vector<uint8_t>(s.begin(), s.end()));
           }))
      .def("all_reduce", [](RcclComm& c, uintptr_t send, uintptr_t recv, size_t count, int dtype, int red,
                            int64_t s) { c.all_reduce(P(send), P(recv), count, dtype, red, S(s)); })
      .def("all_gather", [](RcclComm& c, uintptr_t send, uintptr_t recv, size_t count, int dtype, int64_t s) {
        c.all_gather(P(send), P(recv), count, dtype, S(s));
      })
      .def("reduce_scatter", [](RcclComm& c, uintptr_t send, uintptr_t recv, size_t count, int dtype, int red,
                                int64_t s) { c.reduce_scatter(P(send), P(recv), count, dtype, red, S(s)); })
      .def("broadcast", [](RcclComm& c, uintptr_t buf, size_t count, int dtype, int root, int64_t s) {
        c.broadcast(P(buf), count, dtype, root, S(s));
      })
      .def("async_error", &RcclComm::async_error)
      .def("abort", &RcclComm::abort, py::call_guard<py::gil_scoped_release>())
      .def_property_readonly("aborted", &RcclComm::aborted)
      .def_property_readonly("world", &RcclComm::world)
      .def_property_readonly("rank", &RcclComm::rank);

  using k8sllm::XgmiComm;
  py::class_<XgmiComm>(m, "XgmiComm")
      .def(py::init<int, int, long long, int, double>(), py::arg("world"), py::arg("rank"), py::arg("slot_bytes"),
           py::arg("blocks") = 16, py::arg("timeout_s") = 30.0)
      .def("handle", [](const XgmiComm& c) { return py::bytes(c.handle()); })
      .def("open", [](XgmiComm& c, const std::vector<py::bytes>& hs) {
        std::vector<std::string> v;
        for (const auto& h : hs) v.emplace_back(h);
        c.open(v);
      })
      .def(
          "all_reduce_bf16",
          [](XgmiComm& c, uintptr_t in, uintptr_t out, long long bytes, int64_t s, uintptr_t residual) {
            c.all_reduce_bf16(P(in), P(out), bytes, S(s), P(residual));
          },
          py::arg("inp"), py::arg("out"), py::arg("bytes"), py::arg("stream") = -1, py::arg("residual") = 0)
      .def("all_gather", [](XgmiComm& c, uintptr_t in, uintptr_t out, long long bytes, int64_t s) {
        c.all_gather(P(in), P(out), bytes, S(s));
      })
      .def(
          "gemv_allreduce",
          [](XgmiComm& c, uintptr_t out, uintptr_t x, uintptr_t w, uintptr_t wscale, int M, int N, int K,
             uintptr_t residual, int64_t s) {
            return c.gemv_allreduce(P(out), P(x), P(w), reinterpret_cast<const float*>(wscale), M, N, K, P(residual),
                                    S(s));
          },
          py::arg("out"), py::arg("x"), py::arg("w"), py::arg("wscale"), py::arg("M"), py::arg("N"), py::arg("K"),
          py::arg("residual") = 0, py::arg("stream") = -1)
      .def("error", &XgmiComm::error)
      .def("snapshot_error", [](XgmiComm& c, int64_t s) { c.snapshot_error(S(s)); }, py::arg("stream") = -1)
      .def("last_error", &XgmiComm::last_error)
      .def("reset_error", &XgmiComm::reset_error)
      .def("reset", &XgmiComm::reset, py::call_guard<py::gil_scoped_release>())
      .def_property_readonly("world", &XgmiComm::world)
      .def_property_readonly("rank", &XgmiComm::rank)
      .def_property_readonly("slot_bytes", &XgmiComm::slot_bytes)
      .def_property_readonly("blocks", &XgmiComm::blocks)
      .def_property_readonly("is_open", &XgmiComm::is_open)
      .def_property("ll_max_bytes", &XgmiComm::ll_max_bytes, &XgmiComm::set_ll_max_bytes)
      .def_property("twoshot_min_bytes", &XgmiComm::twoshot_min_bytes, &XgmiComm::set_twoshot_min_bytes)
      .def_property_readonly("max_allreduce_bytes", &XgmiComm::max_allreduce_bytes);

#endif
  using k8sllm::BlockAllocator;
  py::class_<BlockAllocator::Allocation>(m, "Allocation")
      .def_readonly("blocks", &BlockAllocator::Allocation::blocks)
      .def_readonly("cached_tokens", &BlockAllocator::Allocation::cached_tokens)
      .def_readonly("copy_src", &BlockAllocator::Allocation::copy_src)
      .def_readonly("copy_tokens", &BlockAllocator::Allocation::copy_tokens);
  py::class_<BlockAllocator>(m, "BlockAllocator")
      .def(py::init<int, int, bool>(), py::arg("num_blocks"), py::arg("block_size"), py::arg("prefix_caching") = true)
      .def("allocate", &BlockAllocator::allocate)
      .def("can_allocate", &BlockAllocator::can_allocate)
      .def("commit_prefix", &BlockAllocator::commit_prefix)
      .def("release", &BlockAllocator::release)
      .def("reset_prefix_cache", &BlockAllocator::reset_prefix_cache)
      .def_property_readonly("num_blocks", &BlockAllocator::num_blocks)
      .def_property_readonly("block_size", &BlockAllocator::block_size)
      .def_property_readonly("num_free", &BlockAllocator::num_free)
      .def_property_readonly("num_cached", &BlockAllocator::num_cached)
      .def_property_readonly("hits", &BlockAllocator::hits)
      .def_property_readonly("queries", &BlockAllocator::queries)
      .def("refcount", &BlockAllocator::refcount);
}
