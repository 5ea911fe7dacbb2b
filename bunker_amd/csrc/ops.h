// Internal launcher declarations: one per kernel family.  All pointers are
// device pointers; every launcher validates its shapes on the host before it
// launches and enqueues on bk::stream().
#pragma once
#include "common.h"

namespace bk {

enum : int { DT_F32 = 0, DT_BF16 = 1 };

// runtime.hip
bool inited();
bool capturing();        // between bk_capture_begin and bk_capture_end: nothing may allocate, free, copy or wait
int current_device();
bool prof_on();
int prof_begin(int kernel);
int prof_end();

// quant.hip
int launch_quantize_q8_1(const void* x, int x_dtype, void* out, int K, int batch);
int launch_dequant_legacy_i8(const void* blocks, void* out, int64_t nblocks);
int launch_q4k_nibbles(const void* blocks, void* out, int64_t nblocks);
int launch_q4k_dequant_f32(const void* blocks, void* out, int64_t nblocks);

// gdn_chunk.hip: the chunked form of the recurrence (f32 matrix instruction), between gdn_prefill's preparation and output norm
size_t gdn_chunk_workspace_bytes(int Hg, int T);
int launch_gdn_chunked_core(const void* conv_out, const float* A_log, const void* dt_bias, const float* a_p, const float* qk, const float* gates,
                            const float* S_in, float* S_out, float* o_raw, void* workspace, size_t workspace_bytes, int Hg, int T);
// gdn_prefill.hip
size_t gdn_prefill_workspace_bytes(int Hg, int T, bool chunked = false);
int launch_gdn_prefill(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                       const float* b_p, const float* norm_w, const float* S_in, void* out, float* S_out, void* workspace,
                       size_t workspace_bytes, int Hg, int T, bool chunked = false);

// quant_q4k.hip
int launch_quantize_q4k(const void* w, int w_dtype, void* out, int64_t rows, int K);

int launch_memread(const void* src, int64_t bytes, void* sink);
int launch_memcopy(const void* src, void* dst, int64_t bytes);

// gemv.hip
extern int g_tune_steps;
int gemv_grid_for(int wgs);
extern int g_tune_rpi, g_tune_cap, g_tune_mr_unroll, g_tune_mr_cap, g_tune_mr_nt, g_tune_gemv_impl;
int launch_gemv_q4k_f32(const void* W, const float* x, float* y, int N, int K);
int launch_gemv_q4k_q8_1(const void* W, const void* xq, void* y, int N, int K, int batch,
                         int out_dtype, const void* residual);
int launch_q4k_q8_1_subdots(const void* W, const void* xq, int32_t* I, int N, int K);

// gemv_fused.hip   pro: 0 = x is Q8_1, 1 = x is bf16 (quantized in the kernel), 2 = rmsnorm(x, norm_w) then quantized
extern int g_tune_fused_cap;
bool gemv_fused_fast_path(int K, int batch, bool swiglu);
struct FusedConv { const void* st; void* st_new; const void* w; };   // epi 3 of matrix 0: conv1d_decode's state, new state, taps
int launch_gemv_fused(int pro, const void* x, const void* norm_w, int K, int batch, int ngroups, const void* const* W,
                      void* const* out, const void* const* res, const int* N, const int* epi, bool swiglu,
                      const FusedConv* conv = nullptr);

// gemm_mfma.hip
extern int g_tune_small_rows;
extern int g_tune_gemm_nw, g_tune_gemm_r16, g_tune_gdn_nt, g_tune_attn_nt, g_tune_attn_bal;
int launch_gemm_group_mfma(const void* xq, int K, int batch, int ngroups, const void* const* W, void* const* out,
                           const void* const* res, const int* N, const int* epi);
int launch_gemm_swiglu_mfma(const void* xq, int K, int batch, const void* Wg, const void* Wu, int N, void* act, void* act_q8);
int launch_gemm_q4k_q8_1_mfma(const void* W, const void* xq, void* y, int N, int K, int batch, int out_dtype,
                              const void* residual);

// glue.hip
enum : int { EW_CAST_OP = 0, EW_ADD_OP = 1, EW_SWIGLU_OP = 2 };
int launch_embed(const void* E, const int32_t* ids_dev, int32_t id_scalar, void* out, int H, int vocab, int batch);
int launch_rmsnorm(const void* x, const void* w, void* out, void* xq, int N, int rows);
int launch_rmsnorm_small_rows(const void* x, const void* w, void* xq, int N, int rows, const void* Wa, const void* Wb, float* out_a,
                              float* out_b, int na, int nb_rows);
int launch_elementwise(int op, const void* a, const void* b, void* out, int64_t n);
int launch_swiglu_q8_1(const float* g, const float* u, void* out, void* out_q8, int64_t n);
int launch_conv1d_decode(const void* x, const void* st, const void* w, void* out, void* st_new, int C, int batch);
int launch_conv1d_prefill(const void* x, const void* st, const void* w, void* out, void* st_new, int C, int T);
int launch_headnorm(const void* x, const void* w, void* out, int nheads, int HD, int in_stride, int64_t in_bstride,
                    int batch, const float* cos_t, const float* sin_t, const int32_t* pos_dev, int pos_scalar, int half,
                    int max_len);
int launch_rope(void* x, const float* cos_t, const float* sin_t, const int32_t* pos_dev, int pos_scalar, int nheads,
                int HD, int half, int max_len, int batch);
size_t argmax_workspace_bytes(int n, int batch);
int launch_argmax(const float* logits, float* val, int32_t* idx, void* workspace, int n, int batch);

int launch_argmax_feed(const float* logits, float* val, int32_t* idx, void* workspace, int n, int batch, int32_t* ids, int32_t* pos,
                       int32_t* hist, int32_t* counter, int max_steps, int max_pos, const void* E, void* x, int H);
int launch_advance(const int32_t* idx, const float* val, int32_t* ids, int32_t* pos, int32_t* hist, int32_t* counter, int batch,
                   int max_steps, int max_pos);

// gdn.hip
extern int g_tune_gdn_cs;
int launch_gdn_fused(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                     const float* b_p, const float* norm_w, const float* S_in, void* out, float* S_out, int Hg, int batch);
int launch_gdn_conv_fused(const void* qkv, const void* conv_st, const void* conv_w, const void* z, const float* A_log,
                          const void* dt_bias, const float* a_p, const float* b_p, const float* norm_w, const float* S_in,
                          void* out, void* conv_st_new, float* S_out, void* out_q8, int Hg, int batch);
int launch_gdn_core(const void* q, const void* k, const void* v, const float* g, const float* beta, const float* S_in,
                    void* out, float* S_out, int Hg, int batch);
// column-slab form without the gated norm: raw = per sequence f32 o[Hg*128] | f32 z*sigmoid(z)[Hg*128] | f64 sum o^2 [Hg][4]
size_t gdn_raw_bytes(int Hg, int batch);
int launch_gdn_slabs(const void* conv_out, const void* z, const float* A_log, const void* dt_bias, const float* a_p,
                     const float* b_p, const float* S_in, void* raw, float* S_out, int Hg, int batch);

// attn.hip
// what launch_attn_decode needs to fold the step's preparation (head norms, rotation, cache append) into the
// double-precision attention kernel: the inputs of launch_attn_prep
struct AttnPrepFuse {
  const void *qg, *k, *v, *qw, *kw;
  const float *cos_t, *sin_t;
  int half, max_len;
};
size_t attn_workspace_bytes(int batch, int NKV, int max_splits);
int attn_choose_splits(int batch, int NKV, int max_ctx);
int launch_attn_decode(const void* q, const void* kc, const void* vc, const int32_t* block_table, int bt_stride,
                       const int32_t* ctx_len, int ctx_scalar, int ctx_add, int max_ctx, const void* gate, int64_t gate_bstride,
                       int64_t gate_hstride, void* out, float* lse, void* workspace, size_t workspace_bytes, int batch,
                       int NH, int NKV, int HD, int page_size, int splits, void* out_q8 = nullptr, int tpw = 1, int exact = 0,
                       const uint32_t* qf_ready = nullptr, const AttnPrepFuse* prep = nullptr);
// attn_prefill.hip: causal attention of T prompt tokens, query tile x K/V tile on the bf16 matrix cores
bool attn_prefill_tiled_serves(int NH, int NKV, int max_ctx);
extern int g_tune_prefill_ksplit, g_tune_prefill_xmap;
size_t attn_prefill_workspace_bytes(int T, int NH, int NKV, int max_ctx);     // partial rows of a launch cut along K/V
int launch_attn_prefill_tiled(const void* q, const void* kc, const void* vc, const int32_t* block_table, const int32_t* pos, int max_ctx,
                              const void* gate, int64_t gate_bstride, int64_t gate_hstride, void* out, int T, int NH, int NKV, int HD,
                              int page_size, void* workspace = nullptr, size_t workspace_bytes = 0);
// attn_exact.hip: the double-precision form (workspace: f64 partials, plan, f64 copy of q)
size_t attn_exact_qf_bytes(int rows, int NKV);
size_t attn_exact_workspace_bytes(int rows, int NKV, int max_splits);
int attn_noalloc_setup(int device);
void attn_noalloc_teardown(int device);
int launch_attn_decode_noalloc(int device, const void* q, const void* kc, const void* vc, const int32_t* block_table, int bt_stride,
                               const int32_t* ctx_len, int max_ctx, const void* gate, int64_t gate_bstride, int64_t gate_hstride,
                               void* out, float* lse, int batch, int NH, int NKV, int HD, int page_size, int splits);
int launch_attn_prep(const void* qg, const void* k, const void* v, const void* qw, const void* kw, const float* cos_t,
                     const float* sin_t, const int32_t* pos_dev, int pos_scalar, int half, int max_len, void* qout, void* kc,
                     void* vc, const int32_t* block_table, int bt_stride, int batch, int NH, int NKV, int HD, int page_size,
                     uint32_t* qf = nullptr);
int launch_kv_append(const void* k, const void* v, void* kc, void* vc, const int32_t* block_table, int bt_stride,
                     const int32_t* pos_dev, int pos_scalar, int max_len, int batch, int NKV, int HD, int page_size);

}  // namespace bk
