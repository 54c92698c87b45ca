// Flat C ABI over the device operators, contexts, programs and launch queues.
#include "../../include/torch_col_hip.h"

#include "context.h"
#include <vector>

#include "ops.h"

#include <stdio.h>

using namespace tch;

struct tch_context {
  Context ctx;
  explicit tch_context(hipStream_t s) : ctx(s) {}
};
struct tch_program {
  Program prog;
};

namespace {
inline Context* C(tch_context* c) { return c ? &c->ctx : nullptr; }
inline ConvShape shape(int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad, int c_logical = 0) {
  ConvShape s{N, H, W, Cc, K, R, S, stride, pad, c_logical};
  return s;
}
}  // namespace

extern "C" {

const char* tch_last_error(void) { return last_error(); }
int tch_has_device_code(void) { return 1; }

int tch_context_create(void* hip_stream, tch_context** out) {
  if (!out) {
    set_error("tch_context_create: null output");
    return -22;
  }
  auto* c = new tch_context(static_cast<hipStream_t>(hip_stream));
  c->ctx.queue = queue_for_stream(reinterpret_cast<uint64_t>(hip_stream));
  *out = c;
  return 0;
}

void tch_context_destroy(tch_context* ctx) { delete ctx; }

uint64_t tch_context_take_rejected(tch_context* ctx) { return ctx ? ctx->ctx.rejected.exchange(0) : 0; }

int tch_context_set_lane(tch_context* ctx, int lane, int wait_main) {
  if (!ctx || (lane != 0 && lane != 1)) {
    set_error("tch_context_set_lane: lane must be 0 or 1");
    return -22;
  }
  ctx->ctx.lane = lane;
  ctx->ctx.wait_main = lane == 1 && wait_main != 0;
  return 0;
}

int tch_context_join(tch_context* ctx) {
  if (!ctx) {
    set_error("tch_context_join: null context");
    return -22;
  }
  return ctx->ctx.record_join();
}

int tch_context_join_behind(tch_context* ctx) {
  if (!ctx) {
    set_error("tch_context_join_behind: null context");
    return -22;
  }
  return ctx->ctx.record_join(true);
}

int tch_context_synchronize(tch_context* ctx) {
  if (!ctx) {
    set_error("tch_context_synchronize: null context");
    return -22;
  }
  return ctx->ctx.synchronize();
}

int tch_program_create(tch_program** out) {
  if (!out) {
    set_error("tch_program_create: null output");
    return -22;
  }
  *out = new tch_program();
  return 0;
}

void tch_program_destroy(tch_program* prog) { delete prog; }

int64_t tch_program_size(const tch_program* prog) { return prog ? static_cast<int64_t>(prog->prog.launches.size()) : 0; }

int tch_program_begin_record(tch_context* ctx, tch_program* prog) {
  if (!ctx || !prog) {
    set_error("tch_program_begin_record: null argument");
    return -22;
  }
  if (ctx->ctx.recording) {
    set_error("tch_program_begin_record: context is already recording");
    return -16;
  }
  ctx->ctx.recording = &prog->prog;
  return 0;
}

int tch_program_end_record(tch_context* ctx) {
  if (!ctx || !ctx->ctx.recording) {
    set_error("tch_program_end_record: context is not recording");
    return -22;
  }
  ctx->ctx.recording = nullptr;
  ctx->ctx.lane = 0;
  ctx->ctx.wait_main = false;
  return 0;
}

int tch_program_run(tch_context* ctx, const tch_program* prog, int64_t first, int64_t last) {
  if (!ctx || !prog) {
    set_error("tch_program_run: null argument");
    return -22;
  }
  if (ctx->ctx.recording) {
    set_error("tch_program_run: context is recording");
    return -16;
  }
  const int64_t n = static_cast<int64_t>(prog->prog.launches.size());
  if (last < 0 || last > n) last = n;
  if (first < 0 || first > last) {
    set_error("tch_program_run: bad range");
    return -22;
  }
  // the stream may have been registered after the context was made
  ctx->ctx.queue = queue_for_stream(reinterpret_cast<uint64_t>(ctx->ctx.stream));
  const uint64_t before = ctx->ctx.rejected.load();
  ctx->ctx.note_foreign_work();   // the caller may have given the stream work of its own since the last run
  // with a compute-unit limit the launches go to another stream than the caller's: order them behind
  // what the caller's stream holds, and what the caller does next behind them
  const bool limited = ctx->ctx.cu_limit > 0 && first < last;
  if (limited)
    if (int rc = ctx->ctx.depend(ctx->ctx.stream, ctx->ctx.main_stream())) return rc;
  for (int64_t i = first; i < last; ++i) {
    const auto& launches = prog->prog.launches;
    int rc = ctx->ctx.dispatch(launches[static_cast<size_t>(i)], i + 1 < last ? &launches[static_cast<size_t>(i + 1)] : nullptr);
    if (rc) return rc;
  }
  if (limited)
    if (int rc = ctx->ctx.depend(ctx->ctx.main_stream(), ctx->ctx.stream)) return rc;
  return ctx->ctx.rejected.load() != before ? 1 : 0;
}

int tch_cu_partition_init(int total_cus, int min_train_cus, int max_train_cus) {
  return cu_partition_init(total_cus, min_train_cus, max_train_cus);
}
int tch_cu_partition_total(void) { return cu_partition_total(); }
int tch_cu_partition_train_avail(int infer_required_cus) { return cu_partition_train_avail(infer_required_cus); }
int tch_context_set_cu_limit(tch_context* ctx, int n_cus) {
  if (!ctx) {
    set_error("tch_context_set_cu_limit: null context");
    return -22;
  }
  if (ctx->ctx.recording) {
    set_error("tch_context_set_cu_limit: context is recording");
    return -16;
  }
  ctx->ctx.queue = queue_for_stream(reinterpret_cast<uint64_t>(ctx->ctx.stream));
  return ctx->ctx.set_cu_limit(n_cus);
}
int tch_context_get_cu_limit(tch_context* ctx) { return ctx ? ctx->ctx.cu_limit : -22; }

uint64_t tch_RegisterStream(uint64_t hip_stream) { return register_stream(hip_stream); }
int tch_UnRegisterStream(uint64_t hip_stream) { return unregister_stream(hip_stream); }
void tch_UnRegisterAllStreams(void) { unregister_all_streams(); }
size_t tch_GetXQueueSize(uint64_t hip_stream) { return queue_size(hip_stream); }
size_t tch_GetXQueueSizeAllStreams(void) { return queue_size_all_streams(); }
size_t tch_GetTotalXQueueSize(void) { return queue_size_all_streams(); }
size_t tch_AbortStream(uint64_t hip_stream) { return abort_stream(hip_stream); }
size_t tch_AbortAllStreams(void) { return abort_all_streams(); }
int tch_SyncStream(uint64_t hip_stream) { return sync_stream(hip_stream); }
int tch_SyncAllStreams(void) { return sync_all_streams(); }
int tch_QueryRejectCudaCalls(void) { return query_reject_calls() ? 1 : 0; }
void tch_SetRejectCudaCalls(int reject) { set_reject_calls(reject != 0); }
void tch_SuspendAllStreams(int sync_hw) { suspend_all_streams(sync_hw != 0); }
void tch_ResumeAllStreams(int drop_commands) { resume_all_streams(drop_commands != 0); }
void tch_SetXQueueShape(int queue_length, int sync_interval) { set_queue_shape(queue_length, sync_interval); }
size_t tch_GetXQueueInFlight(uint64_t hip_stream) {
  auto q = queue_for_stream(hip_stream);
  return q ? q->in_flight() : 0;
}

int tch_conv2d_fwd(tch_context* ctx, int dtype, const void* x, const void* w, void* y, const void* add,
                   const void* mask, const float* bias, int out_f32, int N, int H, int W, int Cc, int K, int R, int S,
                   int stride, int pad, int tile_cfg, int c_logical) {
  return conv2d_fwd(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, w, y, add, mask, bias, out_f32,
                    tile_cfg);
}

int tch_conv2d_fwd_affine(tch_context* ctx, int dtype, const void* x, const void* w, void* y, const float* scale,
                          const float* shift, const void* residual, int relu, int N, int H, int W, int Cc, int K, int R,
                          int S, int stride, int pad, int tile_cfg, int c_logical) {
  return conv2d_fwd(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, w, y, residual, nullptr, shift, 0,
                    tile_cfg, nullptr, nullptr, scale, relu);
}

int tch_conv2d_fwd_bnstats(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W,
                           int Cc, int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical,
                           float* bn_partial) {
  if (!bn_partial) {
    set_error("tch_conv2d_fwd_bnstats: null statistics buffer");
    return -22;
  }
  return conv2d_fwd(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, w, y, nullptr, nullptr, nullptr,
                    0, tile_cfg, bn_partial);
}

int tch_conv2d_fwd_stat_rows(int dtype, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                             int tile_cfg) {
  return conv2d_fwd_stat_rows(shape(N, H, W, Cc, K, R, S, stride, pad), dtype, tile_cfg);
}

int tch_bn_fwd_train_partials(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                              int64_t rows, int Cc, const float* gamma, const float* beta, float* running_mean,
                              float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                              const float* partial, int row_blocks, float* scratch) {
  return bn_fwd_train_partials(C(ctx), dtype, x, y, residual, relu, rows, Cc, gamma, beta, running_mean, running_var,
                               save_mean, save_invstd, momentum, eps, partial, row_blocks, scratch);
}

int tch_conv2d_dgrad(tch_context* ctx, int dtype, const void* dy, const void* w, void* dx, const void* add,
                     const void* mask, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                     int tile_cfg, int c_logical, int add_stride) {
  return conv2d_dgrad(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), dy, w, dx, add, mask, tile_cfg,
                      nullptr, add_stride);
}

int tch_conv2d_dgrad_bnsums(tch_context* ctx, int dtype, const void* dy, const void* w, void* dx, const void* add,
                            const void* mask, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                            int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                            const float* bn_invstd, float* bn_partial, int add_stride) {
  BnBwdSums bn{bn_mask, bn_x, bn_mean, bn_invstd, bn_partial, nullptr};
  return conv2d_dgrad(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), dy, w, dx, add, mask, tile_cfg,
                      &bn, add_stride);
}

int tch_conv2d_dgrad_stat_rows(int dtype, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                               int tile_cfg) {
  return conv2d_dgrad_stat_rows(shape(N, H, W, Cc, K, R, S, stride, pad), dtype, tile_cfg);
}

int tch_bn_bwd_partials(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int Cc,
                        const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma,
                        float* dbeta, int accumulate, const float* partial, int row_blocks, float* scratch) {
  return bn_bwd_partials(C(ctx), dtype, g, x, dx, rows, Cc, gamma, save_mean, save_invstd, dgamma, dbeta, accumulate,
                         partial, row_blocks, scratch);
}

int tch_conv2d_fwd_bnacc(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W,
                         int Cc, int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical,
                         int64_t* bn_acc, int acc_copies) {
  if (!bn_acc) {
    set_error("tch_conv2d_fwd_bnacc: null accumulator buffer");
    return -22;
  }
  return conv2d_fwd(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, w, y, nullptr, nullptr, nullptr,
                    0, tile_cfg, nullptr, nullptr, nullptr, 0, reinterpret_cast<long long*>(bn_acc), acc_copies);
}

int tch_conv2d_dgrad_bnacc(tch_context* ctx, int dtype, const void* dy, const void* w, void* dx, const void* add,
                           const void* mask, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                           int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                           const float* bn_invstd, int64_t* bn_acc, int acc_copies, int add_stride) {
  BnBwdSums bn{bn_mask, bn_x, bn_mean, bn_invstd, nullptr, nullptr, reinterpret_cast<long long*>(bn_acc), acc_copies};
  return conv2d_dgrad(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), dy, w, dx, add, mask, tile_cfg,
                      &bn, add_stride);
}

int tch_bn_fwd_train_acc(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                         int64_t rows, int Cc, const float* gamma, const float* beta, float* running_mean,
                         float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                         const int64_t* acc, int acc_copies) {
  return bn_fwd_train_acc(C(ctx), dtype, x, y, residual, relu, rows, Cc, gamma, beta, running_mean, running_var, save_mean,
                          save_invstd, momentum, eps, reinterpret_cast<const long long*>(acc), acc_copies);
}

int tch_bn_bwd_acc(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int Cc,
                   const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
                   int accumulate, const int64_t* acc, int acc_copies) {
  return bn_bwd_acc(C(ctx), dtype, g, x, dx, rows, Cc, gamma, save_mean, save_invstd, dgamma, dbeta, accumulate,
                    reinterpret_cast<const long long*>(acc), acc_copies);
}

int tch_layernorm_fwd(tch_context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta,
                      float* mean, float* rstd, int64_t rows, int Cc, float eps) {
  return layernorm_fwd(C(ctx), dtype, x, y, gamma, beta, mean, rstd, rows, Cc, eps);
}

int tch_layernorm_fwd_windowed(tch_context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta,
                               float* mean, float* rstd, int64_t rows, int Cc, float eps, int H, int W, int window,
                               int shift, int windowed_tensors, const void* add, void* sum_out) {
  LnWindow win{H, W, window, shift, windowed_tensors};
  return layernorm_fwd(C(ctx), dtype, x, y, gamma, beta, mean, rstd, rows, Cc, eps, &win, add, sum_out);
}

int tch_layernorm_bwd_windowed(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual,
                               const float* gamma, const float* mean, const float* rstd, float* dgamma, float* dbeta,
                               int accumulate, int64_t rows, int Cc, float* partial, int H, int W, int window, int shift,
                               int windowed_tensors) {
  LnWindow win{H, W, window, shift, windowed_tensors};
  return layernorm_bwd(C(ctx), dtype, dy, x, dx, residual, gamma, mean, rstd, dgamma, dbeta, accumulate, rows, Cc,
                       partial, &win);
}

int tch_layernorm_bwd_partial_rows(int64_t rows) { return layernorm_bwd_partial_rows(rows); }

int tch_layernorm_bwd(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual,
                      const float* gamma,
                      const float* mean, const float* rstd, float* dgamma, float* dbeta, int accumulate, int64_t rows,
                      int Cc, float* partial) {
  return layernorm_bwd(C(ctx), dtype, dy, x, dx, residual, gamma, mean, rstd, dgamma, dbeta, accumulate, rows, Cc,
                       partial);
}

int tch_gelu_fwd(tch_context* ctx, int dtype, const void* x, void* y, int64_t n, int tanh_form) {
  return gelu_fwd(C(ctx), dtype, x, y, n, tanh_form);
}

int tch_gelu_bwd(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, int64_t n, int tanh_form) {
  return gelu_bwd(C(ctx), dtype, dy, x, dx, n, tanh_form);
}

int tch_attn_softmax_fwd(tch_context* ctx, int dtype, const void* scores, void* probs, int64_t batch, int heads, int Lq,
                         int Lk, float scale, const float* bias, const float* mask, int windows, int causal) {
  return attn_softmax_fwd(C(ctx), dtype, scores, probs, batch, heads, Lq, Lk, scale, bias, mask, windows, causal);
}

int tch_attn_softmax_bwd(tch_context* ctx, int dtype, const void* probs, const void* dprobs, void* dscores, int64_t rows,
                         int Lq, int Lk, float scale, int causal) {
  return attn_softmax_bwd(C(ctx), dtype, probs, dprobs, dscores, rows, Lq, Lk, scale, causal);
}

int tch_adamw_step(tch_context* ctx, float* param, const float* grad, float* exp_avg, float* exp_avg_sq,
                   void* shadow_bf16, int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay,
                   int* step_dev, float* scalars_dev) {
  return adamw_step(C(ctx), param, grad, exp_avg, exp_avg_sq, shadow_bf16, n, lr, beta1, beta2, eps, weight_decay,
                    step_dev, scalars_dev);
}

int tch_embedding_fwd(tch_context* ctx, int dtype, const int64_t* ids, const void* wte, const void* wpe, void* out, int B,
                      int T, int Cc, int vocab) {
  return embedding_fwd(C(ctx), dtype, ids, wte, wpe, out, B, T, Cc, vocab);
}

int tch_embedding_bwd(tch_context* ctx, int dtype, const int64_t* ids, const void* dy, float* dwte, float* dwpe, int B,
                      int T, int Cc, int vocab, int accumulate_wpe, int32_t* chain) {
  return embedding_bwd(C(ctx), dtype, ids, dy, dwte, dwpe, B, T, Cc, vocab, accumulate_wpe, chain);
}

int tch_batched_gemm(tch_context* ctx, int dtype, const void* a, const void* b, void* c, int M, int N, int K,
                     int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t ldc, int batch_outer,
                     int batch_inner, int64_t a_bo, int64_t a_bi, int64_t b_bo, int64_t b_bi, int64_t c_bo, int64_t c_bi,
                     float alpha, int accumulate, int causal) {
  return batched_gemm(C(ctx), dtype, a, b, c, M, N, K, a_rs, a_cs, b_rs, b_cs, ldc, batch_outer, batch_inner, a_bo, a_bi,
                      b_bo, b_bi, c_bo, c_bi, alpha, accumulate, causal);
}

int tch_window_attn_fwd(tch_context* ctx, int dtype, const void* qkv, void* o, void* probs, const float* bias,
                        const float* mask, int windows, int heads, int N, int Cc, int nW, float scale) {
  return window_attn_fwd(C(ctx), dtype, qkv, o, probs, bias, mask, windows, heads, N, Cc, nW, scale);
}

int tch_window_attn_bwd(tch_context* ctx, int dtype, const void* qkv, const void* probs, const void* dout, void* dqkv,
                        void* ds, int windows, int heads, int N, int Cc, float scale) {
  return window_attn_bwd(C(ctx), dtype, qkv, probs, dout, dqkv, ds, windows, heads, N, Cc, scale);
}

int tch_relpos_bias_gather_pairs(tch_context* ctx, const float* table, const int32_t* index, float* bias, int heads,
                                 int pairs, int entries) {
  return relpos_bias_gather_pairs(C(ctx), table, index, bias, heads, pairs, entries);
}

int tch_relpos_bias_gather_batch(tch_context* ctx, const float* const* tables, const int32_t* const* indices,
                                 float* const* biases, const int* heads, int count, int pairs, int entries) {
  return relpos_bias_gather_batch(C(ctx), tables, indices, biases, heads, count, pairs, entries);
}

int tch_relpos_bias_scatter_pairs(tch_context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads,
                                  int pairs, int entries, int accumulate) {
  return relpos_bias_scatter_pairs(C(ctx), dbias, index, dtable, heads, pairs, entries, accumulate);
}

int tch_relpos_bias_scatter_csr(tch_context* ctx, const float* dbias, const int32_t* ptr, const int32_t* list,
                                float* dtable, int heads, int pairs, int entries, int accumulate) {
  return relpos_bias_scatter_csr(C(ctx), dbias, ptr, list, dtable, heads, pairs, entries, accumulate);
}

int tch_flash_attn_fwd(tch_context* ctx, int dtype, const void* q, const void* k, const void* v, void* o, float* lse,
                       int B, int H, int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale,
                       int causal) {
  return flash_attn_fwd(C(ctx), dtype, q, k, v, o, lse, B, H, T, qkv_rs, qkv_bs, o_rs, o_bs, scale, causal);
}

int tch_flash_attn_bwd(tch_context* ctx, int dtype, const void* q, const void* k, const void* v, const void* o,
                       const void* dout, const float* lse, float* delta, void* dq, void* dk, void* dv, int B, int H,
                       int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal) {
  return flash_attn_bwd(C(ctx), dtype, q, k, v, o, dout, lse, delta, dq, dk, dv, B, H, T, qkv_rs, qkv_bs, o_rs, o_bs,
                        scale, causal);
}

int tch_conv2d_fwd_bn(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W, int Cc,
                      int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical, float* bn_partial,
                      int* counters, const float* gamma, const float* beta, float* running_mean, float* running_var,
                      float* save_mean, float* save_invstd, float momentum, float eps, float* coef) {
  BnFinalize fin{counters, gamma, beta, running_mean, running_var, save_mean, save_invstd, coef, momentum, eps, 0};
  return conv2d_fwd(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, w, y, nullptr, nullptr, nullptr,
                    0, tile_cfg, bn_partial, &fin);
}

int tch_conv2d_dgrad_bn(tch_context* ctx, int dtype, const void* dy, const void* w, void* dx, const void* add,
                        const void* mask, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                        int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                        const float* bn_invstd, float* bn_partial, int* counters, const float* gamma, float* dgamma,
                        float* dbeta, int accumulate, float* coef, int add_stride) {
  BnFinalize fin{counters, gamma, nullptr, nullptr, nullptr, dgamma, dbeta, coef, 0.f, 0.f, accumulate};
  BnBwdSums bn{bn_mask, bn_x, bn_mean, bn_invstd, bn_partial, &fin};
  return conv2d_dgrad(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), dy, w, dx, add, mask, tile_cfg,
                      &bn, add_stride);
}

int tch_bn_apply_fwd(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows,
                     int Cc, const float* coef) {
  return bn_apply_fwd(C(ctx), dtype, x, y, residual, relu, rows, Cc, coef);
}

int tch_bn_eval_coef(tch_context* ctx, const float* gamma, const float* beta, const float* running_mean,
                     const float* running_var, float* coef, int Cc, float eps) {
  return bn_eval_coef(C(ctx), gamma, beta, running_mean, running_var, coef, Cc, eps);
}

int tch_bn_apply_bwd(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int Cc,
                     const float* coef) {
  return bn_apply_bwd(C(ctx), dtype, g, x, dx, rows, Cc, coef);
}

int tch_window_partition(tch_context* ctx, int dtype, const void* src, void* dst, const void* add, int B, int H, int W,
                         int Cc, int window, int shift, int reverse) {
  return window_partition(C(ctx), dtype, src, dst, add, B, H, W, Cc, window, shift, reverse);
}

int tch_patch_merge_gather(tch_context* ctx, int dtype, const void* src, void* dst, int B, int H, int W, int Cc,
                           int reverse) {
  return patch_merge_gather(C(ctx), dtype, src, dst, B, H, W, Cc, reverse);
}

int tch_relpos_bias_gather(tch_context* ctx, const float* table, const int32_t* index, float* bias, int heads,
                           int tokens, int entries) {
  return relpos_bias_gather(C(ctx), table, index, bias, heads, tokens, entries);
}

int tch_relpos_bias_scatter(tch_context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads,
                            int tokens, int entries, int accumulate) {
  return relpos_bias_scatter(C(ctx), dbias, index, dtable, heads, tokens, entries, accumulate);
}

int64_t tch_column_sum_workspace_floats(int rows, int cols) { return column_sum_workspace_floats(rows, cols); }

int tch_column_sum(tch_context* ctx, int dtype, const void* x, float* out, int rows, int cols, int accumulate,
                   float* workspace) {
  return column_sum(C(ctx), dtype, x, out, rows, cols, accumulate, workspace);
}

int tch_conv2d_wgrad_pick_splits(int dtype, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad) {
  return conv2d_wgrad_pick_splits(shape(N, H, W, Cc, K, R, S, stride, pad), dtype);
}

int64_t tch_conv2d_wgrad_workspace_bytes(int dtype, int K, int R, int S, int Cc, int splits) {
  return conv2d_wgrad_workspace_bytes(shape(1, 1, 1, Cc, K, R, S, 1, 0), dtype, splits);
}

int tch_conv2d_wgrad(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* workspace,
                     int splits, int accumulate, int N, int H, int W, int Cc, int K, int R, int S, int stride,
                     int pad, int tile_cfg, int c_logical) {
  ConvShape s = shape(N, H, W, Cc, K, R, S, stride, pad, c_logical);
  if (splits <= 0) splits = workspace ? conv2d_wgrad_pick_splits(s, dtype) : 1;
  return conv2d_wgrad(C(ctx), dtype, s, x, dy, dw, workspace, splits, accumulate, tile_cfg);
}

int tch_conv2d_wgrad_trailing(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* dbias,
                              float* workspace, int splits, int accumulate, int N, int H, int W, int Cc, int K, int R,
                              int S, int stride, int pad, int tile_cfg, int c_logical) {
  ConvShape s = shape(N, H, W, Cc, K, R, S, stride, pad, c_logical);
  if (splits <= 0) splits = workspace ? conv2d_wgrad_pick_splits(s, dtype) : 1;
  return conv2d_wgrad(C(ctx), dtype, s, x, dy, dw, workspace, splits, accumulate, tile_cfg, dbias, 1);
}

int tch_conv2d_wgrad_flush(tch_context* ctx) { return conv2d_wgrad_flush(C(ctx)); }

int tch_conv2d_wgrad_group_plan(int dtype, int n, const int* shapes, int target_wgs, int tile_cfg, int* splits,
                                int64_t* table_bytes, int64_t* workspace_bytes) {
  if (n <= 0 || !shapes || !splits) {
    set_error("tch_conv2d_wgrad_group_plan: empty group");
    return -22;
  }
  std::vector<ConvShape> v(static_cast<size_t>(n));
  for (int i = 0; i < n; ++i) {
    const int* q = shapes + 9 * i;
    v[static_cast<size_t>(i)] = shape(q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], q[8]);
  }
  return conv2d_wgrad_group_plan(dtype, n, v.data(), target_wgs, tile_cfg, splits, table_bytes, workspace_bytes);
}

int tch_conv2d_wgrad_group(tch_context* ctx, int dtype, int n, const int* shapes, const uint64_t* x, const uint64_t* dy,
                           const uint64_t* dw, const uint64_t* dbias, const int* splits, int tile_cfg, int accumulate,
                           float* workspace, void* table, int max_wgs) {
  if (n <= 0 || !shapes || !x || !dy || !dw || !splits) {
    set_error("tch_conv2d_wgrad_group: empty group or null array");
    return -22;
  }
  std::vector<WgradGroupItem> v(static_cast<size_t>(n));
  for (int i = 0; i < n; ++i) {
    const int* q = shapes + 9 * i;
    WgradGroupItem& it = v[static_cast<size_t>(i)];
    it.shape = shape(q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7], q[8]);
    it.x = reinterpret_cast<const void*>(x[i]);
    it.dy = reinterpret_cast<const void*>(dy[i]);
    it.dw = reinterpret_cast<float*>(dw[i]);
    it.dbias = dbias ? reinterpret_cast<float*>(dbias[i]) : nullptr;
    it.splits = splits[i];
  }
  return conv2d_wgrad_group(C(ctx), dtype, n, v.data(), tile_cfg, accumulate, workspace, table, max_wgs);
}

int64_t tch_conv2d_wgrad_static_capacity_bytes(void) { return conv2d_wgrad_static_capacity_bytes(); }

int tch_conv2d_wgrad_static(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, int splits,
                            int accumulate, int N, int H, int W, int Cc, int K, int R, int S, int stride, int pad,
                            int tile_cfg, int c_logical) {
  return conv2d_wgrad_static(C(ctx), dtype, shape(N, H, W, Cc, K, R, S, stride, pad, c_logical), x, dy, dw, splits,
                             accumulate, tile_cfg);
}

int tch_conv2d_wgrad_bias(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* dbias,
                          float* workspace, int splits, int accumulate, int N, int H, int W, int Cc, int K, int R, int S,
                          int stride, int pad, int tile_cfg, int c_logical) {
  ConvShape s = shape(N, H, W, Cc, K, R, S, stride, pad, c_logical);
  if (splits <= 0) splits = workspace ? conv2d_wgrad_pick_splits(s, dtype) : 1;
  return conv2d_wgrad(C(ctx), dtype, s, x, dy, dw, workspace, splits, accumulate, tile_cfg, dbias);
}

int64_t tch_bn_workspace_bytes(int dtype, int64_t rows, int Cc) { return bn_workspace_bytes(rows, Cc, dtype); }

int tch_bn_fwd_train(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                     int64_t rows, int Cc, const float* gamma, const float* beta, float* running_mean,
                     float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                     float* workspace) {
  return bn_fwd_train(C(ctx), dtype, x, y, residual, relu, rows, Cc, gamma, beta, running_mean, running_var,
                      save_mean, save_invstd, momentum, eps, workspace);
}

int tch_bn_bwd(tch_context* ctx, int dtype, const void* dy, const void* relu_mask, const void* x, void* dx,
               int64_t rows, int Cc, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dgamma, float* dbeta, int accumulate, float* workspace) {
  return bn_bwd(C(ctx), dtype, dy, relu_mask, x, dx, rows, Cc, gamma, save_mean, save_invstd, dgamma, dbeta,
                accumulate, workspace);
}

int tch_maxpool_fwd(tch_context* ctx, int dtype, const void* x, void* y, int32_t* index, int N, int H, int W, int Cc,
                    int ksize, int stride, int pad) {
  return maxpool_fwd(C(ctx), dtype, x, y, index, N, H, W, Cc, ksize, stride, pad);
}

int tch_maxpool_bwd(tch_context* ctx, int dtype, const void* dy, const int32_t* index, void* dx, int N, int H, int W,
                    int Cc, int ksize, int stride, int pad) {
  return maxpool_bwd(C(ctx), dtype, dy, index, dx, N, H, W, Cc, ksize, stride, pad);
}

int tch_avgpool_fwd(tch_context* ctx, int dtype, const void* x, void* y, int N, int HW, int Cc) {
  return avgpool_fwd(C(ctx), dtype, x, y, N, HW, Cc);
}

int tch_avgpool_bwd(tch_context* ctx, int dtype, const void* dy, void* dx, int N, int HW, int Cc) {
  return avgpool_bwd(C(ctx), dtype, dy, dx, N, HW, Cc);
}

int tch_softmax_ce_fwd_bwd(tch_context* ctx, int dtype, const float* logits, const int64_t* labels, float* loss_rows,
                           float* loss_mean, void* dlogits, int rows, int classes, int ld_dlogits, float grad_scale) {
  return softmax_ce_fwd_bwd(C(ctx), dtype, logits, labels, loss_rows, loss_mean, dlogits, rows, classes, ld_dlogits,
                            grad_scale);
}

int tch_softmax_ce_lm(tch_context* ctx, int dtype, const float* logits, int ld_logits, const int64_t* labels,
                      float* loss_rows, float* loss_mean, void* dlogits, int ld_dlogits, int rows, int classes,
                      int valid_rows, float loss_scale) {
  return softmax_ce_lm(C(ctx), dtype, logits, ld_logits, labels, loss_rows, loss_mean, dlogits, ld_dlogits, rows, classes,
                       valid_rows, loss_scale);
}

int tch_bias_grad_ws(tch_context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld,
                     int accumulate, float* workspace, int64_t workspace_floats) {
  return bias_grad(C(ctx), dtype, dy, dbias, rows, cols, ld, accumulate, workspace, workspace_floats);
}

int tch_sgd_momentum_step(tch_context* ctx, float* param, const float* grad, float* momentum_buf, void* shadow_bf16,
                          int64_t n, float lr, float momentum, float weight_decay) {
  return sgd_momentum_step(C(ctx), param, grad, momentum_buf, shadow_bf16, n, lr, momentum, weight_decay);
}

int tch_grad_accumulate(tch_context* ctx, float* global, float* grad, int64_t n) {
  return grad_accumulate(C(ctx), global, grad, n);
}

int tch_fill_zero(tch_context* ctx, void* ptr, int64_t bytes) { return fill_zero(C(ctx), ptr, bytes); }

int tch_bias_grad(tch_context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld,
                  int accumulate) {
  return bias_grad(C(ctx), dtype, dy, dbias, rows, cols, ld, accumulate);
}

int tch_nchw_to_nhwc_pad(tch_context* ctx, int dtype, const float* x_nchw, void* y_nhwc, int N, int Cc, int H, int W,
                         int Cpad) {
  return nchw_to_nhwc_pad(C(ctx), dtype, x_nchw, y_nhwc, N, Cc, H, W, Cpad);
}

int tch_filter_transpose_batched(tch_context* ctx, int dtype, const void* src, void* dst, const int64_t* table_dev,
                                 int n_filters, int64_t total_tiles, int64_t total_elems) {
  return filter_transpose_batched(C(ctx), dtype, src, dst, table_dev, n_filters, total_tiles, total_elems);
}

int tch_cast_from_f32(tch_context* ctx, int dtype, const float* src, void* dst, int64_t n) {
  return cast_f32(C(ctx), dtype, src, dst, n);
}

int tch_cast_to_f32(tch_context* ctx, int dtype, const void* src, float* dst, int64_t n) {
  return cast_to_f32(C(ctx), dtype, src, dst, n);
}

}  // extern "C"

// ---- built-in per-kernel profiler -------------------------------------------------
extern "C" int tch_program_profile(tch_context* ctx, const tch_program* prog, int reps, tch_kernel_stat* out,
                                   int max_out, int* n_out) {
  if (!ctx || !prog || !out || !n_out || max_out < 1) {
    set_error("tch_program_profile: bad arguments");
    return -22;
  }
  std::vector<KernelStat> stats;
  int rc = profile_program(&ctx->ctx, prog->prog, reps, &stats);
  if (rc) return rc;
  int n = 0;
  for (auto& s : stats) {
    if (n >= max_out) break;
    tch_kernel_stat& o = out[n++];
    snprintf(o.name, sizeof(o.name), "%s", s.name.c_str());
    o.total_ms = s.total_ms;
    o.work = s.work;
    o.launches = s.launches;
    o.work_is_bytes = s.work_is_bytes;
    o.bytes = s.bytes;
  }
  *n_out = n;
  return 0;
}

extern "C" int tch_program_time_kernel(tch_context* ctx, const tch_program* prog, const char* kernel_name, int reps,
                                       double* mean_us, int64_t* launches_per_replay) {
  if (!ctx || !prog) {
    set_error("tch_program_time_kernel: null argument");
    return -22;
  }
  // the name must outlive the call only: launches are compared by content
  return time_kernel_in_program(&ctx->ctx, prog->prog, kernel_name, reps, mean_us, launches_per_replay);
}

extern "C" int tch_program_profile_launches(tch_context* ctx, const tch_program* prog, int reps, tch_launch_stat* out,
                                            int64_t max_out, int64_t* n_out) {
  if (!ctx || !prog || !out || !n_out || max_out < 1) {
    set_error("tch_program_profile_launches: bad arguments");
    return -22;
  }
  std::vector<LaunchStat> stats;
  int rc = profile_program(&ctx->ctx, prog->prog, reps, nullptr, &stats);
  if (rc) return rc;
  int64_t n = 0;
  for (auto& s : stats) {
    if (n >= max_out) break;
    tch_launch_stat& o = out[n++];
    snprintf(o.name, sizeof(o.name), "%s", s.name.c_str());
    o.ms = s.ms;
    o.flops = s.flops;
    o.bytes = s.bytes;
    o.lane = s.lane;
    o.workgroups = s.grid;
  }
  *n_out = n;
  return 0;
}
