// Host-side entry points of the device operators (C++ level; the flat C ABI
// in capi.cc forwards to these).  All tensors are NHWC, dtype 0 = fp32,
// 1 = bf16; every function only ENQUEUES work on the context and returns 0 or
// a negative errno-style code with a message retrievable via last_error().
#pragma once

#include <stdint.h>

namespace tch {

class Context;

struct ConvShape {
  int N, H, W, C;  // input batch / height / width / channels
  int K;           // output channels
  int R, S;        // filter height / width
  int stride, pad;
  int c_logical;  // input channels that carry data (<= C; the rest is zero padding); 0 = C
};

void conv_output_hw(const ConvShape& s, int* Ho, int* Wo);

// Turns the sums a convolution epilogue leaves into the BatchNorm's per-channel coefficients as part of the
// convolution call: inside the kernel (the workgroup that finishes a column tile last does it) when there
// are at most kBnFinalizeInKernelTiles row tiles, by a finalize launch otherwise.
constexpr int kBnFinalizeInKernelTiles = 256;
struct BnFinalize {
  int* counters;        // >= ceil(C / 64) ints, zero before the call; left zero
  const float* gamma;
  const float* beta;    // forward
  float* running_mean;  // forward, may be null together with running_var
  float* running_var;
  float* out0;          // forward: saved batch mean      backward: dgamma
  float* out1;          // forward: saved inverse std     backward: dbeta
  float* coef;          // forward: scale[C], shift[C]    backward: coef[3][C]
  float momentum, eps;  // forward
  int accumulate;       // backward: dgamma / dbeta +=
};

// conv_igemm.hip
int conv2d_fwd(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* w, void* y, const void* add,
               const void* mask, const float* bias, int out_f32, int tile_cfg, float* bn_partial = nullptr,
               const BnFinalize* finalize = nullptr, const float* scale = nullptr, int relu_out = 0,
               long long* bn_acc = nullptr, int bn_acc_copies = 1);
// rows of partial statistics conv2d_fwd writes for this shape and tiling (one per row tile)
int conv2d_fwd_stat_rows(const ConvShape& s, int dtype, int tile_cfg);
// The two reductions of a BatchNorm backward, taken in the epilogue of the data-gradient
// convolution that produces the gradient behind that BatchNorm (+ReLU): see finish_tile.
struct BnBwdSums {
  const void* mask;     // optional ReLU output: the gradient is zeroed where mask <= 0 before it is stored
  const void* x;        // the BatchNorm's input, laid out like dx
  const float* mean;    // saved batch statistics, one per channel of dx
  const float* invstd;
  float* partial;       // [conv2d_dgrad_stat_rows][C][2]
  const BnFinalize* finalize;  // optional
  long long* acc = nullptr;    // instead of partial: exact accumulators [copies][4][C] the sums are added to
  int acc_copies = 1;          // power of two: row tile t adds to copy t % copies
};
int conv2d_dgrad(Context* ctx, int dtype, const ConvShape& s, const void* dy, const void* w, void* dx,
                 const void* add, const void* mask, int tile_cfg, const BnBwdSums* bn = nullptr, int add_stride = 1);
int conv2d_dgrad_stat_rows(const ConvShape& s, int dtype, int tile_cfg);
int conv2d_wgrad_pick_splits(const ConvShape& s, int dtype);
int64_t conv2d_wgrad_workspace_bytes(const ConvShape& s, int dtype, int splits);
// dbias (optional, [K] fp32): also the column sums of dy, i.e. the gradient of a bias added to the output
// trailing != 0: the split reduction of THIS call is not launched with it; it rides the next conv2d_wgrad call of the
// context with trailing != 0 (as extra workgroups of that launch: its partials are complete by stream order), or goes
// out with conv2d_wgrad_flush.  The workspace must stay untouched until then: consecutive calls alternate between
// two workspaces.  dw is complete once the launch that carries its reduction has run.
int conv2d_wgrad(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* dy, float* dw,
                 float* workspace, int splits, int accumulate, int tile_cfg, float* dbias = nullptr, int trailing = 0);
int conv2d_wgrad_flush(Context* ctx);
// Several weight gradients as one launch (+ one for the split reductions that remain).  _plan picks a split
// count per convolution so that the group yields about target_wgs workgroups of equal length (one split each if
// the group is large enough without), says how large the device table and the workspace must be, and returns
// the tiling (0 = 128x128, 2 = 64x64) it chose for tile_cfg < 0.
struct WgradGroupItem {
  ConvShape shape;
  const void* x;
  const void* dy;
  float* dw;
  float* dbias;  // optional
  int splits;
};
int conv2d_wgrad_group_plan(int dtype, int n, const ConvShape* shapes, int target_wgs, int tile_cfg, int* splits,
                            int64_t* table_bytes, int64_t* workspace_bytes);
// max_wgs > 0: launch at most that many workgroups, each taking every max_wgs-th tile of the group
int conv2d_wgrad_group(Context* ctx, int dtype, int n, const WgradGroupItem* items, int tile_cfg, int accumulate,
                       float* workspace, void* table, int max_wgs = 0);
// the same with the split-K partials in the library's static device buffer: no workspace, no allocation
int64_t conv2d_wgrad_static_capacity_bytes();
int conv2d_wgrad_static(Context* ctx, int dtype, const ConvShape& s, const void* x, const void* dy, float* dw, int splits,
                        int accumulate, int tile_cfg);

// bn.hip -- training-mode BatchNorm over [rows, C] with fused ReLU / residual
int bn_partial_rows(int64_t rows, int C, int dtype);  // number of row blocks the reductions use
int64_t bn_workspace_bytes(int64_t rows, int C, int dtype);
int bn_fwd_train(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows, int C,
                 const float* gamma, const float* beta, float* running_mean, float* running_var, float* save_mean,
                 float* save_invstd, float momentum, float eps, float* workspace);
// the same with the batch statistics already summed per row block by the producer of x:
// partial[(b * C + c) * 2 + {0, 1}] = sum, sum of squares over the rows of block b; scratch holds 2 C floats
int bn_fwd_train_partials(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                          int64_t rows, int C, const float* gamma, const float* beta, float* running_mean,
                          float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                          const float* partial, int row_blocks, float* scratch);
int bn_bwd(Context* ctx, int dtype, const void* dy, const void* relu_mask, const void* x, void* dx, int64_t rows,
           int C, const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
           int accumulate, float* workspace);
// pieces of the above for callers whose sums come from a convolution epilogue
int bn_fwd_finalize(Context* ctx, const float* partial, int row_blocks, int C, int64_t rows, const float* gamma,
                    const float* beta, float* running_mean, float* running_var, float* save_mean, float* save_invstd,
                    float* coef, float momentum, float eps);
int bn_bwd_finalize(Context* ctx, const float* partial, int row_blocks, int C, int64_t rows, const float* gamma,
                    const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta, float* coef,
                    int accumulate);
int bn_apply_fwd(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows, int C,
                 const float* coef);
int bn_eval_coef(Context* ctx, const float* gamma, const float* beta, const float* running_mean,
                 const float* running_var, float* coef, int C, float eps);
int bn_apply_bwd(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                 const float* coef);
// the same from the sums a convolution epilogue left ([row_blocks][C][2]); g is already gated by the
// ReLU; scratch: 3*C floats
int bn_bwd_partials(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                    const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma,
                    float* dbeta, int accumulate, const float* partial, int row_blocks, float* scratch);
// The same two, where the convolution next to the BatchNorm ADDED its sums to exact per-channel accumulators
// (conv2d_fwd's bn_acc / BnBwdSums::acc) instead of leaving per-tile partials: one launch for any number of rows,
// no finalize.  acc: [copies][4][C] 64-bit words, zero before the convolution ran; C in groups of eight chunks.
int bn_fwd_train_acc(Context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows,
                     int C, const float* gamma, const float* beta, float* running_mean, float* running_var,
                     float* save_mean, float* save_invstd, float momentum, float eps, const long long* acc,
                     int acc_copies);
int bn_bwd_acc(Context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
               const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
               int accumulate, const long long* acc, int acc_copies);

// seq_ops.hip
// Window order (Swin): rows = B * H * W pixels; a tensor flagged in `tensors` (1 = output, 2 = dy, 4 = the addend) is
// laid out as window tokens (cyclic shift by -shift, then ws x ws windows) instead of pixel rows.  ws == 0: none.
struct LnWindow {
  int H = 0, W = 0, ws = 0, shift = 0, tensors = 0;
};
int layernorm_fwd(Context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta, float* mean,
                  float* rstd, int64_t rows, int C, float eps, const LnWindow* win = nullptr,
                  const void* add = nullptr, void* sum_out = nullptr);  // with add: sum_out = x + add, y = LN(sum_out)
int layernorm_bwd_partial_rows(int64_t rows);  // rows of [C][2] fp32 scratch layernorm_bwd needs
int layernorm_bwd(Context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual, const float* gamma,
                  const float* mean, const float* rstd, float* dgamma, float* dbeta, int accumulate, int64_t rows,
                  int C, float* partial, const LnWindow* win = nullptr);
int gelu_fwd(Context* ctx, int dtype, const void* x, void* y, int64_t n, int tanh_form);
int gelu_bwd(Context* ctx, int dtype, const void* dy, const void* x, void* dx, int64_t n, int tanh_form);
int attn_softmax_fwd(Context* ctx, int dtype, const void* scores, void* probs, int64_t batch, int heads, int Lq, int Lk,
                     float scale, const float* bias, const float* mask, int windows, int causal);
int attn_softmax_bwd(Context* ctx, int dtype, const void* probs, const void* dprobs, void* dscores, int64_t rows, int Lq,
                     int Lk, float scale, int causal);
int adamw_step(Context* ctx, float* param, const float* grad, float* exp_avg, float* exp_avg_sq, void* shadow_bf16,
               int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay, int* step_dev,
               float* scalars_dev);
int embedding_fwd(Context* ctx, int dtype, const int64_t* ids, const void* wte, const void* wpe, void* out, int B, int T,
                  int C, int vocab);
int embedding_bwd(Context* ctx, int dtype, const int64_t* ids, const void* dy, float* dwte, float* dwpe, int B, int T,
                  int C, int vocab, int accumulate_wpe, int32_t* chain);

// swin_ops.hip
int window_partition(Context* ctx, int dtype, const void* src, void* dst, const void* add, int B, int H, int W, int C,
                     int window, int shift, int reverse);
int patch_merge_gather(Context* ctx, int dtype, const void* src, void* dst, int B, int H, int W, int C, int reverse);
int relpos_bias_gather(Context* ctx, const float* table, const int32_t* index, float* bias, int heads, int tokens,
                       int entries);
int relpos_bias_scatter(Context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads, int tokens,
                        int entries, int accumulate);
// the same over an arbitrary list of (query, key) pairs, e.g. rows padded to 64 keys: a negative index is padding
// (gathers -inf, receives no gradient)
int relpos_bias_gather_pairs(Context* ctx, const float* table, const int32_t* index, float* bias, int heads, int pairs,
                             int entries);
int relpos_bias_scatter_pairs(Context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads, int pairs,
                              int entries, int accumulate);
// relpos_bias_gather_pairs for `count` tables (host arrays of device pointers) in count / 8 launches
int relpos_bias_gather_batch(Context* ctx, const float* const* tables, const int32_t* const* indices, float* const* biases,
                             const int* heads, int count, int pairs, int entries);
// scatter through the inverse of the index (ptr [entries + 1], list of pair numbers per entry; the caller
// vouches that every listed pair is below `pairs` and ptr is non-decreasing)
int relpos_bias_scatter_csr(Context* ctx, const float* dbias, const int32_t* ptr, const int32_t* list, float* dtable,
                            int heads, int pairs, int entries, int accumulate);
int64_t column_sum_workspace_floats(int rows, int cols);
int column_sum(Context* ctx, int dtype, const void* x, float* out, int rows, int cols, int accumulate, float* workspace);

// bgemm.hip
int batched_gemm(Context* ctx, int dtype, const void* a, const void* b, void* c, int M, int N, int K, int64_t a_rs,
                 int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t ldc, int batch_outer, int batch_inner, int64_t a_bo,
                 int64_t a_bi, int64_t b_bo, int64_t b_bi, int64_t c_bo, int64_t c_bi, float alpha, int accumulate, int causal);

// flash_attn.hip -- attention without the score matrix (bf16, heads 64 wide, T a multiple of 128); head h of
// sample b starts at column 64 h of row b * bs; lse and delta are [B * H][T] fp32
int flash_attn_fwd(Context* ctx, int dtype, const void* q, const void* k, const void* v, void* o, float* lse, int B,
                   int H, int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal);
int flash_attn_bwd(Context* ctx, int dtype, const void* q, const void* k, const void* v, const void* o, const void* dout,
                   const float* lse, float* delta, void* dq, void* dk, void* dv, int B, int H, int T, int64_t qkv_rs,
                   int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal);

// window_attn.hip -- Swin window attention in one launch per direction (bf16, heads 32 wide, N <= 64 tokens):
// qkv [windows * N][3C], o / dout [windows * N][C], probs and ds [windows * heads][N][64], bias [heads][64][64]
// with -inf beyond key N, mask [nW][64][64] or null (window w of an image uses mask w % nW)
int window_attn_fwd(Context* ctx, int dtype, const void* qkv, void* o, void* probs, const float* bias, const float* mask,
                    int windows, int heads, int N, int C, int nW, float scale);
int window_attn_bwd(Context* ctx, int dtype, const void* qkv, const void* probs, const void* dout, void* dqkv, void* ds,
                    int windows, int heads, int N, int C, float scale);

// pool.hip
int maxpool_fwd(Context* ctx, int dtype, const void* x, void* y, int32_t* index, int N, int H, int W, int C, int ksize,
                int stride, int pad);
int maxpool_bwd(Context* ctx, int dtype, const void* dy, const int32_t* index, void* dx, int N, int H, int W, int C,
                int ksize, int stride, int pad);
int avgpool_fwd(Context* ctx, int dtype, const void* x, void* y, int N, int HW, int C);
int avgpool_bwd(Context* ctx, int dtype, const void* dy, void* dx, int N, int HW, int C);

// loss_optim.hip
int softmax_ce_fwd_bwd(Context* ctx, int dtype, const float* logits, const int64_t* labels, float* loss_rows,
                       float* loss_mean, void* dlogits, int rows, int classes, int ld_dlogits, float grad_scale);
// vocabulary-sized rows; rows with a negative label are ignored; mean over valid_rows
int softmax_ce_lm(Context* ctx, int dtype, const float* logits, int ld_logits, const int64_t* labels, float* loss_rows,
                  float* loss_mean, void* dlogits, int ld_dlogits, int rows, int classes, int valid_rows,
                  float loss_scale);
int sgd_momentum_step(Context* ctx, float* param, const float* grad, float* momentum_buf, void* shadow_bf16,
                      int64_t n, float lr, float momentum, float weight_decay);
int grad_accumulate(Context* ctx, float* global, float* grad, int64_t n);
int fill_zero(Context* ctx, void* ptr, int64_t bytes);
int bias_grad(Context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld, int accumulate,
              float* workspace = nullptr, int64_t workspace_floats = 0);

// layout.hip
int nchw_to_nhwc_pad(Context* ctx, int dtype, const float* x_nchw, void* y_nhwc, int N, int C, int H, int W, int Cpad);
int filter_transpose_batched(Context* ctx, int dtype, const void* src, void* dst, const int64_t* table_dev,
                             int n_filters, int64_t total_tiles, int64_t total_elems);
int cast_f32(Context* ctx, int dtype, const float* src, void* dst, int64_t n);
int cast_to_f32(Context* ctx, int dtype, const void* src, float* dst, int64_t n);

}  // namespace tch
