/*
 * torch_col_hip.h -- flat C ABI of libtorch_col_hip.so, part 1: the device side
 * of the colocated training step on MI355X (gfx950).
 *
 * The reference (SiriusInfTra/Sirius) has no arithmetic of its own on this
 * path: train/resnet152.py:22-29,84-91 (and train/swin_b.py:38-45,83-95) build
 * a torchvision model, nn.CrossEntropyLoss and torch.optim.SGD, and every
 * kernel launch of that model travels through the xsched launch queue
 * (third_party/xsched/shim/cuda/shim.cpp:162-203).  The entry points below are
 * what a binding for that path calls instead: NHWC operators that ENQUEUE
 * hand-written HIP kernels on a context (stream + optional preemptible launch
 * queue + optional recording), and the queue controls the reference exposes
 * through common/xsched_ctrl.h:12-40.
 *
 * Conventions
 *   - plain pointers are DEVICE pointers unless a name says host;
 *   - dtype: 0 = fp32, 1 = bf16 (activations and filter shadows); parameters,
 *     gradients, statistics and the loss are always fp32;
 *   - activations are NHWC, filters are [K][R][S][C] (output channel major);
 *   - channel counts must be multiples of one 16-byte chunk (4 fp32 / 8 bf16);
 *   - return value 0 = enqueued, negative = -errno style failure with a
 *     message in tch_last_error() (thread local).  Nothing aborts the process.
 */
#ifndef TORCH_COL_HIP_H_
#define TORCH_COL_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tch_context tch_context;
typedef struct tch_program tch_program;

const char* tch_last_error(void);
/* 1 when the library was built with device code for gfx950 (always, for this build). */
int tch_has_device_code(void);

/* ---- context: where launches go ------------------------------------------------ */
/* hip_stream: a hipStream_t (0 = the null stream).  If the stream is registered
 * (tch_RegisterStream) launches pass through its launch queue. */
int tch_context_create(void* hip_stream, tch_context** out);
void tch_context_destroy(tch_context* ctx);
/* launches skipped since the last call because the reject flag was up */
uint64_t tch_context_take_rejected(tch_context* ctx);
/* While recording: launches are stamped with `lane` (0 = the context's stream, 1 = may run beside
 * lane 0 on a second stream of the same priority); with wait_main the next lane-1 launch first
 * waits for everything lane 0 was given before it.  tch_context_join records the point where
 * lane 0 waits for lane 1; tch_context_join_behind a point where lane 0 waits for what lane 1 had
 * been given at the PREVIOUS such point (for a caller that rotates three sets of buffers: lane 1
 * may trail by one set).  A program stays a valid serial order (tch_program_profile runs it on
 * one stream, in order); behind a registered (preemptible) stream the lanes stay two streams and
 * their meeting points are queued in order with the launches.
 * No counterpart in the reference (its backward runs on one stream). */
int tch_context_set_lane(tch_context* ctx, int lane, int wait_main);
int tch_context_join(tch_context* ctx);
int tch_context_join_behind(tch_context* ctx);
int tch_context_synchronize(tch_context* ctx); /* both streams of the context */

/* ---- programs: record once, replay every step ---------------------------------- */
int tch_program_create(tch_program** out);
void tch_program_destroy(tch_program* prog);
int64_t tch_program_size(const tch_program* prog);
/* Between begin and end every operator call on ctx appends to prog instead of launching. */
int tch_program_begin_record(tch_context* ctx, tch_program* prog);
int tch_program_end_record(tch_context* ctx);
/* Replay launches [first, last) (last < 0: to the end).  The reject flag is a
 * checkpoint between launches: returns 1 if any launch was skipped because of it. */
int tch_program_run(tch_context* ctx, const tch_program* prog, int64_t first, int64_t last);

/* ---- per-kernel timing of a program ---------------------------------------------- */
typedef struct tch_kernel_stat {
  char name[96];      /* kernel name, e.g. "igemm_kernel<bf16,fwd,128x128>" */
  double total_ms;    /* summed HIP-event time of its launches over all repetitions */
  double work;        /* summed ALGORITHMIC work of those launches: flops or bytes */
  int64_t launches;
  int work_is_bytes;  /* 1: work counts bytes (HBM-bound kernel), 0: flops (MFMA kernel) */
  double bytes;       /* summed ALGORITHMIC bytes of those launches (equals work when work counts bytes; 0 where a
                         flops-annotated kernel states none): flops / peak against bytes / bandwidth tells which roof binds */
} tch_kernel_stat;
/* Replays prog `reps` times directly on the context's stream (not through a launch queue)
 * with a HIP event between any two launches; one row per kernel name. */
int tch_program_profile(tch_context* ctx, const tch_program* prog, int reps, tch_kernel_stat* out, int max_out,
                        int* n_out);
typedef struct tch_launch_stat {
  char name[96];      /* kernel name; empty for a program entry that launches nothing (a join of the lanes) */
  double ms;          /* mean HIP-event time of this launch over the repetitions */
  double flops;       /* ALGORITHMIC flops of the launch (0 where it is annotated with bytes only) */
  double bytes;       /* ALGORITHMIC bytes of the launch */
  int lane;           /* 0 = main lane, 1 = the lane that may run beside it */
  int64_t workgroups;
} tch_launch_stat;
/* The same replay, one row per program position (out[i] is launch i): what each launch of a step costs alone
 * on the chip, next to the work it states -- the input of a per-layer roofline table. */
int tch_program_profile_launches(tch_context* ctx, const tch_program* prog, int reps, tch_launch_stat* out,
                                 int64_t max_out, int64_t* n_out);
/* One kernel family INSIDE the program as it runs: `reps` plain replays (both lanes, nothing added between the
 * launches; not for a context behind a launch queue), every launch of the kernel called `kernel_name` carrying
 * a start and a stop event of its own.  mean_us: mean duration of those launches while the rest of the program
 * shares the chip with them -- the figure a rocprofv3 kernel trace of the same run shows, and what a roofline
 * fraction of a kernel that runs beside others should be quoted on. */
int tch_program_time_kernel(tch_context* ctx, const tch_program* prog, const char* kernel_name, int reps,
                            double* mean_us, int64_t* launches_per_replay);

/* ---- preemptible launch queues (replaces common/xsched_ctrl.h:12-40) ------------ */
uint64_t tch_RegisterStream(uint64_t hip_stream);   /* xsched_ctrl.cc:27-46; 0 on failure */
int tch_UnRegisterStream(uint64_t hip_stream);      /* xsched_ctrl.cc:70-78 */
void tch_UnRegisterAllStreams(void);                /* xsched_ctrl.cc:80-86 */
size_t tch_GetXQueueSize(uint64_t hip_stream);      /* xsched_ctrl.cc:158-166 */
size_t tch_GetXQueueSizeAllStreams(void);           /* xsched_ctrl.cc:168-178 */
size_t tch_GetTotalXQueueSize(void);                /* xsched_ctrl.cc:180-190 */
size_t tch_AbortStream(uint64_t hip_stream);        /* xsched_ctrl.cc:110-115 */
size_t tch_AbortAllStreams(void);                   /* xsched_ctrl.cc:117-138 */
int tch_SyncStream(uint64_t hip_stream);            /* xsched_ctrl.cc:140-147 */
int tch_SyncAllStreams(void);                       /* xsched_ctrl.cc:149-156 */
int tch_QueryRejectCudaCalls(void);                 /* xsched_ctrl.cc:192-194 */
void tch_SetRejectCudaCalls(int reject);            /* xsched_ctrl.cc:196-198 */
/* Every registered queue stops handing launches to the hardware (what it already handed over runs on; with
 * sync_hw the call returns when that has finished), until resumed; launches submitted meanwhile wait in
 * order, or are dropped by tch_ResumeAllStreams(1).  Work another tenant submits to its own stream in between
 * runs ahead of everything the queues hold: preemption between kernels
 * (third_party/xsched/preempt/xqueue/xqueue.cpp:80-137 Suspend / Resume). */
void tch_SuspendAllStreams(int sync_hw);
void tch_ResumeAllStreams(int drop_commands);
/* queue length / sync interval used by later tch_RegisterStream calls (reference: 16, 8; default here: 16, 4 --
 * the length bounds what a preempting tenant waits behind, the interval only sets how often the worker can
 * notice that launches finished) */
void tch_SetXQueueShape(int queue_length, int sync_interval);
size_t tch_GetXQueueInFlight(uint64_t hip_stream);

/* ---- compute-unit partitioning (the reference's SMPartitioner, common/sm_partition.cc:26-112, with compute
 * units in the place of TPCs; csrc/init.cc:43-71 installs it) ------------------------------------------
 * init: total_cus <= 0 asks the current device; training may use between min and max compute units.
 * train_avail(required) = min(max, max(min, total - required)).  A context with a limit n launches on streams
 * whose CU mask keeps the highest-numbered n compute units (the other tenant keeps the lowest); 0 lifts the
 * limit.  Changing the limit between two program runs is ordered like any two launches of the context. */
int tch_cu_partition_init(int total_cus, int min_train_cus, int max_train_cus);
int tch_cu_partition_total(void);
int tch_cu_partition_train_avail(int infer_required_cus);
int tch_context_set_cu_limit(tch_context* ctx, int n_cus);
int tch_context_get_cu_limit(tch_context* ctx);

/* ---- convolution (implicit GEMM on MFMA) ---------------------------------------- */
/* y[N,Ho,Wo,K] = conv(x[N,H,W,C], w[K,R,S,C]) (+ bias[K]) (+ add, optionally gated by mask > 0).
 * out_f32 != 0 stores y as fp32 whatever dtype is.  tile_cfg: -1 auto, 0 = 128x128, 1 = 128x64, 2 = 64x64,
 * 3 = 64x64 on the register-staged kernel even where the direct-to-LDS kernel applies, 5 = 128x64 with the
 * activation side of all nine taps of a channel block held in LDS as one patch (bf16, 3x3, stride 1, pad 1,
 * channels a multiple of 64, rows of at most 63 pixels; any other convolution runs tiling 1 for it).  The patch
 * kernel adds up channel block by channel block, the others tap by tap: results agree to rounding, not bit for bit.
 * 6 / 7 = tilings 1 / 2 with two LDS tiles in flight instead of three (more workgroups per CU).
 * c_logical: input channels that carry data when C is zero-padded to a chunk (0 = C); it only enters the
 * algorithmic-work figure the profiler reports, never the arithmetic. */
int tch_conv2d_fwd(tch_context* ctx, int dtype, const void* x, const void* w, void* y, const void* add,
                   const void* mask, const float* bias, int out_f32, int N, int H, int W, int C, int K, int R, int S,
                   int stride, int pad, int tile_cfg, int c_logical);
/* Convolution -> inference-mode BatchNorm (-> + residual) (-> ReLU) as ONE launch: y = relu?(conv(x, w) * scale[K]
 * + shift[K] + residual?), everything after the convolution applied to the fp32 accumulators in the epilogue.
 * scale / shift as tch_bn_eval_coef leaves them (model.eval(): F.batch_norm with training=False); what an
 * inference graph compiler makes of torchvision's conv -> bn -> relu triples, and what the batch-1 ResNet-152
 * requests of the colocated inference side run.  scale, shift, residual may be NULL. */
int tch_conv2d_fwd_affine(tch_context* ctx, int dtype, const void* x, const void* w, void* y, const float* scale,
                          const float* shift, const void* residual, int relu, int N, int H, int W, int C, int K, int R,
                          int S, int stride, int pad, int tile_cfg, int c_logical);
/* The convolution that feeds a BatchNorm (torchvision's conv -> bn pairs, train/resnet152.py:22): y as
 * above (no bias / addend), and per (row tile, output channel) the sum and the sum of squares of y as
 * stored: bn_partial[(tile * K + k) * 2 + {0,1}], tch_conv2d_fwd_stat_rows(...) row tiles.  Saves the
 * statistics pass over y; feed the partials to tch_bn_fwd_train_partials. */
int tch_conv2d_fwd_bnstats(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W,
                           int C, int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical,
                           float* bn_partial);
int tch_conv2d_fwd_stat_rows(int dtype, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                             int tile_cfg);
/* dx[N,H,W,C] = conv_transpose(dy[N,Ho,Wo,K], w) (+ add, optionally gated by mask > 0).
 * wt is the filter TRANSPOSED to [C][R][S][K] (tch_filter_transpose_batched).
 * add_stride (here and in the two forms below): 1 = `add` is laid out like dx; 2 = `add` is [N, ceil(H/2),
 * ceil(W/2), C], the values of the even (h, w) of dx's grid, and counts there only: the data gradient of a
 * stride-2 1x1 convolution (a ResNet downsample branch) is non-zero at those pixels alone, so it is computed on its
 * own small grid (as the stride-1 data gradient over dy's pixels) and never blown up to dx's. */
int tch_conv2d_dgrad(tch_context* ctx, int dtype, const void* dy, const void* wt, void* dx, const void* add,
                     const void* mask, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                     int tile_cfg, int c_logical, int add_stride);
/* The same where dx is the gradient behind a BatchNorm (+ReLU) whose input is bn_x (laid out like dx) and
 * whose ReLU output is bn_mask (may be NULL: no ReLU): dx is zeroed where bn_mask <= 0 before it is stored
 * and the epilogue leaves, per row tile and channel, sum(dx) and sum(dx * (bn_x - mean) * invstd) at
 * bn_partial[(tile * C + c) * 2 + {0,1}], tile < tch_conv2d_dgrad_stat_rows(): the two reductions of that
 * BatchNorm's backward, with no pass over dx; feed them to tch_bn_bwd_partials. */
int tch_conv2d_dgrad_bnsums(tch_context* ctx, int dtype, const void* dy, const void* wt, void* dx, const void* add,
                            const void* mask, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                            int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                            const float* bn_invstd, float* bn_partial, int add_stride);
int tch_conv2d_dgrad_stat_rows(int dtype, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                               int tile_cfg);
/* The same two with the sums ADDED to exact accumulators instead of left per row tile.  bn_acc is
 * [acc_copies][4][channels] 64-bit integers: planes 0 / 1 collect the first sum in units of 2^-24 / 2^-66, planes
 * 2 / 3 the second (integer additions, so the totals do not depend on the order the workgroups finish in and a step
 * stays bit-identical from run to run); row tile t adds to copy t % acc_copies (a power of two: additions to one
 * address queue up behind each other, about 20 ns each, so layers with many row tiles want several copies).
 * bn_acc must be zero before the call (tch_fill_zero); feed it, with the same acc_copies, to tch_bn_fwd_train_acc /
 * tch_bn_bwd_acc, which need no finalize launch and no pass over per-tile partials.
 * What torch's conv2d -> batch_norm pairs (train/resnet152.py:22) need of each other, as two launches. */
int tch_conv2d_fwd_bnacc(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W,
                         int C, int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical,
                         int64_t* bn_acc, int acc_copies);
int tch_conv2d_dgrad_bnacc(tch_context* ctx, int dtype, const void* dy, const void* wt, void* dx, const void* add,
                           const void* mask, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                           int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                           const float* bn_invstd, int64_t* bn_acc, int acc_copies, int add_stride);
/* Convolution + the whole front half of the BatchNorm next to it, in one call: the sums as above, and the
 * per-channel coefficients from them (by the workgroup that finishes a column tile last, or by a finalize launch
 * when there are more than 256 row tiles).  counters: >= ceil(channels / 64) ints, zero before the call, zero
 * after it.  Forward: save_mean / save_invstd / running statistics are updated, coef = scale[K], shift[K];
 * finish with tch_bn_apply_fwd.  Data gradient: dgamma / dbeta (+)=, coef = [3][C]; finish with tch_bn_apply_bwd. */
int tch_conv2d_fwd_bn(tch_context* ctx, int dtype, const void* x, const void* w, void* y, int N, int H, int W, int C,
                      int K, int R, int S, int stride, int pad, int tile_cfg, int c_logical, float* bn_partial,
                      int* counters, const float* gamma, const float* beta, float* running_mean, float* running_var,
                      float* save_mean, float* save_invstd, float momentum, float eps, float* coef);
int tch_conv2d_dgrad_bn(tch_context* ctx, int dtype, const void* dy, const void* wt, void* dx, const void* add,
                        const void* mask, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                        int tile_cfg, int c_logical, const void* bn_mask, const void* bn_x, const float* bn_mean,
                        const float* bn_invstd, float* bn_partial, int* counters, const float* gamma, float* dgamma,
                        float* dbeta, int accumulate, float* coef, int add_stride);
/* y = relu?(x * scale + shift (+ residual)), coef = scale[C], shift[C];  dx = c0 * g + c1 * x + c2, coef = [3][C] */
int tch_bn_apply_fwd(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu, int64_t rows,
                     int C, const float* coef);
/* Inference-mode BatchNorm (model.eval(): F.batch_norm with training=False, as the batch-1 ResNet-152 requests of
 * the colocated inference side run it): coef = scale[C], shift[C] with scale = gamma / sqrt(running_var + eps),
 * shift = beta - running_mean * scale; apply with tch_bn_apply_fwd. */
int tch_bn_eval_coef(tch_context* ctx, const float* gamma, const float* beta, const float* running_mean,
                     const float* running_var, float* coef, int C, float eps);
int tch_bn_apply_bwd(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                     const float* coef);
/* dw[K,R,S,C] (fp32) (+)= sum over pixels of dy x x.  splits > 1 needs a workspace of
 * tch_conv2d_wgrad_workspace_bytes(); splits <= 0 lets the library choose (query with _pick_splits). */
int tch_conv2d_wgrad_pick_splits(int dtype, int N, int H, int W, int C, int K, int R, int S, int stride, int pad);
int64_t tch_conv2d_wgrad_workspace_bytes(int dtype, int K, int R, int S, int C, int splits);
int tch_conv2d_wgrad(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* workspace,
                     int splits, int accumulate, int N, int H, int W, int C, int K, int R, int S, int stride,
                     int pad, int tile_cfg, int c_logical);
/* tch_conv2d_wgrad_bias (dbias may be NULL) for a RUN of weight gradients on one context, without a launch per
 * split reduction: the reduction of a call's partials is not launched with it but rides the NEXT call of this kind
 * on the same context as extra workgroups of that launch (the partials are complete by stream order, and the
 * reduction then runs beside the next gradient's multiplications instead of behind its own), in the same fixed
 * order of the splits: same bits as tch_conv2d_wgrad.  Consecutive calls must alternate between two workspaces
 * (a call's workspace is read by the call after it); dw / dbias of a call are complete once the next call, or
 * tch_conv2d_wgrad_flush, has run: flush before anything reads the last gradient.  What autograd's per-layer
 * weight-gradient calls (train/resnet152.py:84-91) become on a stream of their own. */
int tch_conv2d_wgrad_trailing(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* dbias,
                              float* workspace, int splits, int accumulate, int N, int H, int W, int C, int K, int R,
                              int S, int stride, int pad, int tile_cfg, int c_logical);
int tch_conv2d_wgrad_flush(tch_context* ctx);
/* The weight gradients (and optional bias gradients) of n convolutions as ONE launch over a table in device
 * memory, plus one launch for the split reductions that remain: what a training step does once a stage's
 * data-gradient chain has passed and every dy of the stage is at hand (the reference gets one cuDNN call per
 * layer from autograd: train/resnet152.py:84-91; the result per layer is that of tch_conv2d_wgrad with the same
 * split count, bit for bit).  shapes = n x {N, H, W, C, K, R, S, stride, pad}; x / dy / dw / dbias = n device
 * addresses each (dbias may be NULL, or hold zeros for layers without a bias).
 * _plan writes a split count per convolution so that the group yields about target_wgs (<= 0: 1024) workgroups
 * of about equal length -- one split each, no partial filters at all, if the group is large enough -- and the
 * bytes of `table` and `workspace` the call needs; it returns the tiling (0 = 128x128, 2 = 64x64) that
 * tile_cfg < 0 stands for.  `table` is written by the call (synchronously) and read by the launches whenever
 * they run: it must stay untouched for as long as a recorded program holds them.  max_wgs > 0 caps the launch at
 * that many workgroups, each of which then takes every max_wgs-th tile of the group in turn: a launch that
 * runs beside other kernels on a share of every compute unit instead of flooding the chip (same results). */
int tch_conv2d_wgrad_group_plan(int dtype, int n, const int* shapes, int target_wgs, int tile_cfg, int* splits,
                                int64_t* table_bytes, int64_t* workspace_bytes);
int tch_conv2d_wgrad_group(tch_context* ctx, int dtype, int n, const int* shapes, const uint64_t* x, const uint64_t* dy,
                           const uint64_t* dw, const uint64_t* dbias, const int* splits, int tile_cfg, int accumulate,
                           float* workspace, void* table, int max_wgs);
/* tch_conv2d_wgrad for callers that cannot allocate device memory and hold no workspace of their own: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same kernels and same result, bit for bit, as tch_conv2d_wgrad with the same split count; the
 * split-K partials live in a static device buffer of tch_conv2d_wgrad_static_capacity_bytes() (64 MiB) that is
 * part of the library's code object on every GPU it runs on.  The call allocates and frees nothing.  splits <= 0:
 * the library's choice, lowered to what the buffer holds; an explicit split count whose partials
 * (splits * (K*R*S*C + K) * 4 bytes) exceed the buffer is rejected with an error.  All calls on one GPU share the
 * buffer.  Calls whose launches go to a stream at once are kept apart by the library: a call on another stream
 * than the buffer's last user first waits (on the device, hipStreamWaitEvent) for that user's reduction.  Calls
 * that are recorded into a program, held in a preemptible launch queue or captured into a HIP graph run later, in
 * an order the library does not see: ONE such program / queue / graph may use the buffer at a time, and two that
 * overlap on one GPU race. */
int64_t tch_conv2d_wgrad_static_capacity_bytes(void);
int tch_conv2d_wgrad_static(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, int splits,
                            int accumulate, int N, int H, int W, int C, int K, int R, int S, int stride, int pad,
                            int tile_cfg, int c_logical);
/* The same, and dbias[K] (fp32) (+)= sum over pixels of dy: weight and bias gradient of a linear layer
 * (torch.nn.Linear's backward under train/gpt2.py:26 and train/swin_b.py:38) in one pass over dy. */
int tch_conv2d_wgrad_bias(tch_context* ctx, int dtype, const void* x, const void* dy, float* dw, float* dbias,
                          float* workspace, int splits, int accumulate, int N, int H, int W, int C, int K, int R, int S,
                          int stride, int pad, int tile_cfg, int c_logical);

/* ---- BatchNorm (training mode) with fused ReLU / residual ---------------------- */
int64_t tch_bn_workspace_bytes(int dtype, int64_t rows, int C);
/* y = relu?(bn(x) + residual?) over x viewed as [rows, C]; updates running stats (may be NULL),
 * writes save_mean / save_invstd for the backward pass. */
int tch_bn_fwd_train(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                     int64_t rows, int C, const float* gamma, const float* beta, float* running_mean,
                     float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                     float* workspace);
/* The same, with the batch statistics already summed per row block (tch_conv2d_fwd_bnstats):
 * partial[(b * C + c) * 2 + {0,1}] for b < row_blocks; scratch holds 2 C floats. */
int tch_bn_fwd_train_partials(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                              int64_t rows, int C, const float* gamma, const float* beta, float* running_mean,
                              float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                              const float* partial, int row_blocks, float* scratch);
/* g = dy * (relu_mask > 0) (relu_mask may be NULL); dgamma/dbeta (+)=; dx = bn'(g) */
int tch_bn_bwd(tch_context* ctx, int dtype, const void* dy, const void* relu_mask, const void* x, void* dx,
               int64_t rows, int C, const float* gamma, const float* save_mean, const float* save_invstd,
               float* dgamma, float* dbeta, int accumulate, float* workspace);
/* The same from the sums tch_conv2d_dgrad_bnsums left; g is already gated by the ReLU; scratch holds 3 C floats. */
int tch_bn_bwd_partials(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                        const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma,
                        float* dbeta, int accumulate, const float* partial, int row_blocks, float* scratch);

/* tch_bn_fwd_train_partials / tch_bn_bwd_partials from the accumulators of tch_conv2d_fwd_bnacc /
 * tch_conv2d_dgrad_bnacc (acc[acc_copies * 4 * C] 64-bit words): coefficients and apply in ONE launch whatever the
 * number of rows.  C must be a multiple of eight 16-byte chunks (64 for bf16, 32 for fp32). */
int tch_bn_fwd_train_acc(tch_context* ctx, int dtype, const void* x, void* y, const void* residual, int relu,
                         int64_t rows, int C, const float* gamma, const float* beta, float* running_mean,
                         float* running_var, float* save_mean, float* save_invstd, float momentum, float eps,
                         const int64_t* acc, int acc_copies);
int tch_bn_bwd_acc(tch_context* ctx, int dtype, const void* g, const void* x, void* dx, int64_t rows, int C,
                   const float* gamma, const float* save_mean, const float* save_invstd, float* dgamma, float* dbeta,
                   int accumulate, const int64_t* acc, int acc_copies);

/* ---- pooling -------------------------------------------------------------------- */
/* index[N,Ho,Wo,C] (int32) = h*W + w of the FIRST maximum in row-major window order (NaN wins). */
int tch_maxpool_fwd(tch_context* ctx, int dtype, const void* x, void* y, int32_t* index, int N, int H, int W, int C,
                    int ksize, int stride, int pad);
int tch_maxpool_bwd(tch_context* ctx, int dtype, const void* dy, const int32_t* index, void* dx, int N, int H, int W,
                    int C, int ksize, int stride, int pad);
int tch_avgpool_fwd(tch_context* ctx, int dtype, const void* x, void* y, int N, int HW, int C);
int tch_avgpool_bwd(tch_context* ctx, int dtype, const void* dy, void* dx, int N, int HW, int C);

/* ---- loss, optimizer, accumulation ---------------------------------------------- */
/* loss_rows[i] = logsumexp(logits[i]) - logits[i, label]; loss_mean = mean; dlogits (dtype, leading
 * dimension ld_dlogits) = (softmax - onehot) * grad_scale, grad_scale = loss_scale / rows. */
int tch_softmax_ce_fwd_bwd(tch_context* ctx, int dtype, const float* logits, const int64_t* labels, float* loss_rows,
                           float* loss_mean, void* dlogits, int rows, int classes, int ld_dlogits, float grad_scale);
/* The language-model form (GPT-2's output.loss, train/gpt2.py:93): rows as long as the vocabulary, logits with
 * their own leading dimension, a row whose label is negative is ignored (zero loss, zero gradient);
 * loss_mean = sum / valid_rows, dlogits = (softmax - onehot) * loss_scale / valid_rows.  Columns of dlogits
 * from `classes` up to ld_dlogits are not written. */
int tch_softmax_ce_lm(tch_context* ctx, int dtype, const float* logits, int ld_logits, const int64_t* labels,
                      float* loss_rows, float* loss_mean, void* dlogits, int ld_dlogits, int rows, int classes,
                      int valid_rows, float loss_scale);
/* g += wd*p; buf = momentum*buf + g; p -= lr*buf; shadow_bf16 (may be NULL) = bf16(p) */
int tch_sgd_momentum_step(tch_context* ctx, float* param, const float* grad, float* momentum_buf, void* shadow_bf16,
                          int64_t n, float lr, float momentum, float weight_decay);
/* global += grad; grad = 0   (pytorch/torch_col/accumulate.py:20-24) */
int tch_grad_accumulate(tch_context* ctx, float* global, float* grad, int64_t n);
int tch_fill_zero(tch_context* ctx, void* ptr, int64_t bytes);
/* dbias[c] (+)= sum over rows of dy[r, c] (dy with leading dimension ld) */
int tch_bias_grad(tch_context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld,
                  int accumulate);
/* The same with fp32 scratch memory (workspace_floats >= 2 * cols is useful, 64 * cols is the most it takes): with
 * thousands of rows (tokens) the rows are cut into slabs that separate workgroups sum, in a fixed order. */
int tch_bias_grad_ws(tch_context* ctx, int dtype, const void* dy, float* dbias, int rows, int cols, int ld,
                     int accumulate, float* workspace, int64_t workspace_floats);

/* ---- transformer operators (Swin-B / GPT-2 steps) --------------------------------------
 * The arithmetic restates torch.nn.LayerNorm / GELU / softmax / AdamW / Embedding as the reference's
 * training scripts use them through torchvision and transformers (train/swin_b.py:38-45,
 * train/gpt2.py:26-33; a readable statement of window attention: train/swin_b_tiny.py:8-172). */
/* y = (x - mean) * rstd * gamma + beta over the last dimension of [rows, C] (C <= 2048); mean / rstd [rows]
 * are kept for the backward. */
int tch_layernorm_fwd(tch_context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta,
                      float* mean, float* rstd, int64_t rows, int C, float eps);
/* dx = LayerNorm'(dy) (+ residual, laid out like dx, may be NULL: the gradient that bypasses the LayerNorm);
 * partial: fp32 scratch of tch_layernorm_bwd_partial_rows(rows) * C * 2 floats; dgamma / dbeta (+)= */
int tch_layernorm_bwd_partial_rows(int64_t rows);
int tch_layernorm_bwd(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual,
                      const float* gamma,
                      const float* mean, const float* rstd, float* dgamma, float* dbeta, int accumulate, int64_t rows,
                      int C, float* partial);
/* LayerNorm next to a window partition (Swin: train/swin_b_tiny.py:8-19, 116-131 roll + window_partition /
 * window_reverse around the attention of a block).  rows = B * H * W pixels in row order; x, mean and rstd stay in
 * that order.  windowed_tensors flags the tensors that are laid out as window tokens (cyclic shift by -shift, then
 * window x window windows) instead: forward y (1) and the addend (4); backward dx (1), dy (2), the residual (4).
 * Forward with an addend (add, sum_out both non-NULL; sum_out in pixel order): sum_out = x + add rounded to the
 * tensors' type, y = LayerNorm(sum_out): the residual sum behind the attention of a block (window_reverse + add)
 * and the LayerNorm in front of its MLP in one pass.  Same values as the plain calls with tch_window_partition
 * between them.  Where the window does not tile the image (H or W not a multiple of window) the window tokens live in
 * the frame padded at the bottom and the right to whole windows, as torchvision's shifted_window_attention pads its
 * input: a window-ordered tensor then has B * Hp * Wp rows (Hp, Wp = H, W rounded up), these calls read and write the
 * rows that belong to pixels only, and the caller keeps the others zero where they are read (tch_fill_zero before a
 * forward y / a backward dx is written). */
int tch_layernorm_fwd_windowed(tch_context* ctx, int dtype, const void* x, void* y, const float* gamma, const float* beta,
                               float* mean, float* rstd, int64_t rows, int C, float eps, int H, int W, int window,
                               int shift, int windowed_tensors, const void* add, void* sum_out);
int tch_layernorm_bwd_windowed(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, const void* residual,
                               const float* gamma, const float* mean, const float* rstd, float* dgamma, float* dbeta,
                               int accumulate, int64_t rows, int C, float* partial, int H, int W, int window, int shift,
                               int windowed_tensors);
/* tanh_form 0: 0.5 x (1 + erf(x / sqrt 2)) (nn.GELU); 1: GPT-2's gelu_new.  n is a multiple of a 16-byte chunk. */
int tch_gelu_fwd(tch_context* ctx, int dtype, const void* x, void* y, int64_t n, int tanh_form);
int tch_gelu_bwd(tch_context* ctx, int dtype, const void* dy, const void* x, void* dx, int64_t n, int tanh_form);
/* probs = softmax over the last dimension of scale * scores[batch, heads, Lq, Lk] + bias[heads, Lq, Lk]
 * + mask[windows, Lq, Lk] (window = batch index % windows); bias and mask may be NULL; causal != 0 keeps keys
 * j <= i only (Lq == Lk).  In place (probs == scores) is allowed. */
int tch_attn_softmax_fwd(tch_context* ctx, int dtype, const void* scores, void* probs, int64_t batch, int heads, int Lq,
                         int Lk, float scale, const float* bias, const float* mask, int windows, int causal);
/* dscores = scale * probs * (dprobs - sum_j dprobs_j probs_j) per row; rows = batch * heads * Lq.  causal != 0:
 * dprobs beyond the query's own position is never read and dscores there is zero.  In place (dscores == dprobs)
 * is allowed. */
int tch_attn_softmax_bwd(tch_context* ctx, int dtype, const void* probs, const void* dprobs, void* dscores, int64_t rows,
                         int Lq, int Lk, float scale, int causal);
/* torch.optim.AdamW (decoupled decay, bias correction) over a flat fp32 buffer; step_dev (int32, starts at 0)
 * and scalars_dev (2 floats) live on the device so that a recorded program advances the step by itself. */
int tch_adamw_step(tch_context* ctx, float* param, const float* grad, float* exp_avg, float* exp_avg_sq,
                   void* shadow_bf16, int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay,
                   int* step_dev, float* scalars_dev);
/* out[b, t, :] = wte[ids[b, t], :] + wpe[t, :]; backward: dwte[id] += the dy rows of the positions that hold id,
 * dwpe (+)= sum over b.  chain: 2 * B * T int32 of scratch; with it the rows that share a token are added up in
 * position order by one thread (the same bits every run); NULL: fp32 atomics, order not fixed. */
int tch_embedding_fwd(tch_context* ctx, int dtype, const int64_t* ids, const void* wte, const void* wpe, void* out, int B,
                      int T, int C, int vocab);
int tch_embedding_bwd(tch_context* ctx, int dtype, const int64_t* ids, const void* dy, float* dwte, float* dwpe, int B,
                      int T, int C, int vocab, int accumulate_wpe, int32_t* chain);
/* C[z](m, n) (+)= alpha * sum_k A[z](m, k) B[z](n, k), z = zo * batch_inner + zi; A(m, k) at
 * a + zo * a_bo + zi * a_bi + m * a_rs + k * a_cs (elements), B alike with n; C row-major with ldc.
 * One stride of each operand must be 1.  causal (square problems under a causal mask): 0 nothing is known;
 * 1 only C(m, n) with n <= m is wanted (tiles wholly above the diagonal are left unwritten); 2 A(m, k) = 0 for
 * k > m; 3 A(m, k) = 0 for k < m (the reduction is cut to the part that can be non-zero). */
int tch_batched_gemm(tch_context* ctx, int dtype, const void* a, const void* b, void* c, int M, int N, int K,
                     int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t ldc, int batch_outer,
                     int batch_inner, int64_t a_bo, int64_t a_bi, int64_t b_bo, int64_t b_bi, int64_t c_bo, int64_t c_bi,
                     float alpha, int accumulate, int causal);

/* Attention of the GPT-2 step as one fused pass: o = softmax(scale * q k^T [+ causal mask]) v per head, the
 * [T, T] scores never leave the chip (what transformers' GPT2Attention computes inside train/gpt2.py:26 with
 * the benchmark's dropout of 0).  bf16 only (dtype 1), heads 64 wide, T a multiple of 128.  q, k, v (and dq, dk,
 * dv) share one layout: element (b, t, h, d) at b * qkv_bs + t * qkv_rs + 64 h + d, so the three may be views of
 * one packed [B, T, 3C] projection; o and dout likewise with o_bs / o_rs.  lse [B * H][T] fp32 receives the
 * natural log-sum-exp of the scaled scores; the backward reads it back, fills delta [B * H][T] (row sums of
 * dout * o) and writes dq, dk, dv in two launches without atomics. */
int tch_flash_attn_fwd(tch_context* ctx, int dtype, const void* q, const void* k, const void* v, void* o, float* lse,
                       int B, int H, int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale,
                       int causal);
int tch_flash_attn_bwd(tch_context* ctx, int dtype, const void* q, const void* k, const void* v, const void* o,
                       const void* dout, const float* lse, float* delta, void* dq, void* dk, void* dv, int B, int H,
                       int T, int64_t qkv_rs, int64_t qkv_bs, int64_t o_rs, int64_t o_bs, float scale, int causal);

/* Window attention of the Swin-B step in one launch per direction (train/swin_b_tiny.py:94-110: q k^T * scale +
 * relative position bias (+ shift mask), softmax, @ v; torchvision's shifted_window_attention for
 * train/swin_b.py:38).  bf16 only, heads 32 wide (C = 32 heads), N <= 64 tokens per window.
 * qkv [windows * N][3C] is the packed projection of the window-partitioned tokens, o / dout [windows * N][C];
 * probs and ds are [windows * heads][N][64] (key rows padded to 64; the forward stores the probabilities there,
 * the backward reads them and stores the gradient of the logits, whose sum over the windows is the bias
 * gradient); bias [heads][64][64] fp32 holds -inf in the key columns from N on (tch_relpos_bias_gather_pairs
 * with negative indices there); mask [nW][64][64] fp32 or null, window w uses mask w % nW. */
int tch_window_attn_fwd(tch_context* ctx, int dtype, const void* qkv, void* o, void* probs, const float* bias,
                        const float* mask, int windows, int heads, int N, int C, int nW, float scale);
int tch_window_attn_bwd(tch_context* ctx, int dtype, const void* qkv, const void* probs, const void* dout, void* dqkv,
                        void* ds, int windows, int heads, int N, int C, float scale);
/* tch_relpos_bias_gather / _scatter over an explicit list of (query, key) pairs instead of tokens^2: index[pair]
 * < 0 marks padding (gathers -inf, takes no gradient). */
int tch_relpos_bias_gather_pairs(tch_context* ctx, const float* table, const int32_t* index, float* bias, int heads,
                                 int pairs, int entries);
int tch_relpos_bias_scatter_pairs(tch_context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads,
                                  int pairs, int entries, int accumulate);
/* tch_relpos_bias_gather_pairs for the `count` bias tables of a whole model at once (one launch per eight tables):
 * tables / indices / biases / heads are HOST arrays of `count` device pointers / head counts; table k is
 * [entries][heads[k]], bias k [heads[k]][pairs].  The tables are parameters, so the gathers of every block can run
 * before the first block of the forward pass (torchvision's shifted_window_attention gathers per block;
 * train/swin_b_tiny.py:95-99 likewise). */
int tch_relpos_bias_gather_batch(tch_context* ctx, const float* const* tables, const int32_t* const* indices,
                                 float* const* biases, const int* heads, int count, int pairs, int entries);

/* The scatter through the inverse of the index, built once by the caller: table entry e receives the pairs
 * list[ptr[e]] .. list[ptr[e + 1] - 1] (pair numbers below `pairs`, ptr non-decreasing, both on the device),
 * summed in list order. */
int tch_relpos_bias_scatter_csr(tch_context* ctx, const float* dbias, const int32_t* ptr, const int32_t* list,
                                float* dtable, int heads, int pairs, int entries, int accumulate);

/* Swin-B data movement (train/swin_b_tiny.py:8-19,116-131; patch merging and shift as in torchvision's swin_b,
 * train/swin_b.py:38).
 * reverse == 0: dst[windows of window x window tokens] = roll(src[B,H,W,C], -shift) partitioned;
 * reverse != 0: dst[B,H,W,C] = roll(un-partitioned src, +shift) (+ add, laid out like dst).  Each direction is
 * also the gradient of the other. */
int tch_window_partition(tch_context* ctx, int dtype, const void* src, void* dst, const void* add, int B, int H, int W,
                         int C, int window, int shift, int reverse);
/* reverse == 0: dst[B,H2,W2,4C] = concat(src[0::2,0::2], src[1::2,0::2], src[0::2,1::2], src[1::2,1::2]) with
 * H2 = (H + 1) / 2, W2 = (W + 1) / 2: an odd side is padded with a zero row / column first;
 * reverse != 0: the inverse permutation (its gradient; what fell on the padding is dropped). */
int tch_patch_merge_gather(tch_context* ctx, int dtype, const void* src, void* dst, int B, int H, int W, int C,
                           int reverse);
/* bias[h, i, j] = table[index[i, j], h] (index int32 [tokens * tokens]); scatter: dtable[e, h] (+)= sum of
 * dbias[h, i, j] over the (i, j) with index[i, j] == e. */
int tch_relpos_bias_gather(tch_context* ctx, const float* table, const int32_t* index, float* bias, int heads,
                           int tokens, int entries);
int tch_relpos_bias_scatter(tch_context* ctx, const float* dbias, const int32_t* index, float* dtable, int heads,
                            int tokens, int entries, int accumulate);
/* out[c] (+)= sum over rows of x[r, c], any width; workspace: tch_column_sum_workspace_floats(rows, cols) floats */
int64_t tch_column_sum_workspace_floats(int rows, int cols);
int tch_column_sum(tch_context* ctx, int dtype, const void* x, float* out, int rows, int cols, int accumulate,
                   float* workspace);

/* ---- layout / precision ---------------------------------------------------------- */
int tch_nchw_to_nhwc_pad(tch_context* ctx, int dtype, const float* x_nchw, void* y_nhwc, int N, int C, int H, int W,
                         int Cpad);
/* dst[C][R*S][K] = src[K][R*S][C] for n_filters filters that live at the same element offsets inside
 * two flat buffers, in ONE launch.  table_dev: device int64[n_filters][5] = {first tile, element offset,
 * K, R*S, C}; a filter owns R*S * ceil(K/32) * ceil(C/32) tiles; total_tiles is their sum.
 * tch_conv2d_dgrad reads filters in this transposed layout. */
int tch_filter_transpose_batched(tch_context* ctx, int dtype, const void* src, void* dst, const int64_t* table_dev,
                                 int n_filters, int64_t total_tiles, int64_t total_elems);
int tch_cast_from_f32(tch_context* ctx, int dtype, const float* src, void* dst, int64_t n);
int tch_cast_to_f32(tch_context* ctx, int dtype, const void* src, float* dst, int64_t n);

#ifdef __cplusplus
}
#endif

#endif /* TORCH_COL_HIP_H_ */
