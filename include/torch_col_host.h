/*
 * torch_col_host.h -- flat C ABI of libtorch_col_hip.so, part 2: the host runtime of the
 * training-side plugin.
 *
 * The reference exposes this surface as C++ classes bound with Cython `cdef extern`
 * (pytorch/torch_col/cython/{main.pyx,dist.pyx,ctrl_stub.pxi}); each function below is the
 * `extern "C"` flattening of one of those externs and cites it.  The Python package
 * sirius_amd.torch_col keeps the reference's Python-visible names on top of these.
 *
 * Conventions: int returns are 0 / a value on success and negative on failure with the
 * message in tch_host_last_error() (thread local) -- the reference aborts the process
 * (CHECK / LOG(FATAL), common/util.h:21-54) where this library reports.  Strings returned
 * as const char* stay valid until the next call on the same thread.
 */
#ifndef TORCH_COL_HOST_H_
#define TORCH_COL_HOST_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* tch_host_last_error(void);

/* ---- init / config (cython/main.pyx:77-172, csrc/init.cc:17-41, csrc/config.cc:49-147) ---- */
/* Reads the COLTRAIN_* environment, then in the reference's boot order: pool (if
 * COLTRAIN_USE_SHARED_TENSOR; use_gpu = 0 builds the CPU model of the pool), inf-tra
 * communicator as client (if COLTRAIN_HAS_INFER_SERVER), intra-train sync segment. */
int tch_TorchColInit(int train_rank, int train_world_size, int use_gpu);
void tch_TorchColShutdown(void);
void tch_TorchColConfig_Reload(int train_rank, int train_world_size); /* tests: re-read the environment */
int tch_TorchColConfig_IsConfigured(void);
int tch_TorchColConfig_IsEnableSharedTensor(void);
int tch_TorchColConfig_IsEnableDynamicSmPartition(void);
int tch_TorchColConfig_IsEnableXsched(void);
int tch_TorchColConfig_KillBatchOnRecv(void);
const char* tch_TorchColConfig_GetColocateCtrlHookMode(void);
const char* tch_TorchColConfig_GetColocateTrainMode(void);
int tch_TorchColConfig_IsReleaseIntermMemoryByGradFn(void);
int tch_TorchColConfig_IsReleaseIntermMemoryByTagging(void);
void tch_TorchColConfig_SetReleaseIntermMemoryByGradFn(int v);
void tch_TorchColConfig_SetReleaseIntermMemoryByTagging(int v);
int tch_TorchColConfig_IsEnableFbwardHook(void);
int tch_TorchColConfig_IsTrainMaster(void);
int tch_TorchColConfig_GetTrainRank(void);
void tch_TorchColConfig_SetTrainRank(int rank);
int tch_TorchColConfig_GetTrainWorldSize(void);
void tch_TorchColConfig_SetTrainWorldSize(int world_size);
int tch_TorchColConfig_HasColocatedInferServer(void);
double tch_TorchColConfig_GetSharedTensorPoolGb(void);
const char* tch_TorchColConfig_GetTrainProfileLogPath(void);

/* ---- HBM pool (cython/main.pyx:228-279; common/cuda_allocator.cc:38-105,259-307) ---- */
/* The process that initialises a pool creates its physical pages and its page table, a shared-memory segment
 * "<prefix>_pages_pool_d<device>" (the PagesPool of common/cuda_allocator.cc:61-73: one pool, every page with
 * its owner, visible to both processes), and serves the pages' dma-buf descriptors to peers.  Page size and
 * unmapping policy of tch_pool_init come from COLTRAIN_POOL_PAGE_MB (default 32, CUDAMemPool::PageNbytes) and
 * COLTRAIN_POOL_LAZY_UNMAP (default 0: FreeTrainLocals unmaps what it hands back); _ex states them. */
int tch_pool_init(int device, uint64_t pool_bytes, int use_gpu);
int tch_pool_init_ex(int device, uint64_t pool_bytes, int use_gpu, uint64_t page_bytes, int lazy_unmap);
void tch_pool_shutdown(int device);
uint64_t tch_pool_page_bytes(int device);
int tch_pool_is_enabled(int device);
/* number of pools this device has had so far: a holder of a pool pointer compares it with the value
 * at allocation time before freeing, so that a pointer into a pool that was shut down is dropped */
uint64_t tch_pool_generation(int device);
uint64_t tch_cuda_memory_pool_infer_usage(int device);
uint64_t tch_cuda_memory_pool_train_usage(int device);
uint64_t tch_cuda_memory_pool_train_peak_usage(int device);
uint64_t tch_cuda_memory_pool_train_all_usage(int device);
uint64_t tch_cuda_memory_pool_free_train_local(int device); /* FreeTrainLocals; returns bytes released */
uint64_t tch_cuda_memory_pool_num_free_pages(int device);
uint64_t tch_cuda_memory_pool_nbytes(int device);
uint64_t tch_cuda_memory_pool_base(int device);
/* allocator hook in the shape torch.cuda.memory.CUDAPluggableAllocator binds
 * (replaces CUDAColAllocator::raw_alloc_with_stream / raw_delete,
 * torch_allocator_plugin.cc:108-178) */
void* tch_pool_malloc(ptrdiff_t nbytes, int device, void* hip_stream);
void tch_pool_free(void* ptr, ptrdiff_t nbytes, int device, void* hip_stream);
void tch_pool_record_stream(void* ptr, int device, void* hip_stream); /* :200-229 */
uint64_t tch_pool_process_events(int device);                          /* :383-412 */
int64_t tch_pool_offset_of(int device, const void* ptr);
/* counters (6 x u64): allocs, frees, driver maps, driver unmaps, slots that got their page back
 * without a driver call, stale mappings currently in place */
void tch_pool_counters(int device, uint64_t* out6);
/* Lazy mode only: FreeTrainLocals relabels pages and leaves their mappings in place (removing a mapping costs
 * the driver 0.26 ms whatever the page size); this removes up to max_pages of those stale mappings and returns
 * how many it removed. */
uint64_t tch_pool_trim(int device, uint64_t max_pages);
uint64_t tch_pool_unmap_calls(int device); /* driver calls behind the unmaps (a run of neighbouring slots is one) */
/* The page table as training sees it: owner_out[i] = 0 free / 1 training / 2 inference, slot_out[i] = the slot
 * (offset / page size) of training's range that physical page i is mapped at, live or stale, or -1.  Returns the
 * number of pages written (at most max_pages).  What the pages pool of the reference keeps per page
 * (common/cuda_allocator.h:48-58), exposed so that a model of the placement can be compared page for page. */
int tch_pool_page_table(int device, uint8_t* owner_out, int64_t* slot_out, int max_pages);
/* The pool from ANOTHER process (the inference side; the TVM-side allocator over the same PagesPool,
 * common/cuda_allocator.cc:86-99): attach to the page table, claim FREE pages (lowest index first; returns how
 * many, indices in pages_out), map a claimed page (its device address in this process; the descriptor comes from
 * the pool's creator, who hands it only to the page's owner), unmap, give pages back (still-mapped ones are
 * unmapped first), detach (gives back whatever is still owned). */
int tch_pool_peer_attach(int device);
void tch_pool_peer_detach(int device);
int tch_pool_peer_num_pages(int device);
uint64_t tch_pool_peer_page_bytes(int device);
int tch_pool_peer_free_pages(int device);
int tch_pool_peer_claim(int device, int n, int* pages_out);
int tch_pool_peer_release(int device, const int* pages, int n);
void* tch_pool_peer_map(int device, int page);
/* A pool in lazy mode answers the other tenant first and removes its own mappings of the pages it handed back right
 * after the reply (the driver takes 0.26 ms per mapping, one after the other, from however many threads): such a
 * page is FREE and claimable at once, and flagged in the page table until its old mapping is gone.
 * tch_pool_peer_map waits up to 5 s for the flag of the page it maps (tch_pool_peer_map_wait: up to wait_ms), so a
 * page is never usable by two processes at once; tch_pool_peer_still_mapped counts the flagged ones among `pages`. */
void* tch_pool_peer_map_wait(int device, int page, int wait_ms);
int tch_pool_peer_still_mapped(int device, const int* pages, int n);
int tch_pool_peer_unmap(int device, int page);
/* the inference side inside the training process (a stand-in peer on a thread): label n FREE pages
 * inference-owned / give back */
int tch_pool_infer_claim_pages(int device, int n);
int tch_pool_infer_release_pages(int device, int n);
void tch_tag_model_start(int device);       /* main.pyx tag_model_start */
void tch_tag_model_end(int device);         /* main.pyx tag_model_end */
int tch_tag_interm_memory(int device, void* ptr);      /* TagIntermMemory :322-341 */
uint64_t tch_release_interm_memory(int device);        /* ReleaseIntermMemory :343-369 */
void tch_untag_interm_memory(int device);              /* UntagIntermMemory */
/* fn(arg) is called by FreeTrainLocals before the pool takes any lock and before it waits for the device: where a
 * runtime that holds launches in queues of its own hands them over and waits for them, so that nothing submitted
 * earlier can touch a page after it has changed hands.  (The launch queues of this library are drained by the
 * pool itself.)  fn may call back into the pool.  NULL removes the hook.  Same role as the synchronisation the
 * reference does before FreeTrainLocals (pytorch/torch_col/csrc/torch_allocator_plugin.cc:383-412). */
void tch_pool_set_quiesce_hook(int device, void (*fn)(void*), void* arg);
/* CPU model only: let the first n recorded events count as finished */
void tch_pool_null_backend_complete_events(int device, uint64_t upto);
/* CPU model only: the nth mapping from now is refused by the "driver" (0: none) */
void tch_pool_null_backend_fail_map_in(int device, int nth);
/* CPU model only: 0 = mapped slots that never got access rights, 1 = quiesce calls, 2 = access-right calls */
int64_t tch_pool_null_backend_probe(int device, int what);

/* ---- inference <-> training communicator (cython/main.pyx:346-528) ---- */
typedef struct tch_ctrl_msg {
  uint64_t id;
  int event; /* CtrlEvent 0..12, common/inf_tra_comm/message_queue.h:18-40 */
  int value;
} tch_ctrl_msg;
int tch_InfTraCommunicator_Init(int is_server, int cleanup, int train_world_size);
void tch_InfTraCommunicator_Shutdown(void);
int tch_InfTraCommunicator_IsInitialized(void);
/* direction: 0 = inf2tra, 1 = tra2inf */
int tch_mq_put(int direction, int id, const tch_ctrl_msg* msg);
int tch_mq_put_all(int direction, const tch_ctrl_msg* msg);
int tch_mq_put_all_vec(int direction, const tch_ctrl_msg* msgs, int n);
int tch_mq_block_get(int direction, int id, tch_ctrl_msg* out);
int tch_mq_try_get(int direction, int id, tch_ctrl_msg* out);                       /* 1 got, 0 empty */
int tch_mq_timed_get(int direction, int id, uint32_t timeout_ms, tch_ctrl_msg* out); /* 1 got, 0 timeout */
int tch_mq_timed_get_from_any(int direction, uint32_t timeout_ms, int* id, tch_ctrl_msg* out);
void tch_mq_clear(void);
/* information board (common/inf_tra_comm/shared_info.h:21-35, shared_info.cc:54-108) */
int tch_init_train_info(int init_batch_size, int current_batch_size, const char* model_name); /* main.pyx:485-515 */
int tch_update_current_batch_size(int batch_size);
/* field: 0 pid, 1 rank, 2 world size, 3 init bs, 4 current bs, 5 target bs, 6 target bs unpublished, 7 first epoch done */
int tch_train_info_get_field(int id, int field);
int tch_train_info_set_field(int id, int field, int value);
/* Compute units the inference side wants on `device` (shared-memory board; the reference's
 * SMPartitioner::Set/Add/Dec/GetInferRequiredTpcNum, common/sm_partition.cc:60-76).  add returns the new value. */
int tch_infer_required_cus_get(int device);
int tch_infer_required_cus_set(int device, int n);
int tch_infer_required_cus_add(int device, int delta);
int tch_train_info_is_valid(int id);
int tch_train_info_model_name(int id, char* out, int cap);

/* ---- control stubs (cython/ctrl_stub.pxi:69-231; csrc/control_stub.{h,cc}) ---- */
typedef struct tch_stub tch_stub;
/* kind: 0 Dummy, 1 Switch, 2 Colocate (batch_size only used by Colocate) */
tch_stub* tch_stub_create(int kind, int batch_size);
void tch_stub_destroy(tch_stub* s);
void tch_stub_stop(tch_stub* s);
int tch_stub_cmd(tch_stub* s);
void tch_stub_set_cmd(tch_stub* s, int cmd);
void tch_stub_train_start(tch_stub* s);
void tch_stub_train_end(tch_stub* s);
void tch_stub_report_batch_size(tch_stub* s, int batch_size);
void tch_stub_StepsNoInteruptBegin(tch_stub* s);
void tch_stub_StepsNoInteruptEnd(tch_stub* s);
int tch_stub_can_exit_after_infer_worklaod_done(tch_stub* s); /* sic, ctrl_stub.pxi */
void tch_stub_set_train_first_epoch_done(tch_stub* s);
const char* tch_stub_last_error(tch_stub* s);
int tch_stub_process_msg(tch_stub* s, const tch_ctrl_msg* msg); /* deliver one message synchronously */
/* Colocate */
int tch_stub_target_batch_size(tch_stub* s);
int tch_stub_unpub_target_batch_size(tch_stub* s);
void tch_stub_adjust_l1_done(tch_stub* s);
void tch_stub_adjust_l2_done(tch_stub* s);
double tch_stub_passed_time_from_set_cmd(tch_stub* s);
void tch_stub_set_killed_batch_recover(tch_stub* s);
void tch_stub_set_killed_batch_reconfiged(tch_stub* s);
/* Switch */
int tch_stub_try_interrupt_train_done(tch_stub* s, int barrier);
void tch_stub_train_resume_done(tch_stub* s);
int tch_stub_prepare_resume(tch_stub* s);
void tch_stub_set_global_interrupt_flag(tch_stub* s, int flag);
int tch_stub_get_global_interrupt_flag(tch_stub* s);
void tch_stub_set_global_has_batch_killed(tch_stub* s, int flag);
int tch_stub_get_global_has_batch_killed(tch_stub* s);
/* StubProfiler (control_stub.cc:642-652): copies up to cap timestamps (us), returns the count */
int tch_get_adjust_request_time_stamp(int64_t* out, int cap);
int tch_get_adjust_done_time_stamp(int64_t* out, int cap);

/* ---- intra-train sync, batch distributor, perf model (cython/dist.pyx:25-193) ---- */
int tch_DistTrainSync_Init(int rank, int world_size);
void tch_wait_barrier(void);
int tch_send_msg(int dst, const char* msg, int len);
int tch_recv_msg(int src, char* out, int cap); /* returns the length, or -needed if cap is too small */
/* csrc/dynamic_batch.cc:40-65 */
int tch_init_dynamic_batch_distributor(int dataset_size, int batch_size, int global_batch_size, int lazy,
                                       const char* policy);
void tch_shutdown_dynamic_batch_distributor(void);
/* ranges_out: 2*cap ints (lo, hi pairs); returns the number of ranges, *last_micro_batch set */
int tch_distributor_get_batch(int batch_size, int* ranges_out, int cap, int* last_micro_batch);
int tch_distributor_query_next_batch_size(int batch_size);
int tch_distributor_finish_batch(const int* ranges, int n, int end_of_global_batch);
int tch_distributor_abort_batch(const int* ranges, int n, int end_of_global_batch);
int tch_distributor_vote_finish_last_micro_batch(void);
void tch_distributor_vote_abort_last_micro_batch(void);
void tch_distributor_reset_last_micro_batch_finish_vote(void);
void tch_distributor_distribute_batch(int check_num_unproced_samples, int distribute_to_all, int at_global_batch_begin);
int tch_distributor_next_epoch(void);
void tch_distributor_next_global_batch(void);
int tch_distributor_get_global_batch_size(void);
int tch_distributor_get_num_global_batch_per_epoch(void);
int tch_distributor_get_num_proced_global_batch(void);
int tch_distributor_snapshot(int which, int* ranges_out, int cap); /* 0 unproc, 1 procing, 2 proced */
int tch_distributor_counters(int* out, int cap);
/* csrc/perf_model.cc:25-94 */
void tch_perf_model_record_thpt(int batch_size, double batch_time_ms);
double tch_perf_model_get_thpt(int batch_size);
void tch_perf_model_get_thpt_vec(const int* batch_sizes, int n, double* out);
void tch_perf_model_clear(void);

/* ---- util (cython/main.pyx:534-567) ---- */
int64_t tch_get_unix_timestamp(void);
int64_t tch_get_unix_timestamp_us(void);

#ifdef __cplusplus
}
#endif

#endif /* TORCH_COL_HOST_H_ */
