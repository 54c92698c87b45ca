// Flat C ABI over the host runtime (config, HBM pool, communicator, stubs, batch distributor,
// perf model).  Nothing here aborts the process: failures return a negative value and leave
// a message for tch_host_last_error().
#include "../../../include/torch_col_host.h"

#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <mutex>

#include <string>

#include "config.h"
#include "control_stub.h"
#include "dist_train.h"
#include "inf_tra_comm.h"
#include "mem_pool.h"

using namespace tch::host;

namespace {
thread_local std::string g_err;
thread_local std::string g_str;

int fail(const std::string& msg, int code = -1) {
  g_err = msg;
  return code;
}
const char* keep(const std::string& s) {
  g_str = s;
  return g_str.c_str();
}
CtrlMsgEntry to_msg(const tch_ctrl_msg* m) { return CtrlMsgEntry{m->id, m->event, m->value}; }
void from_msg(const CtrlMsgEntry& m, tch_ctrl_msg* out) {
  out->id = m.id;
  out->event = m.event;
  out->value = m.value;
}
bool dir_ok(int d) { return d == kInf2Tra || d == kTra2Inf; }
}  // namespace

namespace {
PoolOptions options_from_env() {
  PoolOptions o;
  if (const char* e = getenv("COLTRAIN_POOL_PAGE_MB"))
    if (atoi(e) > 0) o.page_bytes = static_cast<size_t>(atoi(e)) << 20;
  if (const char* e = getenv("COLTRAIN_POOL_LAZY_UNMAP")) o.lazy_unmap = atoi(e) != 0;
  return o;
}
std::mutex g_peer_mu;
std::shared_ptr<PoolPeer> g_peers[kMaxDeviceNum];
std::shared_ptr<PoolPeer> peer(int device) {
  if (device < 0 || device >= kMaxDeviceNum) return nullptr;
  std::lock_guard<std::mutex> l(g_peer_mu);
  return g_peers[device];
}
}  // namespace

struct tch_stub {
  int kind;
  std::unique_ptr<StubBase> stub;
  ColocateStub* colocate() { return kind == 2 ? static_cast<ColocateStub*>(stub.get()) : nullptr; }
  SwitchStub* sw() { return kind == 1 ? static_cast<SwitchStub*>(stub.get()) : nullptr; }
};

extern "C" {

const char* tch_host_last_error(void) { return g_err.c_str(); }

// ---------------------------------------------------------------------------
int tch_TorchColInit(int train_rank, int train_world_size, int use_gpu) {
  if (train_rank < 0 || train_world_size <= 0 || train_rank >= train_world_size)
    return fail("torch_col_init: need 0 <= rank < world size");
  init_config(train_rank, train_world_size, false);
  Config& c = config();
  std::string err;
  // one pool per device; a rank trains on the device of its own index (init.cc:23-28)
  if (c.use_shared_tensor && !pool(train_rank)) {
    const size_t bytes = static_cast<size_t>(c.shared_tensor_pool_gb * (1ull << 30));
    if (!pool_init(train_rank, bytes, use_gpu != 0, options_from_env(), &err)) return fail("pool init: " + err);
  }
  if (c.has_colocated_infer_server && !communicator()) {
    if (!communicator_init(false, false, train_world_size, &err)) return fail("communicator init: " + err);
  }
  if (!DistTrainSync::initialized()) {
    if (!DistTrainSync::init(train_rank, train_world_size, &err)) return fail("dist train sync init: " + err);
  }
  return 0;
}

void tch_TorchColShutdown(void) {
  StubBase::stop_all();
  StubProfiler::clear();
  DynamicBatchDistributor::shutdown();
  DistTrainSync::shutdown();
  communicator_shutdown();
  for (int d = 0; d < kMaxDeviceNum; ++d) pool_shutdown(d);
  config().configured = false;
}

void tch_TorchColConfig_Reload(int train_rank, int train_world_size) { init_config(train_rank, train_world_size, true); }
int tch_TorchColConfig_IsConfigured(void) { return config().configured; }
int tch_TorchColConfig_IsEnableSharedTensor(void) { return config().use_shared_tensor; }
int tch_TorchColConfig_IsEnableDynamicSmPartition(void) { return config().dynamic_sm_partition; }
int tch_TorchColConfig_IsEnableXsched(void) { return config().colocate_use_xsched; }
int tch_TorchColConfig_KillBatchOnRecv(void) { return config().kill_batch_on_recv; }
const char* tch_TorchColConfig_GetColocateCtrlHookMode(void) { return config().colocate_ctrl_hook_mode.c_str(); }
const char* tch_TorchColConfig_GetColocateTrainMode(void) { return config().colocate_train_mode.c_str(); }
int tch_TorchColConfig_IsReleaseIntermMemoryByGradFn(void) { return config().release_interm_memory_by_grad_fn; }
int tch_TorchColConfig_IsReleaseIntermMemoryByTagging(void) { return config().release_interm_memory_by_tagging; }
void tch_TorchColConfig_SetReleaseIntermMemoryByGradFn(int v) { config().release_interm_memory_by_grad_fn = v != 0; }
void tch_TorchColConfig_SetReleaseIntermMemoryByTagging(int v) { config().release_interm_memory_by_tagging = v != 0; }
int tch_TorchColConfig_IsEnableFbwardHook(void) { return config().use_fbward_hook; }
int tch_TorchColConfig_IsTrainMaster(void) { return config().train_rank == 0; }
int tch_TorchColConfig_GetTrainRank(void) { return config().train_rank; }
void tch_TorchColConfig_SetTrainRank(int rank) { config().train_rank = rank; }
int tch_TorchColConfig_GetTrainWorldSize(void) { return config().train_world_size; }
void tch_TorchColConfig_SetTrainWorldSize(int w) { config().train_world_size = w; }
int tch_TorchColConfig_HasColocatedInferServer(void) { return config().has_colocated_infer_server; }
double tch_TorchColConfig_GetSharedTensorPoolGb(void) { return config().shared_tensor_pool_gb; }
const char* tch_TorchColConfig_GetTrainProfileLogPath(void) { return config().train_profile_log_path.c_str(); }

// ---------------------------------------------------------------------------
int tch_pool_init(int device, uint64_t pool_bytes, int use_gpu) {
  std::string err;
  if (!pool_init(device, pool_bytes, use_gpu != 0, options_from_env(), &err)) return fail(err);
  return 0;
}
int tch_pool_init_ex(int device, uint64_t pool_bytes, int use_gpu, uint64_t page_bytes, int lazy_unmap) {
  std::string err;
  PoolOptions o;
  if (page_bytes) o.page_bytes = page_bytes;
  o.lazy_unmap = lazy_unmap != 0;
  if (!pool_init(device, pool_bytes, use_gpu != 0, o, &err)) return fail(err);
  return 0;
}
void tch_pool_shutdown(int device) { pool_shutdown(device); }
int tch_pool_is_enabled(int device) { return pool(device) != nullptr; }
uint64_t tch_pool_generation(int device) { return pool_generation(device); }
uint64_t tch_pool_page_bytes(int d) { auto p = pool(d); return p ? p->page_bytes() : 0; }
uint64_t tch_cuda_memory_pool_infer_usage(int d) { auto p = pool(d); return p ? p->stats().infer_usage : 0; }
uint64_t tch_cuda_memory_pool_train_usage(int d) { auto p = pool(d); return p ? p->stats().train_usage : 0; }
uint64_t tch_cuda_memory_pool_train_peak_usage(int d) { auto p = pool(d); return p ? p->stats().train_peak_usage : 0; }
uint64_t tch_cuda_memory_pool_train_all_usage(int d) { auto p = pool(d); return p ? p->stats().train_all_usage : 0; }
uint64_t tch_cuda_memory_pool_free_train_local(int d) { auto p = pool(d); return p ? p->empty_cache() : 0; }
uint64_t tch_cuda_memory_pool_num_free_pages(int d) { auto p = pool(d); return p ? p->stats().free_pages : 0; }
uint64_t tch_cuda_memory_pool_nbytes(int d) { auto p = pool(d); return p ? p->stats().pool_bytes : 0; }
uint64_t tch_cuda_memory_pool_base(int d) { auto p = pool(d); return p ? p->base() : 0; }

void* tch_pool_malloc(ptrdiff_t nbytes, int device, void* hip_stream) {
  auto p = pool(device);
  if (!p) {
    fail("tch_pool_malloc: pool not initialised for this device");
    return nullptr;
  }
  if (nbytes <= 0) return nullptr;
  p->process_events();
  std::string err;
  void* ptr = p->alloc(static_cast<size_t>(nbytes), reinterpret_cast<uint64_t>(hip_stream), &err);
  if (!ptr) fail(err);
  return ptr;
}

void tch_pool_free(void* ptr, ptrdiff_t, int device, void*) {
  auto p = pool(device);
  if (!p || !ptr) return;
  std::string err;
  if (!p->free(ptr, &err)) fail(err);
}

void tch_pool_record_stream(void* ptr, int device, void* hip_stream) {
  if (auto p = pool(device)) p->record_stream(ptr, reinterpret_cast<uint64_t>(hip_stream));
}
uint64_t tch_pool_process_events(int device) { auto p = pool(device); return p ? p->process_events() : 0; }
int64_t tch_pool_offset_of(int device, const void* ptr) { auto p = pool(device); return p ? p->offset_of(ptr) : -1; }
void tch_pool_counters(int device, uint64_t* out6) {
  if (!out6) return;
  PoolStats s{};
  if (auto p = pool(device)) s = p->stats();
  out6[0] = s.num_allocs;
  out6[1] = s.num_frees;
  out6[2] = s.num_maps;
  out6[3] = s.num_unmaps;
  out6[4] = s.num_revives;
  out6[5] = s.stale_pages;
}
int tch_pool_page_table(int device, uint8_t* owner_out, int64_t* slot_out, int max_pages) {
  auto p = pool(device);
  return p ? p->page_table(owner_out, slot_out, max_pages) : 0;
}
uint64_t tch_pool_unmap_calls(int device) { auto p = pool(device); return p ? p->stats().num_unmap_calls : 0; }
uint64_t tch_pool_trim(int device, uint64_t max_pages) { auto p = pool(device); return p ? p->trim(max_pages) : 0; }
int tch_pool_infer_claim_pages(int d, int n) { auto p = pool(d); return p ? p->infer_claim_pages(n) : 0; }
int tch_pool_infer_release_pages(int d, int n) { auto p = pool(d); return p ? p->infer_release_pages(n) : 0; }
void tch_tag_model_start(int d) { if (auto p = pool(d)) p->tag_model_start(); }
void tch_tag_model_end(int d) { if (auto p = pool(d)) p->tag_model_end(); }
int tch_tag_interm_memory(int d, void* ptr) { auto p = pool(d); return p && p->tag_interm_memory(ptr) ? 1 : 0; }
uint64_t tch_release_interm_memory(int d) { auto p = pool(d); return p ? p->release_interm_memory() : 0; }
void tch_untag_interm_memory(int d) { if (auto p = pool(d)) p->untag_interm_memory(); }
void tch_pool_set_quiesce_hook(int d, void (*fn)(void*), void* arg) {
  auto p = pool(d);
  if (!p) return;
  if (fn)
    p->set_quiesce_hook([fn, arg] { fn(arg); });
  else
    p->set_quiesce_hook(nullptr);
}
void tch_pool_null_backend_fail_map_in(int d, int nth) {
  auto p = pool(d);
  if (!p) return;
  if (auto* nb = dynamic_cast<NullBackend*>(p->backend())) nb->fail_map_in = nth;
}
int64_t tch_pool_null_backend_probe(int d, int what) {
  auto p = pool(d);
  if (!p) return -1;
  auto* nb = dynamic_cast<NullBackend*>(p->backend());
  if (!nb) return -1;
  switch (what) {
    case 0: return static_cast<int64_t>(nb->no_access.size());
    case 1: return nb->quiesces;
    case 2: return nb->access_calls;
    default: return -1;
  }
}
void tch_pool_null_backend_complete_events(int d, uint64_t upto) {
  auto p = pool(d);
  if (!p) return;
  if (auto* nb = dynamic_cast<NullBackend*>(p->backend())) nb->completed_upto = upto;
}

// ---- the pool as another process sees it ----
int tch_pool_peer_attach(int device) {
  if (device < 0 || device >= kMaxDeviceNum) return fail("bad device");
  std::lock_guard<std::mutex> l(g_peer_mu);
  if (g_peers[device]) return fail("this process is already attached to the pool of this device");
  std::string err;
  g_peers[device].reset(PoolPeer::attach(device, &err));
  return g_peers[device] ? 0 : fail("tch_pool_peer_attach: " + err);
}
void tch_pool_peer_detach(int device) {
  std::shared_ptr<PoolPeer> last;
  std::lock_guard<std::mutex> l(g_peer_mu);
  if (device >= 0 && device < kMaxDeviceNum) last.swap(g_peers[device]);
}
int tch_pool_peer_num_pages(int device) { auto p = peer(device); return p ? p->num_pages() : fail("not attached"); }
uint64_t tch_pool_peer_page_bytes(int device) { auto p = peer(device); return p ? p->page_bytes() : 0; }
int tch_pool_peer_free_pages(int device) { auto p = peer(device); return p ? p->free_pages() : fail("not attached"); }
int tch_pool_peer_claim(int device, int n, int* pages_out) {
  auto p = peer(device);
  if (!p) return fail("tch_pool_peer_claim: not attached");
  if (n < 0) return fail("tch_pool_peer_claim: negative page count");
  return p->claim(n, pages_out);
}
int tch_pool_peer_release(int device, const int* pages, int n) {
  auto p = peer(device);
  if (!p) return fail("tch_pool_peer_release: not attached");
  if (!pages || n < 0) return fail("tch_pool_peer_release: bad arguments");
  return p->release(pages, n);
}
void* tch_pool_peer_map(int device, int page) {
  auto p = peer(device);
  if (!p) {
    fail("tch_pool_peer_map: not attached");
    return nullptr;
  }
  std::string err;
  void* ptr = p->map(page, &err);
  if (!ptr) fail("tch_pool_peer_map: " + err);
  return ptr;
}
void* tch_pool_peer_map_wait(int device, int page, int wait_ms) {
  auto p = peer(device);
  if (!p) {
    fail("tch_pool_peer_map_wait: not attached");
    return nullptr;
  }
  std::string err;
  void* ptr = p->map(page, &err, wait_ms);
  if (!ptr) fail("tch_pool_peer_map_wait: " + err);
  return ptr;
}
int tch_pool_peer_still_mapped(int device, const int* pages, int n) {
  auto p = peer(device);
  if (!p) return fail("tch_pool_peer_still_mapped: not attached");
  return p->still_mapped_by_creator(pages, n);
}
int tch_pool_peer_unmap(int device, int page) {
  auto p = peer(device);
  if (!p) return fail("tch_pool_peer_unmap: not attached");
  std::string err;
  return p->unmap(page, &err) ? 0 : fail("tch_pool_peer_unmap: " + err);
}

// ---------------------------------------------------------------------------
int tch_InfTraCommunicator_Init(int is_server, int cleanup, int world) {
  std::string err;
  if (!communicator_init(is_server != 0, cleanup != 0, world, &err)) return fail(err);
  return 0;
}
void tch_InfTraCommunicator_Shutdown(void) {
  StubBase::stop_all();
  communicator_shutdown();
}
int tch_InfTraCommunicator_IsInitialized(void) { return communicator() != nullptr; }

// one counted reference for the whole entry point: the segment stays mapped until it returns, also when another
// thread shuts the communicator down meanwhile
#define NEED_COMM()            \
  auto comm = communicator();  \
  if (!comm) return fail("InfTraCommunicator has not been initialized")

int tch_mq_put(int d, int id, const tch_ctrl_msg* msg) {
  NEED_COMM();
  if (!dir_ok(d) || !msg) return fail("tch_mq_put: bad arguments");
  return comm->put(to_msg(msg), static_cast<Direction>(d), id) ? 0 : fail("tch_mq_put: bad rank");
}
int tch_mq_put_all(int d, const tch_ctrl_msg* msg) {
  NEED_COMM();
  if (!dir_ok(d) || !msg) return fail("tch_mq_put_all: bad arguments");
  comm->put_all(to_msg(msg), static_cast<Direction>(d));
  return 0;
}
int tch_mq_put_all_vec(int d, const tch_ctrl_msg* msgs, int n) {
  NEED_COMM();
  if (!dir_ok(d) || !msgs) return fail("tch_mq_put_all_vec: bad arguments");
  std::vector<CtrlMsgEntry> v;
  for (int i = 0; i < n; ++i) v.push_back(to_msg(&msgs[i]));
  return comm->put_all(v, static_cast<Direction>(d)) ? 0 : fail("one message per training rank is required");
}
int tch_mq_block_get(int d, int id, tch_ctrl_msg* out) {
  NEED_COMM();
  if (!dir_ok(d) || !out || id < 0 || id >= comm->world_size()) return fail("tch_mq_block_get: bad arguments");
  from_msg(comm->block_get(static_cast<Direction>(d), id), out);
  return 0;
}
int tch_mq_try_get(int d, int id, tch_ctrl_msg* out) {
  NEED_COMM();
  if (!dir_ok(d) || !out || id < 0 || id >= comm->world_size()) return fail("tch_mq_try_get: bad arguments");
  CtrlMsgEntry m;
  if (!comm->try_get(static_cast<Direction>(d), id, &m)) return 0;
  from_msg(m, out);
  return 1;
}
int tch_mq_timed_get(int d, int id, uint32_t timeout_ms, tch_ctrl_msg* out) {
  NEED_COMM();
  if (!dir_ok(d) || !out || id < 0 || id >= comm->world_size()) return fail("tch_mq_timed_get: bad arguments");
  CtrlMsgEntry m;
  if (!comm->timed_get(timeout_ms, static_cast<Direction>(d), id, &m)) return 0;
  from_msg(m, out);
  return 1;
}
int tch_mq_timed_get_from_any(int d, uint32_t timeout_ms, int* id, tch_ctrl_msg* out) {
  NEED_COMM();
  if (!dir_ok(d) || !out || !id) return fail("tch_mq_timed_get_from_any: bad arguments");
  CtrlMsgEntry m;
  if (!comm->timed_get_from_any(timeout_ms, static_cast<Direction>(d), id, &m)) return 0;
  from_msg(m, out);
  return 1;
}
void tch_mq_clear(void) { if (auto comm = communicator()) comm->clear(); }

int tch_init_train_info(int init_bs, int cur_bs, const char* model_name) {
  if (!config().has_colocated_infer_server) return 0;  // nothing to publish to (main.pyx:485-515)
  NEED_COMM();
  pid_t pid = getpid();
  int rank = config().train_rank, world = config().train_world_size;
  if (!comm->set_train_info(rank, &pid, &rank, &world, &init_bs, &cur_bs, model_name))
    return fail("init_train_info: board slot rejected the update");
  return 0;
}
int tch_update_current_batch_size(int bs) {
  if (!config().has_colocated_infer_server) return 0;
  NEED_COMM();
  comm->update_field(config().train_rank, kFieldCurrentBatchSize, bs);
  return 0;
}
int tch_train_info_get_field(int id, int field) {
  NEED_COMM();
  if (id < 0 || id >= kMaxDeviceNum || field < 0 || field > kFieldFirstEpochDone) return fail("bad board slot or field");
  return comm->get_field(id, static_cast<TrainInfoField>(field));
}
int tch_train_info_set_field(int id, int field, int value) {
  NEED_COMM();
  if (id < 0 || id >= kMaxDeviceNum || field < 0 || field > kFieldFirstEpochDone) return fail("bad board slot or field");
  comm->update_field(id, static_cast<TrainInfoField>(field), value);
  return 0;
}
int tch_infer_required_cus_get(int device) {
  NEED_COMM();
  if (device < 0 || device >= kMaxDeviceNum) return fail("bad device");
  return comm->infer_required_cus(device);
}
int tch_infer_required_cus_set(int device, int n) {
  NEED_COMM();
  if (device < 0 || device >= kMaxDeviceNum || n < 0) return fail("bad device or compute-unit count");
  comm->set_infer_required_cus(device, n);
  return 0;
}
int tch_infer_required_cus_add(int device, int delta) {
  NEED_COMM();
  if (device < 0 || device >= kMaxDeviceNum) return fail("bad device");
  return comm->add_infer_required_cus(device, delta);
}
int tch_train_info_is_valid(int id) {
  NEED_COMM();
  if (id < 0 || id >= kMaxDeviceNum) return fail("bad board slot");
  return comm->train_info_valid(id) ? 1 : 0;
}
int tch_train_info_model_name(int id, char* out, int cap) {
  NEED_COMM();
  if (id < 0 || id >= kMaxDeviceNum || !out || cap < 1) return fail("bad arguments");
  TrainInfo t = comm->get_train_info(id);
  strncpy(out, t.model_name, cap - 1);
  out[cap - 1] = 0;
  return static_cast<int>(strlen(out));
}

// ---------------------------------------------------------------------------
tch_stub* tch_stub_create(int kind, int batch_size) {
  auto* s = new tch_stub();
  s->kind = kind;
  if (kind == 0) s->stub.reset(new DummyStub());
  else if (kind == 1) s->stub.reset(new SwitchStub());
  else if (kind == 2) s->stub.reset(new ColocateStub(batch_size));
  else {
    delete s;
    fail("tch_stub_create: kind must be 0 (Dummy), 1 (Switch) or 2 (Colocate)");
    return nullptr;
  }
  s->stub->start();
  return s;
}
void tch_stub_destroy(tch_stub* s) {
  // the control thread calls into the derived class: it has to be gone before any destructor runs
  if (s && s->stub) s->stub->stop();
  delete s;
}
void tch_stub_stop(tch_stub* s) { if (s) s->stub->stop(); }
int tch_stub_cmd(tch_stub* s) { return s ? s->stub->cmd() : -1; }
void tch_stub_set_cmd(tch_stub* s, int cmd) { if (s) s->stub->set_cmd(cmd); }
void tch_stub_train_start(tch_stub* s) { if (s) s->stub->train_start(); }
void tch_stub_train_end(tch_stub* s) { if (s) s->stub->train_end(); }
void tch_stub_report_batch_size(tch_stub* s, int bs) { if (s) s->stub->report_batch_size(bs); }
void tch_stub_StepsNoInteruptBegin(tch_stub* s) { if (s) s->stub->steps_no_interrupt_begin(); }
void tch_stub_StepsNoInteruptEnd(tch_stub* s) { if (s) s->stub->steps_no_interrupt_end(); }
int tch_stub_can_exit_after_infer_worklaod_done(tch_stub* s) { return s && s->stub->can_exit_after_infer_workload_done(); }
void tch_stub_set_train_first_epoch_done(tch_stub* s) { if (s) s->stub->set_train_first_epoch_done(); }
const char* tch_stub_last_error(tch_stub* s) { return s ? keep(s->stub->last_error()) : ""; }
int tch_stub_process_msg(tch_stub* s, const tch_ctrl_msg* msg) {
  if (!s || !msg) return fail("tch_stub_process_msg: null argument");
  const std::string before = s->stub->last_error();
  s->stub->process(to_msg(msg));
  if (s->stub->last_error() != before) return fail(s->stub->last_error());
  return 0;
}
int tch_stub_target_batch_size(tch_stub* s) { return s && s->colocate() ? s->colocate()->target_batch_size() : fail("not a colocate stub"); }
int tch_stub_unpub_target_batch_size(tch_stub* s) { return s && s->colocate() ? s->colocate()->unpub_target_batch_size() : fail("not a colocate stub"); }
void tch_stub_adjust_l1_done(tch_stub* s) { if (s && s->colocate()) s->colocate()->adjust_l1_done(); }
void tch_stub_adjust_l2_done(tch_stub* s) { if (s && s->colocate()) s->colocate()->adjust_l2_done(); }
double tch_stub_passed_time_from_set_cmd(tch_stub* s) { return s && s->colocate() ? s->colocate()->passed_time_from_set_cmd_ms() : 0.0; }
void tch_stub_set_killed_batch_recover(tch_stub* s) {
  if (!s) return;
  if (s->colocate()) s->colocate()->set_killed_batch_recover();
  if (s->sw()) s->sw()->set_killed_batch_recover();
}
void tch_stub_set_killed_batch_reconfiged(tch_stub* s) { if (s && s->colocate()) s->colocate()->set_killed_batch_reconfiged(); }
int tch_stub_try_interrupt_train_done(tch_stub* s, int barrier) { return s && s->sw() && s->sw()->try_interrupt_train_done(barrier != 0); }
void tch_stub_train_resume_done(tch_stub* s) { if (s && s->sw()) s->sw()->train_resume_done(); }
int tch_stub_prepare_resume(tch_stub* s) { return s && s->sw() && s->sw()->prepare_resume(); }
void tch_stub_set_global_interrupt_flag(tch_stub* s, int f) { if (s && s->sw()) s->sw()->set_global_interrupt_flag(f != 0); }
int tch_stub_get_global_interrupt_flag(tch_stub* s) { return s && s->sw() && s->sw()->global_interrupt_flag(); }
void tch_stub_set_global_has_batch_killed(tch_stub* s, int f) { if (s && s->sw()) s->sw()->set_global_has_batch_killed(f != 0); }
int tch_stub_get_global_has_batch_killed(tch_stub* s) { return s && s->sw() && s->sw()->global_has_batch_killed(); }

int tch_get_adjust_request_time_stamp(int64_t* out, int cap) {
  auto v = StubProfiler::adjust_request_time_stamps();
  for (int i = 0; i < cap && i < static_cast<int>(v.size()); ++i) out[i] = v[i];
  return static_cast<int>(v.size());
}
int tch_get_adjust_done_time_stamp(int64_t* out, int cap) {
  auto v = StubProfiler::adjust_done_time_stamps();
  for (int i = 0; i < cap && i < static_cast<int>(v.size()); ++i) out[i] = v[i];
  return static_cast<int>(v.size());
}

// ---------------------------------------------------------------------------
int tch_DistTrainSync_Init(int rank, int world) {
  std::string err;
  if (!DistTrainSync::init(rank, world, &err)) return fail(err);
  return 0;
}
void tch_wait_barrier(void) { DistTrainSync::wait_barrier(); }
int tch_send_msg(int dst, const char* msg, int len) {
  if (!DistTrainSync::initialized() || dst < 0 || dst >= DistTrainSync::world_size() || !msg || len < 0)
    return fail("tch_send_msg: bad arguments or sync segment missing");
  DistTrainSync::send(dst, std::string(msg, len));
  return 0;
}
int tch_recv_msg(int src, char* out, int cap) {
  static thread_local std::string pending;
  static thread_local bool has_pending = false;
  if (!DistTrainSync::initialized() || src < 0 || src >= DistTrainSync::world_size() || !out)
    return fail("tch_recv_msg: bad arguments or sync segment missing");
  if (!has_pending) {
    pending = DistTrainSync::recv(src);
    has_pending = true;
  }
  if (static_cast<int>(pending.size()) > cap) return -static_cast<int>(pending.size());  // call again with room
  memcpy(out, pending.data(), pending.size());
  has_pending = false;
  return static_cast<int>(pending.size());
}

#define NEED_DIST() \
  if (!DynamicBatchDistributor::get()) return fail("batch distributor has not been initialized")

int tch_init_dynamic_batch_distributor(int ds, int bs, int gbs, int lazy, const char* policy) {
  std::string err;
  if (!DynamicBatchDistributor::init(ds, bs, gbs, lazy != 0, policy ? policy : "simple", &err)) return fail(err);
  return 0;
}
void tch_shutdown_dynamic_batch_distributor(void) { DynamicBatchDistributor::shutdown(); }
int tch_distributor_get_batch(int batch_size, int* ranges_out, int cap, int* last) {
  NEED_DIST();
  std::string err;
  auto res = DynamicBatchDistributor::get()->get_batch(batch_size, &err);
  if (!err.empty()) return fail(err);
  if (static_cast<int>(res.first.size()) > cap) return fail("tch_distributor_get_batch: output too small");
  for (size_t i = 0; i < res.first.size(); ++i) {
    ranges_out[2 * i] = res.first[i].first;
    ranges_out[2 * i + 1] = res.first[i].second;
  }
  if (last) *last = res.second ? 1 : 0;
  return static_cast<int>(res.first.size());
}
int tch_distributor_query_next_batch_size(int bs) {
  NEED_DIST();
  return DynamicBatchDistributor::get()->query_next_batch_size(bs);
}
static BatchRangeVec to_ranges(const int* r, int n) {
  BatchRangeVec v;
  for (int i = 0; i < n; ++i) v.emplace_back(r[2 * i], r[2 * i + 1]);
  return v;
}
int tch_distributor_finish_batch(const int* ranges, int n, int end_of_global_batch) {
  NEED_DIST();
  std::string err;
  return DynamicBatchDistributor::get()->finish_batch(to_ranges(ranges, n), end_of_global_batch != 0, &err) ? 0 : fail(err);
}
int tch_distributor_abort_batch(const int* ranges, int n, int end_of_global_batch) {
  NEED_DIST();
  std::string err;
  return DynamicBatchDistributor::get()->abort_batch(to_ranges(ranges, n), end_of_global_batch != 0, &err) ? 0 : fail(err);
}
int tch_distributor_vote_finish_last_micro_batch(void) {
  NEED_DIST();
  return DynamicBatchDistributor::get()->vote_finish_last_micro_batch() ? 1 : 0;
}
void tch_distributor_vote_abort_last_micro_batch(void) { if (DynamicBatchDistributor::get()) DynamicBatchDistributor::get()->vote_abort_last_micro_batch(); }
void tch_distributor_reset_last_micro_batch_finish_vote(void) { if (DynamicBatchDistributor::get()) DynamicBatchDistributor::get()->reset_last_micro_batch_finish_vote(); }
void tch_distributor_distribute_batch(int a, int b, int c) { if (DynamicBatchDistributor::get()) DynamicBatchDistributor::get()->distribute_batch(a != 0, b != 0, c != 0); }
int tch_distributor_next_epoch(void) {
  NEED_DIST();
  std::string err;
  int e = DynamicBatchDistributor::get()->next_epoch(&err);
  return e < 0 ? fail(err) : e;
}
void tch_distributor_next_global_batch(void) { if (DynamicBatchDistributor::get()) DynamicBatchDistributor::get()->next_global_batch(); }
int tch_distributor_get_global_batch_size(void) { NEED_DIST(); return DynamicBatchDistributor::get()->global_batch_size(); }
int tch_distributor_get_num_global_batch_per_epoch(void) { NEED_DIST(); return DynamicBatchDistributor::get()->num_global_batches_per_epoch(); }
int tch_distributor_get_num_proced_global_batch(void) { NEED_DIST(); return DynamicBatchDistributor::get()->num_proced_global_batches(); }
int tch_distributor_snapshot(int which, int* ranges_out, int cap) {
  NEED_DIST();
  auto v = DynamicBatchDistributor::get()->snapshot(which);
  for (int i = 0; i < cap && i < static_cast<int>(v.size()); ++i) {
    ranges_out[2 * i] = v[i].first;
    ranges_out[2 * i + 1] = v[i].second;
  }
  return static_cast<int>(v.size());
}
int tch_distributor_counters(int* out, int cap) {
  NEED_DIST();
  auto v = DynamicBatchDistributor::get()->counters();
  for (int i = 0; i < cap && i < static_cast<int>(v.size()); ++i) out[i] = v[i];
  return static_cast<int>(v.size());
}

void tch_perf_model_record_thpt(int bs, double ms) { PerfModel::record_thpt(bs, ms); }
double tch_perf_model_get_thpt(int bs) { return PerfModel::get_thpt(bs); }
void tch_perf_model_get_thpt_vec(const int* bs, int n, double* out) {
  std::vector<int> v(bs, bs + n);
  auto r = PerfModel::get_thpt_vec(v);
  for (int i = 0; i < n; ++i) out[i] = r[i];
}
void tch_perf_model_clear(void) { PerfModel::clear(); }

int64_t tch_get_unix_timestamp(void) { return unix_timestamp_ms(); }
int64_t tch_get_unix_timestamp_us(void) { return unix_timestamp_us(); }

}  // extern "C"
