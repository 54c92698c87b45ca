#include "inf_tra_comm.h"

#include <string.h>

#include <mutex>

namespace tch {
namespace host {

namespace {
std::mutex g_comm_mu;
std::shared_ptr<InfTraCommunicator> g_comm;   // read and replaced under g_comm_mu only

// longest a blocking get sleeps before it looks at closed() again
constexpr int64_t kWakeMs = 50;

void push(ShmMsgQueue* q, const CtrlMsgEntry& m) {
  if (q->count == kMqCapacity) {  // never expected: drop the oldest rather than block the sender
    q->head = (q->head + 1) % kMqCapacity;
    q->count--;
  }
  q->buf[(q->head + q->count) % kMqCapacity] = m;
  q->count++;
}

CtrlMsgEntry pop(ShmMsgQueue* q) {
  CtrlMsgEntry m = q->buf[q->head];
  q->head = (q->head + 1) % kMqCapacity;
  q->count--;
  return m;
}

int* field_ptr(TrainInfo* t, TrainInfoField f) {
  switch (f) {
    case kFieldPid: return reinterpret_cast<int*>(&t->train_pid);
    case kFieldRank: return &t->train_rank;
    case kFieldWorldSize: return &t->train_world_size;
    case kFieldInitBatchSize: return &t->init_batch_size;
    case kFieldCurrentBatchSize: return &t->current_batch_size;
    case kFieldTargetBatchSize: return &t->target_batch_size;
    case kFieldTargetBatchSizeUnpublished: return &t->target_batch_size_unpublished;
    default: return nullptr;
  }
}
}  // namespace

InfTraCommunicator* InfTraCommunicator::create(bool is_server, bool cleanup, int train_world_size, std::string* err) {
  if (train_world_size < 1 || train_world_size > kMaxDeviceNum) {
    if (err) *err = "train world size out of range";
    return nullptr;
  }
  std::unique_ptr<ShmSegment> seg(
      ShmSegment::open(default_shm_prefix() + "_inf_tra_comm", sizeof(InfTraLayout), is_server, cleanup, err));
  if (!seg) return nullptr;
  auto* c = new InfTraCommunicator();
  c->layout_ = static_cast<InfTraLayout*>(seg->base());
  if (seg->created()) {
    InfTraLayout* l = c->layout_;
    l->train_world_size = train_world_size;
    init_shared_mutex(&l->shm_mutex);
    for (int d = 0; d < kNumDirection; ++d) {
      init_shared_mutex(&l->group_mu[d]);
      init_shared_cond(&l->group_cond[d]);
      for (int i = 0; i < kMaxDeviceNum; ++i) {
        init_shared_mutex(&l->mq[d][i].mu);
        init_shared_cond(&l->mq[d][i].cond);
        l->mq[d][i].head = l->mq[d][i].count = 0;
      }
    }
    for (int i = 0; i < kMaxDeviceNum; ++i) {
      init_shared_mutex(&l->train_info_mu[i]);
      memset(&l->train_info[i], 0, sizeof(TrainInfo));
      l->train_info[i].train_pid = -1;
      l->infer_required_cus[i] = 0;
    }
    seg->mark_ready();
  } else if (c->layout_->train_world_size < train_world_size) {
    if (err) *err = "existing inf-tra segment was made for a smaller training world";
    delete c;
    return nullptr;
  }
  c->seg_ = std::move(seg);
  return c;
}

InfTraCommunicator::~InfTraCommunicator() = default;

bool InfTraCommunicator::put(const CtrlMsgEntry& msg, Direction d, int id) {
  if (id < 0 || id >= world_size()) return false;
  ShmMsgQueue* q = &layout_->mq[d][id];
  {
    ShmLock lock(&q->mu);
    push(q, msg);
    pthread_cond_signal(&q->cond);
  }
  ShmLock g(&layout_->group_mu[d]);
  pthread_cond_signal(&layout_->group_cond[d]);
  return true;
}

bool InfTraCommunicator::put_all(const CtrlMsgEntry& msg, Direction d) {
  for (int i = 0; i < world_size(); ++i) {
    ShmMsgQueue* q = &layout_->mq[d][i];
    ShmLock lock(&q->mu);
    push(q, msg);
    pthread_cond_signal(&q->cond);
  }
  ShmLock g(&layout_->group_mu[d]);
  pthread_cond_signal(&layout_->group_cond[d]);
  return true;
}

bool InfTraCommunicator::put_all(const std::vector<CtrlMsgEntry>& msgs, Direction d) {
  if (static_cast<int>(msgs.size()) != world_size()) return false;
  for (int i = 0; i < world_size(); ++i) {
    ShmMsgQueue* q = &layout_->mq[d][i];
    ShmLock lock(&q->mu);
    push(q, msgs[i]);
    pthread_cond_signal(&q->cond);
  }
  ShmLock g(&layout_->group_mu[d]);
  pthread_cond_signal(&layout_->group_cond[d]);
  return true;
}

CtrlMsgEntry InfTraCommunicator::block_get(Direction d, int id) {
  ShmMsgQueue* q = &layout_->mq[d][id];
  ShmLock lock(&q->mu);
  while (q->count == 0) {
    if (closed()) return CtrlMsgEntry{0, -1, 0};
    cond_wait_ms(&q->cond, &q->mu, kWakeMs);
  }
  return pop(q);
}

bool InfTraCommunicator::try_get(Direction d, int id, CtrlMsgEntry* msg) {
  ShmMsgQueue* q = &layout_->mq[d][id];
  ShmLock lock(&q->mu);
  if (q->count == 0) return false;
  *msg = pop(q);
  return true;
}

bool InfTraCommunicator::timed_get(uint32_t timeout_ms, Direction d, int id, CtrlMsgEntry* msg) {
  ShmMsgQueue* q = &layout_->mq[d][id];
  ShmLock lock(&q->mu);
  const int64_t deadline = unix_timestamp_ms() + timeout_ms;
  while (q->count == 0) {
    int64_t left = deadline - unix_timestamp_ms();
    if (left <= 0 || closed()) return false;
    cond_wait_ms(&q->cond, &q->mu, left < kWakeMs ? left : kWakeMs);
  }
  *msg = pop(q);
  return true;
}

bool InfTraCommunicator::timed_get_from_any(uint32_t timeout_ms, Direction d, int* id, CtrlMsgEntry* msg) {
  const int64_t deadline = unix_timestamp_ms() + timeout_ms;
  ShmLock g(&layout_->group_mu[d]);
  for (;;) {
    for (int i = 0; i < world_size(); ++i) {
      ShmMsgQueue* q = &layout_->mq[d][i];
      ShmLock lock(&q->mu);
      if (q->count > 0) {
        *id = i;
        *msg = pop(q);
        return true;
      }
    }
    int64_t left = deadline - unix_timestamp_ms();
    if (left <= 0 || closed()) return false;
    // a sender signals the group condition after releasing the queue lock; poll at a
    // bounded interval so a signal that slipped in between is never waited on for long
    cond_wait_ms(&layout_->group_cond[d], &layout_->group_mu[d], left < kWakeMs ? left : kWakeMs);
  }
}

std::pair<int, CtrlMsgEntry> InfTraCommunicator::block_get_from_any(Direction d) {
  int id = 0;
  CtrlMsgEntry m{};
  while (!timed_get_from_any(1000, d, &id, &m)) {
    if (closed()) return {-1, CtrlMsgEntry{0, -1, 0}};
  }
  return {id, m};
}

void InfTraCommunicator::clear() {
  for (int d = 0; d < kNumDirection; ++d)
    for (int i = 0; i < world_size(); ++i) {
      ShmMsgQueue* q = &layout_->mq[d][i];
      ShmLock lock(&q->mu);
      q->head = q->count = 0;
    }
}

bool InfTraCommunicator::train_info_valid(int id) {
  ShmLock lock(&layout_->train_info_mu[id]);
  return layout_->train_info[id].train_pid != -1;
}

void InfTraCommunicator::invalidate_train_info(int id) {
  ShmLock lock(&layout_->train_info_mu[id]);
  layout_->train_info[id].train_pid = -1;
}

bool InfTraCommunicator::set_train_info(int id, const pid_t* pid, const int* rank, const int* world_size,
                                        const int* init_batch_size, const int* current_batch_size,
                                        const char* model_name) {
  if (id < 0 || id >= kMaxDeviceNum) return false;
  ShmLock lock(&layout_->train_info_mu[id]);
  TrainInfo* t = &layout_->train_info[id];
  const bool initial = t->train_pid == -1;
  if (initial && !pid) return false;  // the first set must carry the pid
  if (pid) t->train_pid = *pid;
  if (rank) t->train_rank = *rank;
  if (world_size) t->train_world_size = *world_size;
  if (init_batch_size) {
    t->init_batch_size = *init_batch_size;
    if (initial) {
      t->target_batch_size = *init_batch_size;
      t->target_batch_size_unpublished = *init_batch_size;
    }
  }
  if (current_batch_size) t->current_batch_size = *current_batch_size;
  if (model_name) {
    strncpy(t->model_name, model_name, sizeof(t->model_name) - 1);
    t->model_name[sizeof(t->model_name) - 1] = 0;
  }
  return true;
}

TrainInfo InfTraCommunicator::get_train_info(int id) {
  ShmLock lock(&layout_->train_info_mu[id]);
  return layout_->train_info[id];
}

int InfTraCommunicator::get_field(int id, TrainInfoField f) {
  ShmLock lock(&layout_->train_info_mu[id]);
  TrainInfo* t = &layout_->train_info[id];
  if (f == kFieldFirstEpochDone) return t->first_epoch_done ? 1 : 0;
  int* p = field_ptr(t, f);
  return p ? *p : 0;
}

void InfTraCommunicator::update_field(int id, TrainInfoField f, int value) {
  ShmLock lock(&layout_->train_info_mu[id]);
  TrainInfo* t = &layout_->train_info[id];
  if (f == kFieldFirstEpochDone) {
    t->first_epoch_done = value != 0;
    return;
  }
  if (int* p = field_ptr(t, f)) *p = value;
}

std::vector<int> InfTraCommunicator::get_field_vec(TrainInfoField f) {
  // world size as the trainer announced it on slot 0 (shared_info.h:195-207); fall back
  // to the segment's size before any trainer registered
  int n = get_field(0, kFieldWorldSize);
  if (n <= 0 || n > world_size()) n = world_size();
  std::vector<int> out(n);
  for (int i = 0; i < n; ++i) out[i] = get_field(i, f);
  return out;
}

void InfTraCommunicator::update_field_vec(TrainInfoField f, const std::vector<int>& values) {
  for (size_t i = 0; i < values.size() && i < static_cast<size_t>(kMaxDeviceNum); ++i)
    update_field(static_cast<int>(i), f, values[i]);
}

std::vector<pid_t> InfTraCommunicator::train_pids() {
  int n = get_field(0, kFieldWorldSize);
  std::vector<pid_t> out;
  for (int i = 0; i < n && i < kMaxDeviceNum; ++i) out.push_back(get_train_info(i).train_pid);
  return out;
}

std::shared_ptr<InfTraCommunicator> communicator() {
  std::lock_guard<std::mutex> l(g_comm_mu);
  return g_comm;
}

bool communicator_init(bool is_server, bool cleanup, int train_world_size, std::string* err) {
  std::lock_guard<std::mutex> l(g_comm_mu);
  if (g_comm) {
    if (err) *err = "InfTraCommunicator has already been initialized";
    return false;
  }
  g_comm.reset(InfTraCommunicator::create(is_server, cleanup, train_world_size, err));
  return g_comm != nullptr;
}

void communicator_shutdown() {
  // The instance is taken out of the global first, so no new caller can find it; callers that are inside it
  // hold references of their own.  close() makes the blocked ones return within kWakeMs, and the segment is
  // unmapped (and, on the creating side, unlinked) by whichever thread drops the last reference -- never
  // under a thread that still waits on a mutex or condition variable inside the mapping.
  std::shared_ptr<InfTraCommunicator> last;
  {
    std::lock_guard<std::mutex> l(g_comm_mu);
    last.swap(g_comm);
  }
  if (last) last->close();
}

}  // namespace host
}  // namespace tch
