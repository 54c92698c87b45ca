// Inference <-> training control channel: per-rank, per-direction FIFO message queues and
// an information board, in one POSIX shared-memory segment.
//
// Restates common/inf_tra_comm/{message_queue,shared_info,communicator}.{h,cc}:
//   CtrlMsgEntry {u64 id; int event; int value}            message_queue.h:12-16
//   CtrlEvent values 0..12, kNumEvent = 13, in this order  message_queue.h:18-40
//   Put / PutAll / BlockGet / TryGet / TimedGet / BlockGetFromAny   message_queue.cc:110-256
//   TrainInfo fields and first-set rule                    shared_info.h:21-35, shared_info.cc:54-108
//   segment name <prefix>_inf_tra_comm, created (and removed) by the server side
//                                                          communicator.cc:9-62
#pragma once

#include <sys/types.h>

#include <memory>
#include <string>
#include <vector>

#include "shm.h"

namespace tch {
namespace host {

struct CtrlMsgEntry {
  uint64_t id;
  int event;
  int value;
};

enum CtrlEvent : int {
  kTrainStart = 0,
  kTrainEnd,
  kInterruptTrainDone,
  kResumeTrainDone,
  kColocateAdjustL1Done,
  kColocateAdjustL2Done,
  kReportBatchSize,
  kInterruptTrain,
  kResumeTrain,
  kColocateAdjustL1,
  kColocateAdjustL2,
  kInferExit,
  kInferenceWorkloadDone,
  kNumEvent,
};

enum Direction : int { kInf2Tra = 0, kTra2Inf = 1, kNumDirection = 2 };

struct TrainInfo {
  pid_t train_pid;  // -1 = invalid (not yet set by a trainer)
  int train_rank;
  int train_world_size;
  int init_batch_size;
  int current_batch_size;
  int target_batch_size;
  int target_batch_size_unpublished;
  char model_name[256];
  bool first_epoch_done;
};

enum TrainInfoField : int {
  kFieldPid = 0,
  kFieldRank,
  kFieldWorldSize,
  kFieldInitBatchSize,
  kFieldCurrentBatchSize,
  kFieldTargetBatchSize,
  kFieldTargetBatchSizeUnpublished,
  kFieldFirstEpochDone,
};

constexpr int kMqCapacity = 4096;

struct ShmMsgQueue {
  pthread_mutex_t mu;
  pthread_cond_t cond;
  uint32_t head, count;
  CtrlMsgEntry buf[kMqCapacity];
};

struct InfTraLayout {
  ShmHeader header;
  int train_world_size;
  pthread_mutex_t shm_mutex;
  pthread_mutex_t group_mu[kNumDirection];
  pthread_cond_t group_cond[kNumDirection];
  ShmMsgQueue mq[kNumDirection][kMaxDeviceNum];
  pthread_mutex_t train_info_mu[kMaxDeviceNum];
  TrainInfo train_info[kMaxDeviceNum];
  // compute units the inference side wants for itself on each device, read by the trainer before it
  // launches (the tpc_datas[...].infer_required_tpc_num of the reference, common/sm_partition.cc:60-76)
  int infer_required_cus[kMaxDeviceNum];
};

class InfTraCommunicator {
 public:
  // is_server: this process creates (and at the end removes) the segment; cleanup: remove a
  // stale one first.  Returns nullptr + *err on failure.
  static InfTraCommunicator* create(bool is_server, bool cleanup, int train_world_size, std::string* err);
  ~InfTraCommunicator();

  // Ask every blocking get of THIS process to return (block_get: a message with event -1; the *_from_any
  // form: rank -1) at its next wake-up, which is at most 50 ms away.  Called by communicator_shutdown(); the
  // segment itself stays mapped until the last holder of the shared_ptr lets go.
  void close() { closed_.store(true, std::memory_order_release); }
  bool closed() const { return closed_.load(std::memory_order_acquire); }

  int world_size() const { return layout_->train_world_size; }

  // ---- message queues ----
  bool put(const CtrlMsgEntry& msg, Direction d, int id);
  bool put_all(const CtrlMsgEntry& msg, Direction d);
  bool put_all(const std::vector<CtrlMsgEntry>& msgs, Direction d);
  CtrlMsgEntry block_get(Direction d, int id);
  bool try_get(Direction d, int id, CtrlMsgEntry* msg);
  bool timed_get(uint32_t timeout_ms, Direction d, int id, CtrlMsgEntry* msg);
  std::pair<int, CtrlMsgEntry> block_get_from_any(Direction d);
  bool timed_get_from_any(uint32_t timeout_ms, Direction d, int* id, CtrlMsgEntry* msg);
  void clear();

  // ---- information board ----
  bool train_info_valid(int id);
  void invalidate_train_info(int id);
  // fields with has_* false are left alone; the FIRST set of a slot (pid still -1) needs a pid
  // and also seeds target_batch_size and target_batch_size_unpublished with init_batch_size
  bool set_train_info(int id, const pid_t* pid, const int* rank, const int* world_size, const int* init_batch_size,
                      const int* current_batch_size, const char* model_name);
  TrainInfo get_train_info(int id);
  int get_field(int id, TrainInfoField f);
  void update_field(int id, TrainInfoField f, int value);
  std::vector<int> get_field_vec(TrainInfoField f);
  void update_field_vec(TrainInfoField f, const std::vector<int>& values);
  std::vector<pid_t> train_pids();
  // ---- compute-unit demand of the inference side (relaxed atomics on the shared int) ----
  int infer_required_cus(int device) { return __atomic_load_n(&layout_->infer_required_cus[device], __ATOMIC_RELAXED); }
  void set_infer_required_cus(int device, int n) { __atomic_store_n(&layout_->infer_required_cus[device], n, __ATOMIC_RELAXED); }
  int add_infer_required_cus(int device, int delta) {
    return __atomic_add_fetch(&layout_->infer_required_cus[device], delta, __ATOMIC_RELAXED);
  }

 private:
  InfTraCommunicator() = default;
  std::unique_ptr<ShmSegment> seg_;
  InfTraLayout* layout_ = nullptr;
  std::atomic<bool> closed_{false};   // process-local: not part of the shared layout
};

// Process-wide instance used by the stubs and the batch distributor.  Every caller gets a counted reference:
// whoever is inside a call (a control thread waiting in timed_get, a side thread in put) keeps the segment
// mapped for the length of that call, whatever another thread shuts down meanwhile.  Null when not initialised.
std::shared_ptr<InfTraCommunicator> communicator();
bool communicator_init(bool is_server, bool cleanup, int train_world_size, std::string* err);
void communicator_shutdown();

}  // namespace host
}  // namespace tch
