// State shared among the training ranks of one job, and the three components that live on it:
//   DistTrainSync            barrier + 256-byte-chunk string channels
//                            (pytorch/torch_col/csrc/dist_train_sync.cc:30-145)
//   DynamicBatchDistributor  sample-range bookkeeping of one global batch
//                            (pytorch/torch_col/csrc/dynamic_batch.cc:40-819; the reference
//                            spells the class "DynamicBatchDistirbutor")
//   PerfModel                batch size -> running-mean throughput
//                            (pytorch/torch_col/csrc/perf_model.cc:25-94)
// All of it is integer / fp64 bookkeeping, needed at world size 1 too.
#pragma once

#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "shm.h"

namespace tch {
namespace host {

constexpr int kStrChunk = 256;   // dist_train_sync.h kMsgBufSize
constexpr int kStrRing = 64;
constexpr int kRangeCap = 8192;  // ranges one set can hold
constexpr int kPerfCap = 1024;   // distinct batch sizes the perf model can hold

struct StrQueue {
  pthread_mutex_t mu;
  pthread_cond_t get_cond, put_cond;
  uint32_t head, count;
  char buf[kStrRing][kStrChunk];
};

// ordered set of half-open sample ranges [lo, hi), ordered by (lo, hi) like std::pair
struct RangeSet {
  int n;
  int lo[kRangeCap];
  int hi[kRangeCap];
};

struct DistTrainLayout {
  ShmHeader header;
  int world_size;
  // barrier
  pthread_mutex_t barrier_mu;
  pthread_cond_t barrier_cond;
  int barrier_waiting;
  unsigned barrier_generation;
  // string channels [src][dst]
  StrQueue str_mq[kMaxDeviceNum][kMaxDeviceNum];
  // batch distributor (dynamic_batch.h GlobalSharedData)
  pthread_mutex_t db_mu;
  pthread_cond_t db_vote_cond;
  int db_vote_cnt;
  int num_unproc_per_train[kMaxDeviceNum];
  int num_procing_per_train[kMaxDeviceNum];
  int num_proced_per_train[kMaxDeviceNum];
  int has_unproc_batches[kMaxDeviceNum];
  RangeSet unproc, procing, proced;
  int num_unproc, num_procing, num_proced;
  // perf model: sorted by batch size
  pthread_mutex_t pm_mu;
  int pm_n;
  int pm_bs[kPerfCap];
  double pm_thpt[kPerfCap];
  int pm_cnt[kPerfCap];
  // task-switch stub flags (control_stub.h SwitchStub::GlobalSharedData)
  pthread_mutex_t sw_mu;
  int sw_interrupt_flag;
  int sw_has_batch_killed;
};

class DistTrainSync {
 public:
  // rank 0 creates (after removing a stale segment), the others open
  static bool init(int rank, int world_size, std::string* err);
  static bool initialized();
  static void shutdown();
  static DistTrainLayout* layout();
  static int rank();
  static int world_size();
  static void wait_barrier();
  static void send(int dst, const std::string& msg);
  static std::string recv(int src);
};

using BatchRange = std::pair<int, int>;
using BatchRangeVec = std::vector<BatchRange>;

enum class DistributePolicy { kFix, kSimple, kByPerformance };

class DynamicBatchDistributor {
 public:
  // returns false + *err on bad arguments
  static bool init(int dataset_size, int input_batch_size, int global_batch_size, bool lazy_distributing,
                   const std::string& policy, std::string* err);
  static bool initialized();
  static void shutdown();
  static DynamicBatchDistributor* get();

  void distribute_batch(bool check_num_unproced_samples, bool distribute_to_all, bool at_global_batch_begin);
  // ranges for a micro-batch of (at most) batch_size samples, and whether it is the last of
  // this rank's share of the global batch.  err != "" on a broken invariant.
  std::pair<BatchRangeVec, bool> get_batch(int batch_size, std::string* err);
  int query_next_batch_size(int batch_size);
  bool finish_batch(const BatchRangeVec& v, bool end_of_global_batch, std::string* err);
  bool abort_batch(const BatchRangeVec& v, bool end_of_global_batch, std::string* err);
  bool vote_finish_last_micro_batch();
  void vote_abort_last_micro_batch();
  void reset_last_micro_batch_finish_vote();
  void next_global_batch();
  int next_epoch(std::string* err);

  int global_batch_size() const { return global_batch_size_; }
  int num_global_batches_per_epoch() const { return num_global_batches_per_epoch_; }
  int num_proced_global_batches() const { return num_proced_global_batches_; }
  // test / debug views
  BatchRangeVec snapshot(int which);  // 0 unproc, 1 procing, 2 proced
  std::vector<int> counters();        // g_unproc, g_procing, g_proced, then per-rank unproc/procing/proced

 private:
  DynamicBatchDistributor() = default;
  void distribute_without_lock(bool check, bool to_all, bool at_begin);
  void distribute_impl(const std::vector<int>& ongoing, const std::vector<int>& target_bs, int num_unproc);
  std::pair<int, bool> lazy_batch_size(int batch_size);

  bool lazy_ = false;
  DistributePolicy policy_ = DistributePolicy::kSimple;
  int dataset_size_ = 0, input_batch_size_ = 0, global_batch_size_ = 0;
  bool first_epoch_start_ = false;
  int num_proced_sample_of_epoch_ = 0, num_proced_global_batches_ = 0, next_epoch_idx_ = 0;
  int num_global_batches_per_epoch_ = 0;
};

class PerfModel {
 public:
  static void record_thpt(int batch_size, double batch_time_ms);
  static double get_thpt(int batch_size);
  static std::vector<double> get_thpt_vec(const std::vector<int>& batch_sizes);
  static void clear();
};

}  // namespace host
}  // namespace tch
