#include "dist_train.h"

#include <string.h>

#include <algorithm>
#include <limits>

#include "config.h"
#include "inf_tra_comm.h"

namespace tch {
namespace host {

namespace {
std::unique_ptr<ShmSegment> g_seg;
DistTrainLayout* g_layout = nullptr;
int g_rank = 0, g_world = 1;
std::unique_ptr<DynamicBatchDistributor> g_distributor;

constexpr int kAbortLastMicroBatch = std::numeric_limits<int>::min();
constexpr int kVoteFinish = 1;

// ---- ordered range set --------------------------------------------------------
bool range_less(int lo_a, int hi_a, int lo_b, int hi_b) { return lo_a < lo_b || (lo_a == lo_b && hi_a < hi_b); }

int set_lower_bound(const RangeSet* s, int lo, int hi) {
  int a = 0, b = s->n;
  while (a < b) {
    int m = (a + b) / 2;
    if (range_less(s->lo[m], s->hi[m], lo, hi)) a = m + 1; else b = m;
  }
  return a;
}

int set_find(const RangeSet* s, int lo, int hi) {
  int i = set_lower_bound(s, lo, hi);
  return (i < s->n && s->lo[i] == lo && s->hi[i] == hi) ? i : -1;
}

bool set_insert(RangeSet* s, int lo, int hi) {
  int i = set_lower_bound(s, lo, hi);
  if (i < s->n && s->lo[i] == lo && s->hi[i] == hi) return true;  // already there (set semantics)
  if (s->n >= kRangeCap) return false;
  memmove(&s->lo[i + 1], &s->lo[i], sizeof(int) * (s->n - i));
  memmove(&s->hi[i + 1], &s->hi[i], sizeof(int) * (s->n - i));
  s->lo[i] = lo;
  s->hi[i] = hi;
  s->n++;
  return true;
}

void set_erase(RangeSet* s, int i) {
  memmove(&s->lo[i], &s->lo[i + 1], sizeof(int) * (s->n - i - 1));
  memmove(&s->hi[i], &s->hi[i + 1], sizeof(int) * (s->n - i - 1));
  s->n--;
}
}  // namespace

// ---------------------------------------------------------------------------
// DistTrainSync
// ---------------------------------------------------------------------------

bool DistTrainSync::init(int rank, int world_size, std::string* err) {
  if (g_layout) {
    if (err) *err = "DistTrainSync has been initialized";
    return false;
  }
  if (world_size < 1 || world_size > kMaxDeviceNum || rank < 0 || rank >= world_size) {
    if (err) *err = "bad rank / world size";
    return false;
  }
  const bool master = rank == 0;
  g_seg.reset(ShmSegment::open(default_shm_prefix() + "_dist_train_sync", sizeof(DistTrainLayout), master, master, err));
  if (!g_seg) return false;
  g_layout = static_cast<DistTrainLayout*>(g_seg->base());
  g_rank = rank;
  g_world = world_size;
  if (g_seg->created()) {
    DistTrainLayout* l = g_layout;
    l->world_size = world_size;
    init_shared_mutex(&l->barrier_mu);
    init_shared_cond(&l->barrier_cond);
    for (int i = 0; i < kMaxDeviceNum; ++i)
      for (int j = 0; j < kMaxDeviceNum; ++j) {
        init_shared_mutex(&l->str_mq[i][j].mu);
        init_shared_cond(&l->str_mq[i][j].get_cond);
        init_shared_cond(&l->str_mq[i][j].put_cond);
      }
    init_shared_mutex(&l->db_mu);
    init_shared_cond(&l->db_vote_cond);
    init_shared_mutex(&l->pm_mu);
    init_shared_mutex(&l->sw_mu);
    g_seg->mark_ready();
  }
  wait_barrier();
  return true;
}

bool DistTrainSync::initialized() { return g_layout != nullptr; }

void DistTrainSync::shutdown() {
  g_distributor.reset();
  g_layout = nullptr;
  g_seg.reset();
}

DistTrainLayout* DistTrainSync::layout() { return g_layout; }
int DistTrainSync::rank() { return g_rank; }
int DistTrainSync::world_size() { return g_world; }

void DistTrainSync::wait_barrier() {
  DistTrainLayout* l = g_layout;
  if (!l || g_world == 1) return;
  ShmLock lock(&l->barrier_mu);
  const unsigned gen = l->barrier_generation;
  if (++l->barrier_waiting == g_world) {
    l->barrier_waiting = 0;
    l->barrier_generation++;
    pthread_cond_broadcast(&l->barrier_cond);
    return;
  }
  while (l->barrier_generation == gen) cond_wait_ms(&l->barrier_cond, &l->barrier_mu, -1);
}

void DistTrainSync::send(int dst, const std::string& msg) {
  StrQueue* q = &g_layout->str_mq[g_rank][dst];
  // Every chunk is zero-padded and the receiver stops at the first chunk holding a zero byte,
  // so the last chunk must always have room for one: a message whose length is a multiple of
  // the chunk size (the empty message included) is closed by an all-zero chunk.
  const size_t n_chunks = msg.size() / kStrChunk + 1;
  for (size_t c = 0; c < n_chunks; ++c) {
    const size_t off = c * kStrChunk;
    const size_t len = off < msg.size() ? std::min(msg.size() - off, static_cast<size_t>(kStrChunk)) : 0;
    ShmLock lock(&q->mu);
    while (q->count == kStrRing) cond_wait_ms(&q->put_cond, &q->mu, -1);
    char* slot = q->buf[(q->head + q->count) % kStrRing];
    memset(slot, 0, kStrChunk);
    if (len) memcpy(slot, msg.data() + off, len);
    q->count++;
    pthread_cond_signal(&q->get_cond);
  }
}

std::string DistTrainSync::recv(int src) {
  StrQueue* q = &g_layout->str_mq[src][g_rank];
  std::string out;
  for (;;) {
    char chunk[kStrChunk];
    {
      ShmLock lock(&q->mu);
      while (q->count == 0) cond_wait_ms(&q->get_cond, &q->mu, -1);
      memcpy(chunk, q->buf[q->head], kStrChunk);
      q->head = (q->head + 1) % kStrRing;
      q->count--;
      pthread_cond_signal(&q->put_cond);
    }
    const char* z = static_cast<const char*>(memchr(chunk, 0, kStrChunk));
    if (z) {
      out.append(chunk, z - chunk);
      break;
    }
    out.append(chunk, kStrChunk);
  }
  return out;
}

// ---------------------------------------------------------------------------
// DynamicBatchDistributor
// ---------------------------------------------------------------------------

bool DynamicBatchDistributor::init(int dataset_size, int input_batch_size, int global_batch_size, bool lazy,
                                   const std::string& policy_in, std::string* err) {
  if (g_distributor) {
    if (err) *err = "batch distributor has been initialized";
    return false;
  }
  if (!DistTrainSync::initialized()) {
    if (err) *err = "DistTrainSync must be initialized first";
    return false;
  }
  if (dataset_size <= 0 || input_batch_size <= 0 || global_batch_size <= 0) {
    if (err) *err = "dataset size, batch size and global batch size must be positive";
    return false;
  }
  std::string policy = policy_in;
  std::transform(policy.begin(), policy.end(), policy.begin(), ::tolower);
  std::unique_ptr<DynamicBatchDistributor> d(new DynamicBatchDistributor());
  if (policy == "fix") d->policy_ = DistributePolicy::kFix;
  else if (policy == "simple") d->policy_ = DistributePolicy::kSimple;
  else if (policy == "by_performance") d->policy_ = DistributePolicy::kByPerformance;
  else {
    if (err) *err = "Unknown distribute policy " + policy_in;
    return false;
  }
  d->lazy_ = lazy;
  d->dataset_size_ = dataset_size;
  d->input_batch_size_ = input_batch_size;
  d->global_batch_size_ = global_batch_size;
  d->num_global_batches_per_epoch_ = (dataset_size + global_batch_size - 1) / global_batch_size;
  DistTrainLayout* l = DistTrainSync::layout();
  if (lazy) {
    if (DistTrainSync::rank() == 0) {
      ShmLock lock(&l->db_mu);
      for (int i = 0; i < DistTrainSync::world_size(); ++i)
        l->num_unproc_per_train[i] = l->num_procing_per_train[i] = l->num_proced_per_train[i] = -1;
    }
    DistTrainSync::wait_barrier();
  }
  g_distributor = std::move(d);
  return true;
}

bool DynamicBatchDistributor::initialized() { return g_distributor != nullptr; }
void DynamicBatchDistributor::shutdown() { g_distributor.reset(); }
DynamicBatchDistributor* DynamicBatchDistributor::get() { return g_distributor.get(); }

void DynamicBatchDistributor::distribute_batch(bool check, bool to_all, bool at_begin) {
  ShmLock lock(&DistTrainSync::layout()->db_mu);
  distribute_without_lock(check, to_all, at_begin);
}

void DynamicBatchDistributor::distribute_without_lock(bool check, bool to_all, bool at_begin) {
  DistTrainLayout* l = DistTrainSync::layout();
  const int world = DistTrainSync::world_size();
  auto comm = config().has_colocated_infer_server ? communicator() : nullptr;
  const bool has_server = comm != nullptr;
  std::vector<int> target_bs_unpub;
  if (has_server) target_bs_unpub = comm->get_field_vec(kFieldTargetBatchSizeUnpublished);

  const bool do_distribute = !(lazy_ || (!at_begin && policy_ == DistributePolicy::kFix));
  int num_unproc = l->num_unproc;
  if (check && do_distribute) {
    // the per-rank shares must add up to the global count; if they ever do not, the global
    // count is the truth the ranges were carved from
    int sum = 0;
    for (int i = 0; i < world; ++i) sum += l->num_unproc_per_train[i];
    if (sum != l->num_unproc) num_unproc = l->num_unproc;
  }
  if (to_all)
    for (int i = 0; i < world; ++i) l->has_unproc_batches[i] = 1;
  if (do_distribute) {
    std::vector<int> ongoing, target_bs;
    for (int i = 0; i < world; ++i) {
      if (l->has_unproc_batches[i]) {
        ongoing.push_back(i);
        target_bs.push_back(has_server && i < static_cast<int>(target_bs_unpub.size()) ? target_bs_unpub[i]
                                                                                        : input_batch_size_);
      }
    }
    if (!ongoing.empty()) distribute_impl(ongoing, target_bs, num_unproc);
  }
  if (has_server) comm->update_field_vec(kFieldTargetBatchSize, target_bs_unpub);
}

void DynamicBatchDistributor::distribute_impl(const std::vector<int>& ongoing, const std::vector<int>& target_bs,
                                              int num_unproc) {
  DistTrainLayout* l = DistTrainSync::layout();
  const int w = static_cast<int>(ongoing.size());
  if (policy_ != DistributePolicy::kByPerformance) {
    const int per = num_unproc / w, rem = num_unproc % w;
    for (int i = 0; i < w; ++i) l->num_unproc_per_train[ongoing[i]] = per + (i < rem ? 1 : 0);
    return;
  }
  std::vector<double> perf = PerfModel::get_thpt_vec(target_bs);
  double perf_sum = 0;
  for (double p : perf) perf_sum += p;
  int distributed = 0;
  for (int i = 0; i < w; ++i) {
    double ratio = perf_sum == 0 ? 1.0 / w : perf[i] / perf_sum;
    int n = std::max(1, static_cast<int>(num_unproc * ratio));
    l->num_unproc_per_train[ongoing[i]] = n;
    distributed += n;
  }
  int diff = num_unproc - distributed;
  // +-1 round robin until the shares add up; a share never drops below one sample, so when
  // every share is already one and samples are still over-assigned the loop must give up
  int stuck = 0;
  for (int i = 0; diff != 0 && stuck < w; ++i) {
    if (i >= w) i = 0;
    int& n = l->num_unproc_per_train[ongoing[i]];
    if (diff > 0) {
      n += 1, diff--, stuck = 0;
    } else if (n > 1) {
      n -= 1, diff++, stuck = 0;
    } else {
      ++stuck;
    }
  }
}

std::pair<int, bool> DynamicBatchDistributor::lazy_batch_size(int batch_size) {
  DistTrainLayout* l = DistTrainSync::layout();
  int ongoing = 0;
  for (int i = 0; i < DistTrainSync::world_size(); ++i) ongoing += l->has_unproc_batches[i] ? 1 : 0;
  const int max_bs = l->num_unproc - ongoing + 1;
  if (batch_size >= max_bs) return {max_bs, true};
  return {batch_size, false};
}

std::pair<BatchRangeVec, bool> DynamicBatchDistributor::get_batch(int batch_size_in, std::string* err) {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  const int rank = DistTrainSync::rank();
  int& num_unproc = l->num_unproc_per_train[rank];
  int& num_procing = l->num_procing_per_train[rank];
  int batch_size = batch_size_in;
  bool last = false;
  if (lazy_) {
    auto bs = lazy_batch_size(batch_size);
    batch_size = bs.first;
    last = bs.second;
  } else {
    batch_size = std::min(batch_size, num_unproc);
  }
  int taken = 0;
  BatchRangeVec out;
  // ranges leave the LOWEST-index end of the ordered unprocessed set; the last one is sliced
  while (taken < batch_size) {
    if (l->unproc.n == 0) {
      if (err) *err = "unprocessed sample set ran dry before the batch was full";
      break;
    }
    const int lo = l->unproc.lo[0], hi = l->unproc.hi[0];
    const int cur = hi - lo;
    if (cur + taken <= batch_size) {
      taken += cur;
      out.emplace_back(lo, hi);
      set_insert(&l->procing, lo, hi);
      set_erase(&l->unproc, 0);
    } else {
      const int cut = lo + (batch_size - taken);
      taken += cut - lo;
      out.emplace_back(lo, cut);
      set_insert(&l->procing, lo, cut);
      set_erase(&l->unproc, 0);
      set_insert(&l->unproc, cut, hi);
    }
  }
  if (!lazy_) {
    num_unproc -= taken;
    num_procing += taken;
  }
  l->num_unproc -= taken;
  l->num_procing += taken;
  if (!lazy_) last = num_unproc == 0;
  if (last) l->has_unproc_batches[rank] = 0;
  return {out, last};
}

int DynamicBatchDistributor::query_next_batch_size(int batch_size) {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  const int max_bs = lazy_ ? l->num_unproc : l->num_unproc_per_train[DistTrainSync::rank()];
  return std::min(max_bs, batch_size);
}

bool DynamicBatchDistributor::finish_batch(const BatchRangeVec& v, bool end_of_global_batch, std::string* err) {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  const int rank = DistTrainSync::rank();
  int n = 0;
  for (auto& r : v) {
    int i = set_find(&l->procing, r.first, r.second);
    if (i < 0) {
      if (err) *err = "finish_batch: range not in the processing set";
      return false;
    }
    n += r.second - r.first;
    set_insert(&l->proced, r.first, r.second);
    set_erase(&l->procing, i);
  }
  if (!lazy_) {
    l->num_procing_per_train[rank] -= n;
    l->num_proced_per_train[rank] += n;
  }
  l->num_procing -= n;
  l->num_proced += n;
  if (end_of_global_batch) {
    if (!lazy_ && l->num_procing_per_train[rank] != 0) {
      if (err) *err = "finish_batch: samples still in flight at the end of the global batch";
      return false;
    }
    num_proced_global_batches_++;
    num_proced_sample_of_epoch_ = std::min(num_proced_sample_of_epoch_ + global_batch_size_, dataset_size_);
  }
  return true;
}

bool DynamicBatchDistributor::abort_batch(const BatchRangeVec& v, bool /*end_of_global_batch*/, std::string* err) {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  const int rank = DistTrainSync::rank();
  int n = 0;
  for (auto& r : v) {
    int i = set_find(&l->procing, r.first, r.second);
    if (i < 0) {
      if (err) *err = "abort_batch: range not in the processing set";
      return false;
    }
    n += r.second - r.first;
    set_insert(&l->unproc, r.first, r.second);
    set_erase(&l->procing, i);
  }
  if (!lazy_) {
    l->num_procing_per_train[rank] -= n;
    l->num_unproc_per_train[rank] += n;
  }
  l->num_procing -= n;
  l->num_unproc += n;
  return true;
}

bool DynamicBatchDistributor::vote_finish_last_micro_batch() {
  DistTrainLayout* l = DistTrainSync::layout();
  const int world = DistTrainSync::world_size();
  ShmLock lock(&l->db_mu);
  const int before = l->db_vote_cnt;
  if (before >= 0) l->db_vote_cnt = before + kVoteFinish;
  if (before >= 0 && before + kVoteFinish == world) {
    pthread_cond_broadcast(&l->db_vote_cond);
    return true;
  }
  if (before < 0) return false;
  while (!(l->db_vote_cnt == world || l->db_vote_cnt < 0)) cond_wait_ms(&l->db_vote_cond, &l->db_mu, -1);
  return l->db_vote_cnt >= 0;
}

void DynamicBatchDistributor::vote_abort_last_micro_batch() {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  l->db_vote_cnt = kAbortLastMicroBatch;
  pthread_cond_broadcast(&l->db_vote_cond);
}

void DynamicBatchDistributor::reset_last_micro_batch_finish_vote() {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  l->db_vote_cnt = 0;
}

void DynamicBatchDistributor::next_global_batch() {
  DistTrainLayout* l = DistTrainSync::layout();
  DistTrainSync::wait_barrier();  // every rank has finished the previous global batch
  if (DistTrainSync::rank() == 0) {
    ShmLock lock(&l->db_mu);
    const int world = DistTrainSync::world_size();
    l->db_vote_cnt = 0;
    // the last global batch of an epoch is truncated to what is left of the dataset
    int cur = global_batch_size_ + num_proced_sample_of_epoch_ > dataset_size_
                  ? dataset_size_ - num_proced_sample_of_epoch_
                  : global_batch_size_;
    if (cur < 0) cur = 0;
    l->num_unproc = cur;
    l->num_procing = 0;
    l->num_proced = 0;
    l->unproc.n = l->procing.n = l->proced.n = 0;
    if (cur > 0) {
      set_insert(&l->unproc, num_proced_sample_of_epoch_, num_proced_sample_of_epoch_ + cur);
      distribute_without_lock(false, true, true);
      if (!lazy_)
        for (int i = 0; i < world; ++i) l->num_procing_per_train[i] = l->num_proced_per_train[i] = 0;
    } else if (!lazy_) {
      for (int i = 0; i < world; ++i)
        l->num_unproc_per_train[i] = l->num_procing_per_train[i] = l->num_proced_per_train[i] = 0;
    }
  }
  DistTrainSync::wait_barrier();
}

int DynamicBatchDistributor::next_epoch(std::string* err) {
  if (first_epoch_start_) {
    if (num_proced_sample_of_epoch_ != dataset_size_ || num_proced_global_batches_ != num_global_batches_per_epoch_) {
      if (err) *err = "next_epoch before the previous epoch was finished";
      return -1;
    }
  } else {
    first_epoch_start_ = true;
  }
  int ret = next_epoch_idx_;
  next_epoch_idx_ += 1;
  num_proced_global_batches_ = 0;
  num_proced_sample_of_epoch_ = 0;
  return ret;
}

BatchRangeVec DynamicBatchDistributor::snapshot(int which) {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  const RangeSet* s = which == 0 ? &l->unproc : which == 1 ? &l->procing : &l->proced;
  BatchRangeVec out;
  for (int i = 0; i < s->n; ++i) out.emplace_back(s->lo[i], s->hi[i]);
  return out;
}

std::vector<int> DynamicBatchDistributor::counters() {
  DistTrainLayout* l = DistTrainSync::layout();
  ShmLock lock(&l->db_mu);
  std::vector<int> out{l->num_unproc, l->num_procing, l->num_proced};
  for (int i = 0; i < DistTrainSync::world_size(); ++i) {
    out.push_back(l->num_unproc_per_train[i]);
    out.push_back(l->num_procing_per_train[i]);
    out.push_back(l->num_proced_per_train[i]);
  }
  return out;
}

// ---------------------------------------------------------------------------
// PerfModel
// ---------------------------------------------------------------------------

namespace {
double thpt_locked(const DistTrainLayout* l, int bs) {
  if (l->pm_n == 0) return -1;
  if (bs <= 0) return 0;
  const int n = l->pm_n;
  if (l->pm_bs[0] >= bs) return l->pm_thpt[0] / l->pm_bs[0] * bs;
  if (l->pm_bs[n - 1] <= bs) return l->pm_thpt[n - 1] / l->pm_bs[n - 1] * bs;
  int i = static_cast<int>(std::lower_bound(l->pm_bs, l->pm_bs + n, bs) - l->pm_bs);
  if (l->pm_bs[i] == bs) return l->pm_thpt[i];
  return (l->pm_thpt[i] - l->pm_thpt[i - 1]) / (l->pm_bs[i] - l->pm_bs[i - 1]) * (bs - l->pm_bs[i - 1]) +
         l->pm_thpt[i - 1];
}
}  // namespace

void PerfModel::record_thpt(int batch_size, double batch_time_ms) {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l || batch_time_ms <= 0) return;
  const double thpt = static_cast<double>(batch_size) / batch_time_ms;
  ShmLock lock(&l->pm_mu);
  int i = static_cast<int>(std::lower_bound(l->pm_bs, l->pm_bs + l->pm_n, batch_size) - l->pm_bs);
  if (i < l->pm_n && l->pm_bs[i] == batch_size) {
    l->pm_thpt[i] = (l->pm_thpt[i] * l->pm_cnt[i] + thpt) / (l->pm_cnt[i] + 1);
    l->pm_cnt[i]++;
    return;
  }
  if (l->pm_n >= kPerfCap) return;
  for (int j = l->pm_n; j > i; --j) {
    l->pm_bs[j] = l->pm_bs[j - 1];
    l->pm_thpt[j] = l->pm_thpt[j - 1];
    l->pm_cnt[j] = l->pm_cnt[j - 1];
  }
  l->pm_bs[i] = batch_size;
  l->pm_thpt[i] = thpt;
  l->pm_cnt[i] = 1;
  l->pm_n++;
}

double PerfModel::get_thpt(int batch_size) {
  if (batch_size <= 0) return 0;
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return -1;
  ShmLock lock(&l->pm_mu);
  return thpt_locked(l, batch_size);
}

std::vector<double> PerfModel::get_thpt_vec(const std::vector<int>& batch_sizes) {
  DistTrainLayout* l = DistTrainSync::layout();
  std::vector<double> out(batch_sizes.size(), -1);
  if (!l) return out;
  ShmLock lock(&l->pm_mu);
  for (size_t i = 0; i < batch_sizes.size(); ++i) out[i] = thpt_locked(l, batch_sizes[i]);
  return out;
}

void PerfModel::clear() {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return;
  ShmLock lock(&l->pm_mu);
  l->pm_n = 0;
}

}  // namespace host
}  // namespace tch
