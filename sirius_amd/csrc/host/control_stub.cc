#include "control_stub.h"

#include "../context.h"
#include "config.h"
#include "dist_train.h"

namespace tch {
namespace host {

namespace {
std::mutex g_prof_mu;
std::vector<int64_t> g_adjust_request, g_adjust_done;
// stubs whose control thread is running: the thread blocks on the shared segment, so it has to
// be stopped before the segment goes away
std::mutex g_live_mu;
std::vector<StubBase*> g_live;
}  // namespace

void StubBase::stop_all() {
  std::vector<StubBase*> live;
  {
    std::lock_guard<std::mutex> l(g_live_mu);
    live = g_live;
  }
  for (StubBase* s : live) s->stop();
}

void StubProfiler::record_adjust_request() {
  std::lock_guard<std::mutex> l(g_prof_mu);
  g_adjust_request.push_back(unix_timestamp_us());
}
void StubProfiler::record_adjust_done() {
  std::lock_guard<std::mutex> l(g_prof_mu);
  g_adjust_done.push_back(unix_timestamp_us());
}
std::vector<int64_t> StubProfiler::adjust_request_time_stamps() {
  std::lock_guard<std::mutex> l(g_prof_mu);
  return g_adjust_request;
}
std::vector<int64_t> StubProfiler::adjust_done_time_stamps() {
  std::lock_guard<std::mutex> l(g_prof_mu);
  return g_adjust_done;
}
void StubProfiler::clear() {
  std::lock_guard<std::mutex> l(g_prof_mu);
  g_adjust_request.clear();
  g_adjust_done.clear();
}

// ---------------------------------------------------------------------------
StubBase::StubBase() = default;

StubBase::~StubBase() { stop(); }

int StubBase::config_rank() { return config().train_rank; }

void StubBase::start() {
  if (!config().has_colocated_infer_server || !communicator() || thread_) return;
  running_.store(true);
  {
    std::lock_guard<std::mutex> l(g_live_mu);
    g_live.push_back(this);
  }
  thread_.reset(new std::thread([this] {
    while (running_.load()) {
      CtrlMsgEntry msg;
      // a counted reference per wait: a shutdown on another thread cannot unmap the queue under this one
      auto comm = communicator();
      if (!comm) break;
      if (comm->timed_get(1000, kInf2Tra, config_rank(), &msg)) process_ctrl_msg(config_rank(), msg);
    }
  }));
}

void StubBase::stop() {
  std::lock_guard<std::mutex> stop_lock(stop_mutex_);
  if (thread_) {
    running_.store(false);
    thread_->join();
    thread_.reset();
    std::lock_guard<std::mutex> l(g_live_mu);
    for (size_t i = 0; i < g_live.size(); ++i)
      if (g_live[i] == this) {
        g_live.erase(g_live.begin() + i);
        break;
      }
  }
}

void StubBase::set_cmd(int c) {
  std::lock_guard<std::mutex> l(mutex_);
  cmd_.store(c, std::memory_order_release);
}

void StubBase::reply(uint64_t id, int event, int value) {
  if (auto comm = communicator()) comm->put(CtrlMsgEntry{id, event, value}, kTra2Inf, config_rank());
}

void StubBase::train_start() {
  if (config().has_colocated_infer_server && config_rank() == 0) reply(0, kTrainStart);
}

void StubBase::train_end() {
  if (config().has_colocated_infer_server && config_rank() == 0) reply(0, kTrainEnd);
}

void StubBase::report_batch_size(int batch_size) {
  if (config().has_colocated_infer_server) reply(0, kReportBatchSize, batch_size);
}

void StubBase::steps_no_interrupt_begin() {
  step_mutex_.lock();
  exec_step_ = true;
}

void StubBase::steps_no_interrupt_end() {
  exec_step_ = false;
  step_mutex_.unlock();
}

bool StubBase::can_exit_after_infer_workload_done() {
  constexpr int64_t kWaitMs = 30 * 1000;
  if (infer_workload_done_timestamp_ == 0) return false;
  return unix_timestamp_ms() - infer_workload_done_timestamp_ > kWaitMs;
}

void StubBase::set_train_first_epoch_done() {
  if (!config().has_colocated_infer_server) return;
  if (auto comm = communicator()) comm->update_field(config_rank(), kFieldFirstEpochDone, 1);
}

size_t StubBase::kill_in_flight_batch(int64_t* wait_ms) {
  const int64_t t1 = unix_timestamp_ms();
  set_reject_calls(true);
  const size_t removed = abort_all_streams();
  const int64_t t2 = unix_timestamp_ms();
  sync_all_streams();
  if (wait_ms) *wait_ms = unix_timestamp_ms() - t2;
  (void)t1;
  return removed;
}

// ---------------------------------------------------------------------------
void DummyStub::process_ctrl_msg(int, const CtrlMsgEntry& msg) {
  std::lock_guard<std::mutex> l(mutex_);
  if (msg.event == kInferenceWorkloadDone) {
    infer_workload_done_timestamp_ = unix_timestamp_ms();
  } else {
    error_ = "[DummyStub] Unknown command: " + std::to_string(msg.event) + " (id " + std::to_string(msg.id) + ")";
  }
}

// ---------------------------------------------------------------------------
int ColocateStub::target_batch_size() {
  std::lock_guard<std::mutex> l(mutex_);
  if (config().has_colocated_infer_server)
    if (auto comm = communicator()) return comm->get_field(config_rank(), kFieldTargetBatchSize);
  return input_batch_size_;
}

int ColocateStub::unpub_target_batch_size() {
  std::lock_guard<std::mutex> l(mutex_);
  if (config().has_colocated_infer_server)
    if (auto comm = communicator()) return comm->get_field(config_rank(), kFieldTargetBatchSizeUnpublished);
  return input_batch_size_;
}

void ColocateStub::process_ctrl_msg(int, const CtrlMsgEntry& msg) {
  std::lock_guard<std::mutex> l(mutex_);
  switch (msg.event) {
    case kColocateAdjustL1:
    case kColocateAdjustL2: {
      const bool should_kill = config().kill_batch_on_recv && msg.event == kColocateAdjustL1 &&
                               cmd_.load() != kColocateAdjustL1;
      if (should_kill && !has_killed_batch_recover_.load(std::memory_order_acquire)) {
        // the previous kill has not been recovered yet: nothing more to free, reply at once
        reply(msg.id, msg.event == kColocateAdjustL1 ? kColocateAdjustL1Done : kColocateAdjustL2Done);
        break;
      }
      has_killed_batch_recover_.store(false);
      will_killed_batch_reconfig_.store(true);
      if (should_kill) {
        // waits out an optimizer step in progress, then cuts the micro-batch between launches
        std::lock_guard<std::mutex> step(step_mutex_);
        kill_in_flight_batch(nullptr);
      }
      cmd_id_ = msg.id;
      set_cmd_time_ = std::chrono::steady_clock::now();
      cmd_.store(msg.event, std::memory_order_release);
      StubProfiler::record_adjust_request();
      break;
    }
    case kInferExit: {
      auto comm = communicator();
      if (config_rank() != 0 || !comm) break;
      if (config().is_colocate_l1 && will_killed_batch_reconfig_.load(std::memory_order_acquire)) break;
      std::vector<int> cur = comm->get_field_vec(kFieldTargetBatchSize);
      std::vector<int> unpub = comm->get_field_vec(kFieldTargetBatchSizeUnpublished);
      bool all_same = true;
      for (size_t i = 0; i < cur.size() && i < unpub.size(); ++i) all_same = all_same && cur[i] == unpub[i];
      if (!all_same && DynamicBatchDistributor::get()) DynamicBatchDistributor::get()->distribute_batch(true, false, false);
      break;
    }
    case kInferenceWorkloadDone:
      infer_workload_done_timestamp_ = unix_timestamp_ms();
      break;
    default:
      error_ = "[ColocateStub] Unknown command: " + std::to_string(msg.event) + " (id " + std::to_string(msg.id) + ")";
  }
}

void ColocateStub::adjust_l1_done() {
  std::lock_guard<std::mutex> l(mutex_);
  if (cmd_.load() == kColocateAdjustL1) {
    reply(cmd_id_, kColocateAdjustL1Done);
    cmd_.store(-1, std::memory_order_release);
    cmd_id_ = 0;
    set_reject_calls(false);
    StubProfiler::record_adjust_done();
  }
}

void ColocateStub::adjust_l2_done() {
  std::lock_guard<std::mutex> l(mutex_);
  if (cmd_.load() == kColocateAdjustL2) {
    reply(cmd_id_, kColocateAdjustL2Done);
    cmd_.store(-1, std::memory_order_release);
    cmd_id_ = 0;
    StubProfiler::record_adjust_done();
  }
}

double ColocateStub::passed_time_from_set_cmd_ms() {
  return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - set_cmd_time_).count();
}

void ColocateStub::report_batch_size(int batch_size) {
  current_bs_ = batch_size;
  StubBase::report_batch_size(batch_size);
}

// ---------------------------------------------------------------------------
void SwitchStub::set_global_interrupt_flag(bool flag) {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return;
  ShmLock lock(&l->sw_mu);
  l->sw_interrupt_flag = flag ? 1 : 0;
}
bool SwitchStub::global_interrupt_flag() {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return false;
  ShmLock lock(&l->sw_mu);
  return l->sw_interrupt_flag != 0;
}
void SwitchStub::set_global_has_batch_killed(bool flag) {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return;
  ShmLock lock(&l->sw_mu);
  l->sw_has_batch_killed = flag ? 1 : 0;
}
bool SwitchStub::global_has_batch_killed() {
  DistTrainLayout* l = DistTrainSync::layout();
  if (!l) return false;
  ShmLock lock(&l->sw_mu);
  return l->sw_has_batch_killed != 0;
}

void SwitchStub::process_ctrl_msg(int, const CtrlMsgEntry& msg) {
  std::lock_guard<std::mutex> l(mutex_);
  const bool master = config_rank() == 0;
  switch (msg.event) {
    case kInterruptTrain:
      if (cmd_.load() == kInterruptTrain && cmd_id_ == 0) {
        // already interrupted and acknowledged: acknowledge the repeat at once
        cmd_id_ = msg.id;
        last_reply_cmd_id_ = cmd_id_;
        if (master) reply(cmd_id_, kInterruptTrainDone);
        cmd_id_ = 0;
      } else {
        if (master) {
          set_global_interrupt_flag(true);
          set_global_has_batch_killed(false);
        }
        if (config().kill_batch_on_recv && has_killed_batch_recover_.load()) {
          std::lock_guard<std::mutex> step(step_mutex_);
          kill_in_flight_batch(nullptr);
          has_killed_batch_recover_.store(false);
        }
        cmd_id_ = msg.id;
        cmd_.store(kInterruptTrain, std::memory_order_release);
      }
      break;
    case kResumeTrain:
      if (cmd_.load() == kInterruptTrain && cmd_id_ == 0) {
        cmd_.store(kResumeTrain, std::memory_order_release);
        set_global_interrupt_flag(false);
      }
      break;
    case kInferenceWorkloadDone:
      infer_workload_done_timestamp_ = unix_timestamp_ms();
      break;
    default:
      error_ = "[SwitchStub] Unknown command: " + std::to_string(msg.event) + " (id " + std::to_string(msg.id) + ")";
  }
}

bool SwitchStub::try_interrupt_train_done(bool barrier) {
  std::lock_guard<std::mutex> l(mutex_);
  return try_interrupt_train_done_locked(barrier);
}

bool SwitchStub::try_interrupt_train_done_locked(bool barrier) {
  if (cmd_id_ > last_reply_cmd_id_) {
    const uint64_t id = cmd_id_;
    last_reply_cmd_id_ = cmd_id_;
    cmd_id_ = 0;
    set_reject_calls(false);
    if (barrier) DistTrainSync::wait_barrier();
    if (config_rank() == 0) reply(id, kInterruptTrainDone);
    return true;
  }
  return false;
}

void SwitchStub::train_resume_done() {
  if (config_rank() == 0) {
    std::lock_guard<std::mutex> l(mutex_);
    reply(0, kResumeTrainDone);
  }
}

bool SwitchStub::prepare_resume() {
  std::lock_guard<std::mutex> l(mutex_);
  if (cmd_.load() == kInterruptTrain && cmd_id_ != 0) set_global_interrupt_flag(true);
  DistTrainSync::wait_barrier();
  const bool resume = !global_interrupt_flag();
  DistTrainSync::wait_barrier();
  if (!resume) {
    try_interrupt_train_done_locked(false);
    DistTrainSync::wait_barrier();
    return false;
  }
  cmd_.store(kResumeTrain, std::memory_order_release);
  has_killed_batch_recover_.store(true);
  DistTrainSync::wait_barrier();
  if (config_rank() == 0) reply(0, kResumeTrainDone);
  return true;
}

}  // namespace host
}  // namespace tch
