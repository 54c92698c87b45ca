// Training-side endpoints of the inference<->training control protocol.
// Restates pytorch/torch_col/csrc/control_stub.{h,cc}:
//   StubBase      control thread: TimedGet(1000 ms) loop on inf2tra[rank]      control_stub.cc:60-79
//                 StepsNoInteruptBegin/End = step_mutex_                        control_stub.cc:130-138
//   DummyStub     only kInferenceWorkloadDone                                    control_stub.cc:172-184
//   ColocateStub  kColocateAdjustL1/L2, kInferExit, reply via AdjustL1/L2Done   control_stub.cc:423-627
//   SwitchStub    kInterruptTrain / kResumeTrain                                 control_stub.cc:186-400
//   StubProfiler  adjust request / done timestamps (us)                          control_stub.cc:642-652
// Unknown events are reported through last_error() instead of aborting the process; the
// command word is atomic (the reference reads it without a lock).
#pragma once

#include <atomic>
#include <chrono>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "inf_tra_comm.h"

namespace tch {
namespace host {

class StubBase {
 public:
  StubBase();
  virtual ~StubBase();
  void start();  // spawns the control thread when an inference server is colocated
  void stop();
  static void stop_all();  // every running control thread; call before the shared segments are unmapped
  int cmd() const { return cmd_.load(std::memory_order_acquire); }
  void set_cmd(int c);
  void train_start();
  void train_end();
  void steps_no_interrupt_begin();
  void steps_no_interrupt_end();
  virtual void report_batch_size(int batch_size);
  bool can_exit_after_infer_workload_done();
  void set_train_first_epoch_done();
  const std::string& last_error() const { return error_; }
  // feed one message as if it had arrived on the queue (tests, and the control thread itself)
  void process(const CtrlMsgEntry& msg) { process_ctrl_msg(config_rank(), msg); }

 protected:
  virtual void process_ctrl_msg(int id, const CtrlMsgEntry& msg) = 0;
  static int config_rank();
  // stop submission, drop queued launches, wait for the launches in flight
  // (SetRejectCudaCalls(true); AbortAllStreams(); SyncAllStreams())
  size_t kill_in_flight_batch(int64_t* wait_ms);
  void reply(uint64_t id, int event, int value = 0);

  int64_t infer_workload_done_timestamp_ = 0;
  std::atomic<int> cmd_{-1};
  uint64_t cmd_id_ = 0;
  bool exec_step_ = false;
  std::mutex step_mutex_;
  std::atomic<bool> running_{false};
  std::unique_ptr<std::thread> thread_;
  std::mutex mutex_;
  std::mutex stop_mutex_;
  std::string error_;
};

class DummyStub : public StubBase {
 protected:
  void process_ctrl_msg(int id, const CtrlMsgEntry& msg) override;
};

class ColocateStub : public StubBase {
 public:
  explicit ColocateStub(int batch_size) : input_batch_size_(batch_size), current_bs_(batch_size) {}
  int target_batch_size();
  int unpub_target_batch_size();
  void adjust_l1_done();
  void adjust_l2_done();
  double passed_time_from_set_cmd_ms();
  void report_batch_size(int batch_size) override;
  void set_killed_batch_recover() { has_killed_batch_recover_.store(true, std::memory_order_release); }
  void set_killed_batch_reconfiged() { will_killed_batch_reconfig_.store(false, std::memory_order_release); }

 protected:
  void process_ctrl_msg(int id, const CtrlMsgEntry& msg) override;

 private:
  int input_batch_size_, current_bs_;
  std::atomic<bool> has_killed_batch_recover_{true};
  std::atomic<bool> will_killed_batch_reconfig_{false};
  std::chrono::steady_clock::time_point set_cmd_time_;
};

class SwitchStub : public StubBase {
 public:
  bool try_interrupt_train_done(bool barrier);
  void set_killed_batch_recover() { has_killed_batch_recover_.store(true, std::memory_order_release); }
  void train_resume_done();
  bool prepare_resume();
  void set_global_interrupt_flag(bool flag);
  bool global_interrupt_flag();
  void set_global_has_batch_killed(bool flag);
  bool global_has_batch_killed();

 protected:
  void process_ctrl_msg(int id, const CtrlMsgEntry& msg) override;

 private:
  bool try_interrupt_train_done_locked(bool barrier);
  uint64_t last_reply_cmd_id_ = 0;
  std::atomic<bool> has_killed_batch_recover_{true};
};

struct StubProfiler {
  static void record_adjust_request();
  static void record_adjust_done();
  static std::vector<int64_t> adjust_request_time_stamps();
  static std::vector<int64_t> adjust_done_time_stamps();
  static void clear();
};

}  // namespace host
}  // namespace tch
