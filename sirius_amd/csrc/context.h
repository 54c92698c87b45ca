// Execution context of the device operators: which HIP stream launches go to,
// whether they pass through a preemptible launch queue, and whether they are
// being recorded into a replayable program instead of being launched.
//
// The launch queue restates, for HIP and without interposing on the driver,
// what the reference gets from xsched in STOP_SUBMISSION mode
// (common/xsched_ctrl.cc:27-46 creates the queue with length 16 and sync
// interval 8; third_party/xsched/preempt/xqueue/worker.cpp:155-260 bounds the
// commands in flight; xqueue.cpp:150-152 / wait_queue.cpp:135-148 erase the
// not-yet-submitted ones on abort; shim/cuda/intercept.cpp:20-22 turns every
// call into a successful no-op while the reject flag is set).
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "kernels.h"

namespace tch {

class LaunchQueue {
 public:
  LaunchQueue(hipStream_t stream, int queue_length, int sync_interval);
  ~LaunchQueue();
  LaunchQueue(const LaunchQueue&) = delete;
  LaunchQueue& operator=(const LaunchQueue&) = delete;

  // `on` (optional): the stream to launch on instead of the registered one (the second lane of a program, or a
  // stream restricted to a share of the compute units).  Launches on different streams are ordered only by
  // the dependencies the caller queues between them, exactly as when the caller launches directly; the bound
  // on launches in flight holds over all streams together.
  void submit(const LaunchRecord& rec, hipStream_t on = nullptr);
  // Queued in order with the launches: everything given to `to` afterwards waits for what `from` holds now.
  void submit_dependency(hipStream_t from, hipStream_t to);
  // Erase every launch that has not been handed to the hardware queue yet.
  size_t clear();
  // Wait until everything submitted before this call has finished on the GPU.
  // Returns 0 on success, a HIP error code otherwise.
  int synchronize();
  // Stop handing launches to the hardware queue (what is already there runs on; with sync_hw the call
  // returns once it has finished) / go on, optionally dropping what was queued meanwhile.  Another tenant's
  // work submitted in between runs ahead of everything this queue still holds
  // (third_party/xsched/preempt/xqueue/xqueue.cpp:80-137, Suspend / Resume).
  void suspend(bool sync_hw);
  void resume(bool drop_commands);
  // Launches still waiting in the software queue.
  size_t size();
  // Launches handed to the stream and not yet known to be complete.
  size_t in_flight();
  hipStream_t stream() const { return stream_; }
  int sticky_error() const { return error_.load(); }
  uint64_t submitted_total() const { return submitted_total_.load(); }

 private:
  struct Item {
    bool is_sync = false;
    bool is_dependency = false;
    uint64_t sync_ticket = 0;
    hipStream_t on = nullptr;    // launch stream override / dependency source
    hipStream_t to = nullptr;    // dependency target
    LaunchRecord rec;
  };
  struct Logged {
    uint64_t idx;
    hipEvent_t event;    // nullptr unless this command carries a sync point (of its own stream)
    hipStream_t stream;  // where it was launched
  };
  struct StreamState {
    hipStream_t stream;
    uint64_t since_event;  // launches on the stream since its last sync point
  };
  void worker_loop();
  void launch_one(const LaunchRecord& rec, hipStream_t on, bool fork_follows);
  void chain(hipStream_t from, hipStream_t to);
  void drain_log_until(size_t keep);
  void sync_everything();
  StreamState& state_of(hipStream_t s);
  hipEvent_t take_event();

  hipStream_t stream_;
  const size_t queue_length_;
  const uint64_t sync_interval_;
  int device_ = 0;

  std::mutex mu_;
  std::condition_variable cv_work_;
  std::condition_variable cv_done_;
  std::deque<Item> wait_;
  bool stop_ = false;
  bool suspended_ = false, parked_ = false, park_sync_ = false;
  std::condition_variable cv_park_;
  uint64_t next_ticket_ = 1;
  uint64_t done_ticket_ = 0;

  // worker-private
  std::deque<Logged> log_;
  std::vector<hipEvent_t> free_events_;
  hipEvent_t fork_event_ = nullptr;   // stop event of the launch just made, for a dependency entry right behind it
  hipStream_t fork_from_ = nullptr;
  std::vector<StreamState> streams_;  // every stream a launch went to since the last full synchronisation
  uint64_t next_idx_ = 0;

  std::atomic<size_t> in_flight_{0};
  std::atomic<int> error_{0};
  std::atomic<uint64_t> submitted_total_{0};
  std::thread worker_;
};

// A recorded sequence of launches, replayed through a context.
struct Program {
  std::vector<LaunchRecord> launches;
};

class Context {
 public:
  explicit Context(hipStream_t s) : stream(s) {}
  ~Context();
  hipStream_t stream;
  // second stream (default priority) for lane-1 launches of a replayed program; made on first use
  hipStream_t side = nullptr;
  // Compute-unit share: with a limit in force the launches go to a pair of streams whose CU mask keeps
  // the highest-numbered `cu_limit` compute units (made once per limit, kept for the process); 0 = no
  // limit, launches go to `stream` / `side`.
  int cu_limit = 0;
  hipStream_t masked_main = nullptr, masked_side = nullptr;
  int set_cu_limit(int n_cus);
  hipStream_t main_stream() const { return cu_limit > 0 ? masked_main : stream; }
  // everything given to `to` afterwards waits for what `from` holds now (direct or through the queue)
  int depend(hipStream_t from, hipStream_t to);
  bool side_dirty = false;  // lane 1 was given work since the last join
  // A join one point behind (kOpJoinBehind) goes through a stream of its own that carries nothing but waits:
  // at such a point it is made to wait for lane 1, and lane 0 waits for it at the next one.
  hipStream_t relay = nullptr;
  bool relay_dirty = false;  // the relay waits for lane-1 work that lane 0 has not waited for
  // recording state: the lane new launches are stamped with, and whether the next lane-1 launch
  // has to wait for lane 0
  int lane = 0;
  bool wait_main = false;
  int record_join(bool behind = false);
  // work reached lane 0's stream from outside this context: the next fork has to wait for it
  void note_foreign_work() { main_since_fork_ = true; }
  int synchronize();  // both streams
  // set while the stream is registered for preemption; owned by the registry
  std::shared_ptr<LaunchQueue> queue;
  Program* recording = nullptr;
  // launches skipped because the reject flag was up since the last reset
  std::atomic<uint64_t> rejected{0};
  // A split reduction that was not launched with its weight gradient: it rides the next weight-gradient launch of
  // this context as extra workgroups (conv2d_wgrad with trailing = 1), or goes out with conv2d_wgrad_flush.
  struct {
    bool valid = false;
    ReduceArgs args{};
    unsigned blocks = 0;
    double bytes = 0.0;
  } trailing_reduce;

  // `next`: the record that follows in the program being replayed (nullptr: none or unknown).  A lane-0 launch
  // that is followed by a lane-1 launch which has to wait for it carries the event of that wait as its own stop
  // event (the kernel's completion signal), so that no separate event record stands between it and the next
  // lane-0 kernel in the queue.
  int dispatch(const LaunchRecord& rec, const LaunchRecord* next = nullptr);

  // Timing of one kernel family INSIDE a plain replay (both lanes, nothing added between launches): while
  // timed_name is set, every direct launch of a kernel of that name carries a start and a stop event of its
  // own (the launch's own begin / end timestamps), collected in timed_events.
  const char* timed_name = nullptr;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timed_events;

 private:
  int launch_direct(hipStream_t s, const LaunchRecord& rec, hipEvent_t stop);
  hipEvent_t next_event();
  hipEvent_t fork_event_ = nullptr;  // stop event of the last lane-0 launch, not yet waited for by lane 1
  // lane 0 was given a launch since lane 1 last waited for it (a fork with nothing new to wait for is skipped)
  bool main_since_fork_ = true;
  std::vector<hipEvent_t> events_;
  size_t event_next_ = 0;
};

struct KernelStat {
  std::string name;
  double total_ms = 0.0;
  double work = 0.0;  // sum of the algorithmic work of the launches
  int64_t launches = 0;
  int work_is_bytes = 1;
  double bytes = 0.0;  // sum of the algorithmic bytes of the launches (0 where a flops-annotated launch gave none)
};

// One launch of a program as the profiler saw it (entries that are not kernel launches keep an empty name).
struct LaunchStat {
  std::string name;
  double ms = 0.0;     // mean HIP-event time over the repetitions
  double flops = 0.0;  // algorithmic flops (0 for a launch annotated with bytes only)
  double bytes = 0.0;  // algorithmic bytes
  int lane = 0;
  int64_t grid = 0;    // workgroups
};

// Replays prog `reps` times directly on the context's stream with a HIP event between any
// two launches and sums the elapsed time per kernel name (`out`) and / or per launch (`per_launch`,
// one entry per program position).
int profile_program(Context* ctx, const Program& prog, int reps, std::vector<KernelStat>* out,
                    std::vector<LaunchStat>* per_launch = nullptr);

// Replays prog `reps` times as it runs (tch_program_run: two lanes, no launch queue) and measures the launches
// of the kernel called `name` with the begin / end timestamps of each launch itself: their mean duration in
// microseconds while the rest of the program shares the chip with them, and how many there are per replay.
int time_kernel_in_program(Context* ctx, const Program& prog, const char* name, int reps, double* mean_us,
                           int64_t* launches_per_replay);

// ---- process-wide registry of preemptible streams (xsched_ctrl equivalent) ----
uint64_t register_stream(uint64_t stream);  // returns a handle, 0 on failure
int unregister_stream(uint64_t stream);
void unregister_all_streams();
std::shared_ptr<LaunchQueue> queue_for_stream(uint64_t stream);
size_t abort_stream(uint64_t stream);
size_t abort_all_streams();
int sync_stream(uint64_t stream);
int sync_all_streams();
size_t queue_size(uint64_t stream);
size_t queue_size_all_streams();
void suspend_all_streams(bool sync_hw);
void resume_all_streams(bool drop_commands);
void set_reject_calls(bool reject);
bool query_reject_calls();
void set_queue_shape(int queue_length, int sync_interval);

// ---- compute-unit partitioning between training and a colocated tenant (the reference's SMPartitioner,
// common/sm_partition.cc:26-112, with compute units in the place of TPCs) ----
int cu_partition_init(int total_cus, int min_train_cus, int max_train_cus);  // total_cus <= 0: ask the device
int cu_partition_total();
// max(min, total - required) capped at max: what training may use while the other tenant needs `required`
int cu_partition_train_avail(int infer_required_cus);
// a stream (default priority) whose CU mask keeps the highest-numbered n compute units; lane 0 / 1
hipStream_t cu_partition_stream(int n_cus, int lane);

const char* last_error();

}  // namespace tch
