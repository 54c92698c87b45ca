#include "context.h"

#include <hip/hip_ext.h>
#include <stdlib.h>
#include <string.h>

#include <map>

namespace tch {

namespace {
thread_local std::string g_error;
std::atomic<bool> g_reject{false};
std::mutex g_stream_mu;
std::map<uint64_t, std::shared_ptr<LaunchQueue>> g_streams;
int g_queue_length = 16;
// A sync point is an event behind every 4th launch of a stream (the reference asks xsched for one every 8): with
// two lanes feeding 16 slots, a full queue then waits for 4 instead of 8 launches of one lane to finish, which
// is worth 1.2 ms per ResNet-152 step here; one per launch costs more in event records than it saves.
int g_sync_interval = 4;

int launch_now(hipStream_t stream, const LaunchRecord& rec, hipEvent_t stop_event = nullptr) {
  void* args[1] = {const_cast<unsigned char*>(rec.args)};
  hipError_t e = stop_event ? hipExtLaunchKernel(rec.fn, rec.grid, rec.block, args, 0, stream, nullptr, stop_event, 0)
                           : hipLaunchKernel(rec.fn, rec.grid, rec.block, args, 0, stream);
  if (e != hipSuccess) {
    set_error(std::string("hipLaunchKernel failed: ") + hipGetErrorString(e));
    return -5;
  }
  return 0;
}

// TCH_FORK_STOP_EVENT=0: every fork to the second lane records an event of its own behind the lane-0 kernel
bool fork_by_stop_event() {
  static const bool on = [] {
    const char* e = getenv("TCH_FORK_STOP_EVENT");
    return !(e && atoi(e) == 0);
  }();
  return on;
}
}  // namespace

void set_error(const std::string& msg) { g_error = msg; }
const char* last_error() { return g_error.c_str(); }

// ---------------------------------------------------------------------------
// LaunchQueue
// ---------------------------------------------------------------------------

LaunchQueue::LaunchQueue(hipStream_t stream, int queue_length, int sync_interval)
    : stream_(stream),
      queue_length_(queue_length < 1 ? 1 : static_cast<size_t>(queue_length)),
      sync_interval_(sync_interval < 1 ? 1 : static_cast<uint64_t>(sync_interval)) {
  if (hipGetDevice(&device_) != hipSuccess) device_ = 0;
  worker_ = std::thread([this] { worker_loop(); });
}

LaunchQueue::~LaunchQueue() {
  {
    std::lock_guard<std::mutex> lock(mu_);
    stop_ = true;
  }
  cv_work_.notify_all();
  cv_park_.notify_all();
  if (worker_.joinable()) worker_.join();
  for (auto& l : log_)
    if (l.event) (void)hipEventDestroy(l.event);
  for (auto e : free_events_) (void)hipEventDestroy(e);
}

void LaunchQueue::submit(const LaunchRecord& rec, hipStream_t on) {
  {
    std::lock_guard<std::mutex> lock(mu_);
    wait_.emplace_back();
    wait_.back().rec = rec;
    wait_.back().on = on;
  }
  cv_work_.notify_one();
}

void LaunchQueue::submit_dependency(hipStream_t from, hipStream_t to) {
  {
    std::lock_guard<std::mutex> lock(mu_);
    wait_.emplace_back();
    wait_.back().is_dependency = true;
    wait_.back().on = from;
    wait_.back().to = to;
  }
  cv_work_.notify_one();
}

void LaunchQueue::chain(hipStream_t from, hipStream_t to) {
  if (from == to) return;
  hipEvent_t ev = take_event();
  if (!ev || hipEventRecord(ev, from) != hipSuccess || hipStreamWaitEvent(to, ev, 0) != hipSuccess)
    error_.store(static_cast<int>(hipErrorUnknown));
  // the event may be recorded again once the wait is enqueued (the wait holds its own reference to the
  // recorded state)
  if (ev) free_events_.push_back(ev);
}

void LaunchQueue::suspend(bool sync_hw) {
  std::unique_lock<std::mutex> lock(mu_);
  if (stop_) return;
  if (suspended_ && parked_ && !sync_hw) return;
  suspended_ = true;
  parked_ = false;
  park_sync_ = sync_hw;
  cv_work_.notify_all();
  cv_park_.wait(lock, [&] { return parked_ || stop_; });
}

void LaunchQueue::resume(bool drop_commands) {
  {
    std::lock_guard<std::mutex> lock(mu_);
    if (drop_commands)
      for (auto it = wait_.begin(); it != wait_.end();) it = (!it->is_sync && !it->is_dependency) ? wait_.erase(it) : it + 1;
    suspended_ = false;
    parked_ = false;
  }
  cv_work_.notify_all();
}

size_t LaunchQueue::clear() {
  std::lock_guard<std::mutex> lock(mu_);
  size_t removed = 0;
  for (auto it = wait_.begin(); it != wait_.end();) {
    if (!it->is_sync && !it->is_dependency) {
      it = wait_.erase(it);
      ++removed;
    } else {
      ++it;
    }
  }
  return removed;
}

int LaunchQueue::synchronize() {
  std::unique_lock<std::mutex> lock(mu_);
  if (stop_) return 0;
  const uint64_t ticket = next_ticket_++;
  wait_.emplace_back();
  wait_.back().is_sync = true;
  wait_.back().sync_ticket = ticket;
  cv_work_.notify_one();
  cv_done_.wait(lock, [&] { return done_ticket_ >= ticket; });
  return error_.load();
}

size_t LaunchQueue::size() {
  std::lock_guard<std::mutex> lock(mu_);
  size_t n = 0;
  // stream dependencies count: whoever waits for the queue to empty before giving the stream work of
  // its own (copies, read-backs) relies on the trailing dependency of a compute-unit-limited run
  for (auto& it : wait_)
    if (!it.is_sync) ++n;
  return n;
}

size_t LaunchQueue::in_flight() { return in_flight_.load(); }

hipEvent_t LaunchQueue::take_event() {
  if (!free_events_.empty()) {
    hipEvent_t e = free_events_.back();
    free_events_.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return nullptr;
  return e;
}

LaunchQueue::StreamState& LaunchQueue::state_of(hipStream_t s) {
  for (auto& st : streams_)
    if (st.stream == s) return st;
  streams_.push_back(StreamState{s, 0});
  return streams_.back();
}

// Every stream that was given a launch, and the registered one, have finished when this returns.
void LaunchQueue::sync_everything() {
  bool seen_own = false;
  for (auto& st : streams_) {
    hipError_t e = hipStreamSynchronize(st.stream);
    if (e != hipSuccess) error_.store(static_cast<int>(e));
    seen_own = seen_own || st.stream == stream_;
  }
  if (!seen_own) {
    hipError_t e = hipStreamSynchronize(stream_);
    if (e != hipSuccess) error_.store(static_cast<int>(e));
  }
  streams_.clear();
  for (auto& l : log_)
    if (l.event) free_events_.push_back(l.event);
  log_.clear();
  in_flight_.store(0);
}

// Wait on the oldest sync point so that at most `keep` commands stay logged.  A sync point speaks for the
// launches that went to its own stream before it; those of other streams stay logged.
void LaunchQueue::drain_log_until(size_t keep) {
  while (log_.size() > keep) {
    size_t pos = 0;
    bool found = false;
    for (; pos < log_.size(); ++pos) {
      if (log_[pos].event) {
        found = true;
        break;
      }
    }
    if (!found) {
      sync_everything();
      break;
    }
    hipError_t e = hipEventSynchronize(log_[pos].event);
    if (e != hipSuccess) error_.store(static_cast<int>(e));
    const hipStream_t done = log_[pos].stream;
    free_events_.push_back(log_[pos].event);
    std::deque<Logged> rest;
    for (size_t i = 0; i < log_.size(); ++i)
      if (i > pos || log_[i].stream != done) rest.push_back(log_[i]);
    log_.swap(rest);
  }
  in_flight_.store(log_.size());
}

void LaunchQueue::launch_one(const LaunchRecord& rec, hipStream_t on, bool fork_follows) {
  if (log_.size() >= queue_length_) drain_log_until(queue_length_ - 1);
  hipStream_t target = on ? on : stream_;
  void* args[1] = {const_cast<unsigned char*>(rec.args)};
  // a launch that a dependency on its stream follows carries that dependency's event as its stop event
  hipEvent_t stop = fork_follows ? take_event() : nullptr;
  hipError_t e = stop ? hipExtLaunchKernel(rec.fn, rec.grid, rec.block, args, 0, target, nullptr, stop, 0)
                      : hipLaunchKernel(rec.fn, rec.grid, rec.block, args, 0, target);
  if (e != hipSuccess) {
    if (stop) free_events_.push_back(stop);
    error_.store(static_cast<int>(e));
    return;
  }
  fork_event_ = stop;
  fork_from_ = target;
  const uint64_t idx = ++next_idx_;
  StreamState& st = state_of(target);
  hipEvent_t ev = nullptr;
  if (++st.since_event >= sync_interval_) {
    ev = take_event();
    if (ev && hipEventRecord(ev, target) == hipSuccess) {
      st.since_event = 0;
    } else if (ev) {
      free_events_.push_back(ev);
      ev = nullptr;
    }
  }
  log_.push_back(Logged{idx, ev, target});
  in_flight_.store(log_.size());
  submitted_total_.fetch_add(1);
}

void LaunchQueue::worker_loop() {
  (void)hipSetDevice(device_);
  for (;;) {
    Item item;
    bool fork_follows = false;
    {
      std::unique_lock<std::mutex> lock(mu_);
      cv_work_.wait(lock, [&] { return stop_ || (suspended_ ? !parked_ : !wait_.empty()); });
      if (suspended_ && !stop_) {
        // park: nothing more goes to the hardware queue until resume()
        const bool sync = park_sync_;
        if (sync) {
          lock.unlock();
          sync_everything();
          lock.lock();
        }
        parked_ = true;
        cv_park_.notify_all();
        continue;
      }
      if (wait_.empty()) {
        if (stop_) break;
        continue;
      }
      item = wait_.front();
      wait_.pop_front();
      fork_follows = !item.is_dependency && !item.is_sync && fork_by_stop_event() && !wait_.empty() &&
                     wait_.front().is_dependency && wait_.front().on == (item.on ? item.on : stream_);
    }
    if (item.is_dependency) {
      if (fork_event_ && fork_from_ == item.on && item.to != item.on) {
        // the launch before this entry signals fork_event_ when it ends; as in chain(), the event may be used
        // again once the wait is enqueued
        if (hipStreamWaitEvent(item.to, fork_event_, 0) != hipSuccess) error_.store(static_cast<int>(hipErrorUnknown));
        free_events_.push_back(fork_event_);
        fork_event_ = nullptr;
      } else {
        chain(item.on, item.to);
      }
      continue;
    }
    if (fork_event_) {   // nobody asked for it after all
      free_events_.push_back(fork_event_);
      fork_event_ = nullptr;
    }
    if (item.is_sync) {
      sync_everything();
      {
        std::lock_guard<std::mutex> lock(mu_);
        done_ticket_ = item.sync_ticket;
      }
      cv_done_.notify_all();
    } else {
      launch_one(item.rec, item.on, fork_follows);
    }
  }
  // release waiters that raced with shutdown
  {
    std::lock_guard<std::mutex> lock(mu_);
    done_ticket_ = next_ticket_;
  }
  cv_done_.notify_all();
}

// ---------------------------------------------------------------------------
// Context
// ---------------------------------------------------------------------------

Context::~Context() {
  if (side) {
    (void)hipStreamSynchronize(side);
    (void)hipStreamDestroy(side);
  }
  if (relay) {
    (void)hipStreamSynchronize(relay);
    (void)hipStreamDestroy(relay);
  }
  for (hipEvent_t e : events_) (void)hipEventDestroy(e);
}

hipEvent_t Context::next_event() {
  constexpr size_t kRing = 64;
  if (events_.size() < kRing) {
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return nullptr;
    events_.push_back(e);
    return e;
  }
  return events_[event_next_++ % kRing];
}

int Context::record_join(bool behind) {
  if (!recording) return 0;
  LaunchRecord rec{};
  rec.fn = nullptr;
  rec.name = behind ? "join_behind" : "join";
  rec.op = behind ? kOpJoinBehind : kOpJoin;
  recording->launches.push_back(rec);
  return 0;
}

int Context::depend(hipStream_t from, hipStream_t to) {
  if (from == to) return 0;
  if (queue) {
    queue->submit_dependency(from, to);
    return 0;
  }
  hipEvent_t e = next_event();
  if (!e || hipEventRecord(e, from) != hipSuccess || hipStreamWaitEvent(to, e, 0) != hipSuccess) {
    set_error("stream dependency failed");
    return -5;
  }
  return 0;
}

int Context::set_cu_limit(int n_cus) {
  const int total = cu_partition_total();
  if (n_cus <= 0 || (total > 0 && n_cus >= total)) n_cus = 0;
  if (n_cus == cu_limit) return 0;
  hipStream_t new_main = stream, new_side = side;
  if (n_cus > 0) {
    new_main = cu_partition_stream(n_cus, 0);
    new_side = cu_partition_stream(n_cus, 1);
    if (!new_main || !new_side) return -5;
  }
  // what the old pair of streams holds comes first
  hipStream_t old_main = main_stream(), old_side = cu_limit > 0 ? masked_side : side;
  if (int rc = depend(old_main, new_main)) return rc;
  if (side_dirty && old_side) {
    if (int rc = depend(old_side, new_main)) return rc;
    side_dirty = false;
    relay_dirty = false;
  }
  cu_limit = n_cus;
  main_since_fork_ = true;   // another pair of streams
  masked_main = n_cus > 0 ? new_main : nullptr;
  masked_side = n_cus > 0 ? new_side : nullptr;
  return 0;
}

int Context::synchronize() {
  if (masked_side && hipStreamSynchronize(masked_side) != hipSuccess) {
    set_error("side stream synchronize failed");
    return -5;
  }
  if (masked_main && hipStreamSynchronize(masked_main) != hipSuccess) {
    set_error("stream synchronize failed");
    return -5;
  }
  if (side && hipStreamSynchronize(side) != hipSuccess) {
    set_error("side stream synchronize failed");
    return -5;
  }
  if (hipStreamSynchronize(stream) != hipSuccess) {
    set_error("stream synchronize failed");
    return -5;
  }
  side_dirty = false;
  relay_dirty = false;
  return 0;
}

int Context::launch_direct(hipStream_t s, const LaunchRecord& rec, hipEvent_t stop) {
  if (!timed_name || !rec.name || strcmp(rec.name, timed_name) != 0) return launch_now(s, rec, stop);
  hipEvent_t begin = nullptr, end = stop;
  if (hipEventCreate(&begin) != hipSuccess || (!end && hipEventCreate(&end) != hipSuccess)) {
    if (begin) (void)hipEventDestroy(begin);
    set_error("timed launch: hipEventCreate failed");
    return -12;
  }
  timed_events.emplace_back(begin, end);
  void* args[1] = {const_cast<unsigned char*>(rec.args)};
  if (hipExtLaunchKernel(rec.fn, rec.grid, rec.block, args, 0, s, begin, end, 0) != hipSuccess) {
    set_error("timed launch: hipExtLaunchKernel failed");
    return -5;
  }
  return 0;
}

int Context::dispatch(const LaunchRecord& rec, const LaunchRecord* next) {
  if (g_reject.load(std::memory_order_acquire)) {
    if (rec.fn) rejected.fetch_add(1);
    fork_event_ = nullptr;
    return 0;
  }
  hipStream_t main = main_stream();
  if (rec.op == kOpJoinBehind) {
    // depend() makes the event calls here, or queues them in order with the launches behind a launch queue
    if (relay_dirty) {
      if (int rc = depend(relay, main)) return rc;
      relay_dirty = false;
    }
    if (side_dirty) {
      if (!relay && hipStreamCreateWithFlags(&relay, hipStreamNonBlocking) != hipSuccess) {
        set_error("hipStreamCreateWithFlags failed");
        return -5;
      }
      if (int rc = depend(cu_limit > 0 ? masked_side : side, relay)) return rc;
      relay_dirty = true;   // side_dirty stays up: lane 0 has not waited for this work yet
    }
    return 0;
  }
  if (queue) {
    // behind the preemptible queue the two lanes stay two streams: what would be event calls here are
    // dependencies queued in order with the launches, and the worker makes them when their turn comes
    if (rec.op == kOpJoin) {
      if (side_dirty) {
        queue->submit_dependency(cu_limit > 0 ? masked_side : side, main);
        side_dirty = false;
      }
      relay_dirty = false;   // what the relay waits for is older than what lane 0 waits for now
      return 0;
    }
    if (!rec.fn) return 0;
    if (rec.lane == 1) {
      if (cu_limit == 0 && !side && hipStreamCreateWithFlags(&side, hipStreamNonBlocking) != hipSuccess) {
        set_error("hipStreamCreateWithFlags failed");
        return -5;
      }
      hipStream_t s = cu_limit > 0 ? masked_side : side;
      if (rec.op == kOpLaunchAfter && main_since_fork_) {
        queue->submit_dependency(main, s);
        main_since_fork_ = false;
      }
      side_dirty = true;
      queue->submit(rec, s);
      return 0;
    }
    main_since_fork_ = true;
    queue->submit(rec, main);
    return 0;
  }
  if (rec.op == kOpJoin) {
    if (side_dirty) {
      hipStream_t s = cu_limit > 0 ? masked_side : side;
      hipEvent_t e = next_event();
      if (!e || hipEventRecord(e, s) != hipSuccess || hipStreamWaitEvent(main, e, 0) != hipSuccess) {
        set_error("join of the side stream failed");
        return -5;
      }
      side_dirty = false;
    }
    relay_dirty = false;
    return 0;
  }
  if (rec.lane == 1) {
    if (cu_limit == 0 && !side && hipStreamCreateWithFlags(&side, hipStreamNonBlocking) != hipSuccess) {
      set_error("hipStreamCreateWithFlags failed");
      return -5;
    }
    hipStream_t s = cu_limit > 0 ? masked_side : side;
    if (rec.op == kOpLaunchAfter && main_since_fork_) {
      main_since_fork_ = false;
      hipEvent_t e = fork_event_;
      fork_event_ = nullptr;
      if (e) {   // the lane-0 kernel before this record signals e when it ends
        if (hipStreamWaitEvent(s, e, 0) != hipSuccess) {
          set_error("fork to the side stream failed");
          return -5;
        }
      } else {
        e = next_event();
        if (!e || hipEventRecord(e, main) != hipSuccess || hipStreamWaitEvent(s, e, 0) != hipSuccess) {
          set_error("fork to the side stream failed");
          return -5;
        }
      }
    }
    side_dirty = true;
    return launch_direct(s, rec, nullptr);
  }
  fork_event_ = nullptr;
  main_since_fork_ = true;
  if (next && next->fn && next->lane == 1 && next->op == kOpLaunchAfter && fork_by_stop_event()) {
    const bool timed = timed_name && rec.name && strcmp(rec.name, timed_name) == 0;
    if (timed) {   // the fork event doubles as the end of the measurement: it must keep its timestamps
      if (hipEventCreate(&fork_event_) != hipSuccess) {
        fork_event_ = nullptr;
        set_error("timed launch: hipEventCreate failed");
        return -12;
      }
    } else {
      fork_event_ = next_event();
    }
    return launch_direct(main, rec, fork_event_);
  }
  return launch_direct(main, rec, nullptr);
}

// ---------------------------------------------------------------------------
// compute-unit partitioning
// ---------------------------------------------------------------------------
namespace {
std::mutex g_cu_mu;
int g_cu_total = 0, g_cu_min = 1, g_cu_max = 0;
std::map<std::pair<int, int>, hipStream_t> g_cu_streams;
}  // namespace

int cu_partition_init(int total_cus, int min_train_cus, int max_train_cus) {
  std::lock_guard<std::mutex> lock(g_cu_mu);
  if (total_cus <= 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      set_error("cu_partition_init: cannot read the compute-unit count of the device");
      return -5;
    }
    total_cus = n;
  }
  g_cu_total = total_cus;
  g_cu_min = min_train_cus < 1 ? 1 : min_train_cus;
  g_cu_max = (max_train_cus <= 0 || max_train_cus > total_cus) ? total_cus : max_train_cus;
  if (g_cu_min > g_cu_max) {
    set_error("cu_partition_init: min_train_cus exceeds max_train_cus");
    return -22;
  }
  return 0;
}

int cu_partition_total() {
  std::lock_guard<std::mutex> lock(g_cu_mu);
  return g_cu_total;
}

int cu_partition_train_avail(int infer_required_cus) {
  std::lock_guard<std::mutex> lock(g_cu_mu);
  if (g_cu_total <= 0) return 0;
  if (infer_required_cus < 0) infer_required_cus = 0;
  int res = g_cu_total - infer_required_cus;
  if (res < g_cu_min) res = g_cu_min;
  if (res > g_cu_max) res = g_cu_max;
  return res;
}

hipStream_t cu_partition_stream(int n_cus, int lane) {
  std::lock_guard<std::mutex> lock(g_cu_mu);
  if (g_cu_total <= 0 || n_cus <= 0 || n_cus > g_cu_total) {
    set_error("cu_partition_stream: partitioning is not initialised or the share is out of range");
    return nullptr;
  }
  auto key = std::make_pair(n_cus, lane);
  auto it = g_cu_streams.find(key);
  if (it != g_cu_streams.end()) return it->second;
  // training keeps the highest-numbered compute units, the other tenant the lowest (sm_partition.cc:92-94)
  const int words = (g_cu_total + 31) / 32;
  std::vector<uint32_t> mask(static_cast<size_t>(words), 0u);
  for (int cu = g_cu_total - n_cus; cu < g_cu_total; ++cu) mask[static_cast<size_t>(cu / 32)] |= 1u << (cu % 32);
  hipStream_t s = nullptr;
  if (hipExtStreamCreateWithCUMask(&s, static_cast<uint32_t>(words), mask.data()) != hipSuccess) {
    set_error("hipExtStreamCreateWithCUMask failed");
    return nullptr;
  }
  g_cu_streams[key] = s;
  return s;
}

int submit(Context* ctx, const void* fn, dim3 grid, dim3 block, const void* args, size_t arg_bytes,
           const char* name, double work, int work_is_bytes, double bytes) {
  if (!ctx) {
    set_error("null context");
    return -22;
  }
  if (grid.x == 0 || grid.y == 0 || grid.z == 0 || block.x == 0 || block.x * block.y * block.z > 1024) {
    set_error("launch with an empty grid or an oversized block");
    return -22;
  }
  LaunchRecord rec;
  rec.fn = fn;
  rec.grid = grid;
  rec.block = block;
  rec.arg_bytes = static_cast<uint32_t>(arg_bytes);
  rec.name = name;
  rec.work = work;
  rec.work_is_bytes = work_is_bytes;
  rec.bytes = work_is_bytes ? work : bytes;
  memcpy(rec.args, args, arg_bytes);
  rec.lane = 0;
  rec.op = kOpLaunch;
  if (ctx->recording && ctx->lane == 1) {
    rec.lane = 1;
    if (ctx->wait_main) {
      rec.op = kOpLaunchAfter;
      ctx->wait_main = false;
    }
  }
  if (ctx->recording) {
    ctx->recording->launches.push_back(rec);
    return 0;
  }
  return ctx->dispatch(rec);
}

// ---------------------------------------------------------------------------
// per-kernel timing of a recorded program
// ---------------------------------------------------------------------------

int profile_program(Context* ctx, const Program& prog, int reps, std::vector<KernelStat>* out,
                    std::vector<LaunchStat>* per_launch) {
  const size_t n = prog.launches.size();
  if (n == 0 || reps < 1) return 0;
  if (per_launch) per_launch->assign(n, LaunchStat());
  std::vector<hipEvent_t> ev(n + 1, nullptr);
  for (auto& e : ev) {
    if (hipEventCreate(&e) != hipSuccess) {
      set_error("profile_program: hipEventCreate failed");
      for (auto x : ev)
        if (x) (void)hipEventDestroy(x);
      return -12;
    }
  }
  std::map<std::string, KernelStat> agg;
  int rc = 0;
  for (int r = 0; r < reps && rc == 0; ++r) {
    // one event between any two launches: launch i runs between ev[i] and ev[i+1]
    (void)hipEventRecord(ev[0], ctx->stream);
    for (size_t i = 0; i < n && rc == 0; ++i) {
      // everything on the one stream, in program order: lanes only matter for a plain replay
      if (prog.launches[i].fn) rc = launch_now(ctx->stream, prog.launches[i]);
      (void)hipEventRecord(ev[i + 1], ctx->stream);
    }
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
      set_error("profile_program: stream synchronize failed");
      rc = -5;
    }
    for (size_t i = 0; i < n && rc == 0; ++i) {
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
      const LaunchRecord& l = prog.launches[i];
      if (!l.fn) continue;
      KernelStat& k = agg[l.name ? l.name : "kernel"];
      k.name = l.name ? l.name : "kernel";
      k.total_ms += ms;
      k.work += l.work;
      k.launches += 1;
      k.work_is_bytes = l.work_is_bytes;
      k.bytes += l.bytes;
      if (per_launch) {
        LaunchStat& p = (*per_launch)[i];
        p.name = k.name;
        p.ms += ms / reps;
        p.flops = l.work_is_bytes ? 0.0 : l.work;
        p.bytes = l.bytes;
        p.lane = l.lane;
        p.grid = static_cast<int64_t>(l.grid.x) * l.grid.y * l.grid.z;
      }
    }
  }
  for (auto e : ev) (void)hipEventDestroy(e);
  if (rc == 0 && out)
    for (auto& kv : agg) out->push_back(kv.second);
  return rc;
}

int time_kernel_in_program(Context* ctx, const Program& prog, const char* name, int reps, double* mean_us,
                           int64_t* launches_per_replay) {
  if (!name || reps < 1 || ctx->recording || ctx->queue) {
    set_error("time_kernel_in_program: needs a kernel name, reps >= 1 and a context that is neither recording nor "
              "behind a launch queue");
    return -22;
  }
  const size_t n = prog.launches.size();
  double sum_ms = 0.0;
  int64_t count = 0;
  int rc = 0;
  for (int r = 0; r < reps && rc == 0; ++r) {
    ctx->timed_name = name;
    ctx->note_foreign_work();
    for (size_t i = 0; i < n && rc == 0; ++i) rc = ctx->dispatch(prog.launches[i], i + 1 < n ? &prog.launches[i + 1] : nullptr);
    ctx->timed_name = nullptr;
    if (ctx->synchronize() != 0 && rc == 0) rc = -5;
    for (auto& be : ctx->timed_events) {
      float ms = 0.f;
      if (rc == 0 && hipEventElapsedTime(&ms, be.first, be.second) == hipSuccess) {
        sum_ms += ms;
        ++count;
      }
      (void)hipEventDestroy(be.first);
      (void)hipEventDestroy(be.second);
    }
    ctx->timed_events.clear();
  }
  if (rc) return rc;
  if (mean_us) *mean_us = count ? sum_ms / static_cast<double>(count) * 1e3 : 0.0;
  if (launches_per_replay) *launches_per_replay = count / reps;
  return 0;
}

// ---------------------------------------------------------------------------
// stream registry
// ---------------------------------------------------------------------------

void set_queue_shape(int queue_length, int sync_interval) {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  g_queue_length = queue_length < 1 ? 1 : queue_length;
  g_sync_interval = sync_interval < 1 ? 1 : sync_interval;
}

uint64_t register_stream(uint64_t stream) {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  if (g_streams.count(stream)) {
    set_error("stream already registered");
    return 0;
  }
  auto q = std::make_shared<LaunchQueue>(reinterpret_cast<hipStream_t>(stream), g_queue_length, g_sync_interval);
  g_streams[stream] = q;
  return reinterpret_cast<uint64_t>(q.get());
}

int unregister_stream(uint64_t stream) {
  std::shared_ptr<LaunchQueue> q;
  {
    std::lock_guard<std::mutex> lock(g_stream_mu);
    auto it = g_streams.find(stream);
    if (it == g_streams.end()) {
      set_error("stream not registered");
      return -2;
    }
    q = it->second;
    g_streams.erase(it);
  }
  q->synchronize();
  return 0;
}

void unregister_all_streams() {
  std::map<uint64_t, std::shared_ptr<LaunchQueue>> taken;
  {
    std::lock_guard<std::mutex> lock(g_stream_mu);
    taken.swap(g_streams);
  }
  for (auto& kv : taken) kv.second->synchronize();
}

std::shared_ptr<LaunchQueue> queue_for_stream(uint64_t stream) {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  auto it = g_streams.find(stream);
  return it == g_streams.end() ? nullptr : it->second;
}

size_t abort_stream(uint64_t stream) {
  auto q = queue_for_stream(stream);
  return q ? q->clear() : 0;
}

size_t abort_all_streams() {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  size_t total = 0;
  for (auto& kv : g_streams) total += kv.second->clear();
  return total;
}

int sync_stream(uint64_t stream) {
  auto q = queue_for_stream(stream);
  if (!q) {
    set_error("stream not registered");
    return -2;
  }
  return q->synchronize();
}

int sync_all_streams() {
  std::vector<std::shared_ptr<LaunchQueue>> qs;
  {
    std::lock_guard<std::mutex> lock(g_stream_mu);
    for (auto& kv : g_streams) qs.push_back(kv.second);
  }
  int rc = 0;
  for (auto& q : qs) {
    int r = q->synchronize();
    if (r) rc = r;
  }
  return rc;
}

size_t queue_size(uint64_t stream) {
  auto q = queue_for_stream(stream);
  return q ? q->size() : 0;
}

size_t queue_size_all_streams() {
  std::lock_guard<std::mutex> lock(g_stream_mu);
  size_t total = 0;
  for (auto& kv : g_streams) total += kv.second->size();
  return total;
}

void suspend_all_streams(bool sync_hw) {
  std::vector<std::shared_ptr<LaunchQueue>> qs;
  {
    std::lock_guard<std::mutex> lock(g_stream_mu);
    for (auto& kv : g_streams) qs.push_back(kv.second);
  }
  for (auto& q : qs) q->suspend(sync_hw);
}

void resume_all_streams(bool drop_commands) {
  std::vector<std::shared_ptr<LaunchQueue>> qs;
  {
    std::lock_guard<std::mutex> lock(g_stream_mu);
    for (auto& kv : g_streams) qs.push_back(kv.second);
  }
  for (auto& q : qs) q->resume(drop_commands);
}

void set_reject_calls(bool reject) { g_reject.store(reject, std::memory_order_release); }
bool query_reject_calls() { return g_reject.load(std::memory_order_acquire); }

}  // namespace tch
