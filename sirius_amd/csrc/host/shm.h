// POSIX shared-memory plumbing for the host runtime: named segments with a fixed POD
// layout, process-shared (robust) mutexes and monotonic-clock condition variables.
//
// The reference keeps the same state in boost.interprocess managed segments
// (common/inf_tra_comm/communicator.cc:38-62, pytorch/torch_col/csrc/dist_train_sync.cc:69-145);
// this build has no boost, so every segment is one struct that both sides map.
#pragma once

#include <pthread.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>
#include <string>

namespace tch {
namespace host {

constexpr int kMaxDeviceNum = 8;  // common/util.h MAX_DEVICE_NUM

// "colserve_shm_<uid>_p<port>" with port from SIRIUS_PORT (0 if unset): common/util.h:120-132
std::string default_shm_prefix();

struct ShmHeader {
  std::atomic<uint32_t> ready;  // set to kReadyMagic by the creator once the body is initialised
  uint32_t layout_bytes;        // sizeof of the struct the creator mapped
};
constexpr uint32_t kReadyMagic = 0x54434852u;

class ShmSegment {
 public:
  // create: make (or reuse) the segment and become its owner; cleanup: unlink a stale
  // segment of that name first.  Non-owners open an existing segment and wait for `ready`.
  // Returns nullptr and fills *err on failure.
  static ShmSegment* open(const std::string& name, size_t bytes, bool create, bool cleanup, std::string* err);
  ~ShmSegment();
  void* base() const { return base_; }
  bool created() const { return created_; }  // this process initialises the body
  bool owner() const { return owner_; }
  void mark_ready();
  const std::string& name() const { return name_; }

 private:
  ShmSegment() = default;
  std::string name_;
  void* base_ = nullptr;
  size_t bytes_ = 0;
  bool created_ = false;
  bool owner_ = false;
};

void init_shared_mutex(pthread_mutex_t* m);
void init_shared_cond(pthread_cond_t* c);

// lock that survives the death of a holder in another process
class ShmLock {
 public:
  explicit ShmLock(pthread_mutex_t* m);
  ~ShmLock();
  ShmLock(const ShmLock&) = delete;
  ShmLock& operator=(const ShmLock&) = delete;
  pthread_mutex_t* native() { return m_; }

 private:
  pthread_mutex_t* m_;
};

// wait on a monotonic-clock condition variable; timeout_ms < 0 waits forever.
// Returns false on timeout.
bool cond_wait_ms(pthread_cond_t* c, pthread_mutex_t* m, int64_t timeout_ms);

int64_t unix_timestamp_ms();
int64_t unix_timestamp_us();

}  // namespace host
}  // namespace tch
