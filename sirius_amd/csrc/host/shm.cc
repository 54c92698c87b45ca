#include "shm.h"

#include <errno.h>
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

#include <chrono>
#include <thread>

namespace tch {
namespace host {

std::string default_shm_prefix() {
  const char* port = getenv("SIRIUS_PORT");
  int p = port ? atoi(port) : 0;
  return "colserve_shm_" + std::to_string(getuid()) + "_p" + std::to_string(p);
}

ShmSegment* ShmSegment::open(const std::string& name, size_t bytes, bool create, bool cleanup, std::string* err) {
  const std::string path = "/" + name;
  if (create && cleanup) shm_unlink(path.c_str());
  int fd = -1;
  bool created = false;
  if (create) {
    fd = shm_open(path.c_str(), O_RDWR | O_CREAT | O_EXCL, 0600);
    if (fd >= 0) {
      created = true;
      if (ftruncate(fd, static_cast<off_t>(bytes)) != 0) {
        if (err) *err = "ftruncate(" + path + "): " + strerror(errno);
        close(fd);
        shm_unlink(path.c_str());
        return nullptr;
      }
    } else if (errno == EEXIST) {
      fd = shm_open(path.c_str(), O_RDWR, 0600);
    }
  } else {
    // the creator may still be starting: retry for a while
    for (int i = 0; i < 2000 && fd < 0; ++i) {
      fd = shm_open(path.c_str(), O_RDWR, 0600);
      if (fd < 0) std::this_thread::sleep_for(std::chrono::milliseconds(5));
    }
  }
  if (fd < 0) {
    if (err) *err = "shm_open(" + path + "): " + strerror(errno);
    return nullptr;
  }
  if (!created) {
    // wait until the creator has sized the segment
    struct stat st;
    for (int i = 0; i < 2000; ++i) {
      if (fstat(fd, &st) == 0 && static_cast<size_t>(st.st_size) >= bytes) break;
      std::this_thread::sleep_for(std::chrono::milliseconds(5));
    }
    if (fstat(fd, &st) != 0 || static_cast<size_t>(st.st_size) < bytes) {
      if (err) *err = "segment " + path + " is smaller than its layout";
      close(fd);
      return nullptr;
    }
  }
  void* base = mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (base == MAP_FAILED) {
    if (err) *err = "mmap(" + path + "): " + strerror(errno);
    if (created) shm_unlink(path.c_str());
    return nullptr;
  }
  auto* seg = new ShmSegment();
  seg->name_ = name;
  seg->base_ = base;
  seg->bytes_ = bytes;
  seg->created_ = created;
  seg->owner_ = create;
  if (created) {
    memset(base, 0, bytes);
    static_cast<ShmHeader*>(base)->layout_bytes = static_cast<uint32_t>(bytes);
  } else {
    auto* h = static_cast<ShmHeader*>(base);
    for (int i = 0; i < 4000 && h->ready.load(std::memory_order_acquire) != kReadyMagic; ++i)
      std::this_thread::sleep_for(std::chrono::milliseconds(5));
    if (h->ready.load(std::memory_order_acquire) != kReadyMagic) {
      if (err) *err = "segment " + path + " was never initialised by its creator";
      delete seg;
      return nullptr;
    }
  }
  return seg;
}

void ShmSegment::mark_ready() { static_cast<ShmHeader*>(base_)->ready.store(kReadyMagic, std::memory_order_release); }

ShmSegment::~ShmSegment() {
  if (base_) munmap(base_, bytes_);
  if (owner_) shm_unlink(("/" + name_).c_str());
}

void init_shared_mutex(pthread_mutex_t* m) {
  pthread_mutexattr_t a;
  pthread_mutexattr_init(&a);
  pthread_mutexattr_setpshared(&a, PTHREAD_PROCESS_SHARED);
  pthread_mutexattr_setrobust(&a, PTHREAD_MUTEX_ROBUST);
  pthread_mutex_init(m, &a);
  pthread_mutexattr_destroy(&a);
}

void init_shared_cond(pthread_cond_t* c) {
  pthread_condattr_t a;
  pthread_condattr_init(&a);
  pthread_condattr_setpshared(&a, PTHREAD_PROCESS_SHARED);
  pthread_condattr_setclock(&a, CLOCK_MONOTONIC);
  pthread_cond_init(c, &a);
  pthread_condattr_destroy(&a);
}

ShmLock::ShmLock(pthread_mutex_t* m) : m_(m) {
  int rc = pthread_mutex_lock(m_);
  if (rc == EOWNERDEAD) pthread_mutex_consistent(m_);  // the previous holder died: state is ours to keep
}

ShmLock::~ShmLock() { pthread_mutex_unlock(m_); }

bool cond_wait_ms(pthread_cond_t* c, pthread_mutex_t* m, int64_t timeout_ms) {
  if (timeout_ms < 0) {
    int rc = pthread_cond_wait(c, m);
    if (rc == EOWNERDEAD) pthread_mutex_consistent(m);
    return true;
  }
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  ts.tv_sec += timeout_ms / 1000;
  ts.tv_nsec += (timeout_ms % 1000) * 1000000;
  if (ts.tv_nsec >= 1000000000) {
    ts.tv_sec += 1;
    ts.tv_nsec -= 1000000000;
  }
  int rc = pthread_cond_timedwait(c, m, &ts);
  if (rc == EOWNERDEAD) pthread_mutex_consistent(m);
  return rc != ETIMEDOUT;
}

int64_t unix_timestamp_ms() {
  return std::chrono::duration_cast<std::chrono::milliseconds>(std::chrono::system_clock::now().time_since_epoch())
      .count();
}

int64_t unix_timestamp_us() {
  return std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::system_clock::now().time_since_epoch())
      .count();
}

}  // namespace host
}  // namespace tch
