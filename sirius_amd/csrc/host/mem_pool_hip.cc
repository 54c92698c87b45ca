// HIP virtual-memory backend of the HBM pool: one reserved address range, physical pages
// created once with hipMemCreate and afterwards only mapped / unmapped, events for frees that
// wait on other streams.  (The reference reaches the same driver facilities through the
// absent mpool submodule; call sites common/cuda_allocator.cc:62-99.)
#include <hip/hip_runtime.h>

#include <unordered_map>
#include <vector>

#include "mem_pool.h"

namespace tch {
namespace host {

namespace {

class HipVmmBackend : public PoolBackend {
 public:
  explicit HipVmmBackend(int device) : device_(device) {}

  ~HipVmmBackend() override {
    (void)hipSetDevice(device_);
    (void)hipDeviceSynchronize();
    for (auto& kv : mapped_) (void)hipMemUnmap(reinterpret_cast<void*>(kv.first), kPageBytes);
    for (auto h : pages_) (void)hipMemRelease(h);
    if (base_) (void)hipMemAddressFree(reinterpret_cast<void*>(base_), va_bytes_);
    for (auto& kv : events_) (void)hipEventDestroy(kv.second);
  }

  bool reserve(size_t va_bytes, uint64_t* base, std::string* err) override {
    if (!check(hipSetDevice(device_), "hipSetDevice", err)) return false;
    hipMemAllocationProp prop = props();
    size_t gran = 0;
    if (!check(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended),
               "hipMemGetAllocationGranularity", err))
      return false;
    if (gran == 0 || kPageBytes % gran != 0) {
      if (err) *err = "32 MB pages are not a multiple of the device's allocation granularity";
      return false;
    }
    void* p = nullptr;
    if (!check(hipMemAddressReserve(&p, va_bytes, kPageBytes, nullptr, 0), "hipMemAddressReserve", err)) return false;
    base_ = reinterpret_cast<uint64_t>(p);
    va_bytes_ = va_bytes;
    *base = base_;
    return true;
  }

  bool create_pages(int n, std::string* err) override {
    hipMemAllocationProp prop = props();
    pages_.reserve(n);
    for (int i = 0; i < n; ++i) {
      hipMemGenericAllocationHandle_t h;
      if (!check(hipMemCreate(&h, kPageBytes, &prop, 0), "hipMemCreate", err)) return false;
      pages_.push_back(h);
    }
    return true;
  }

  bool map(uint64_t va, int page, std::string* err) override {
    void* p = reinterpret_cast<void*>(va);
    if (!check(hipMemMap(p, kPageBytes, 0, pages_[page], 0), "hipMemMap", err)) return false;
    hipMemAccessDesc acc{};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = device_;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    if (!check(hipMemSetAccess(p, kPageBytes, &acc, 1), "hipMemSetAccess", err)) {
      (void)hipMemUnmap(p, kPageBytes);
      return false;
    }
    mapped_[va] = page;
    return true;
  }

  bool unmap(uint64_t va, int, std::string* err) override {
    if (!check(hipMemUnmap(reinterpret_cast<void*>(va), kPageBytes), "hipMemUnmap", err)) return false;
    mapped_.erase(va);
    return true;
  }

  void quiesce() override {
    (void)hipSetDevice(device_);
    (void)hipDeviceSynchronize();
  }

  uint64_t record_event(uint64_t stream) override {
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return 0;
    (void)hipEventRecord(e, reinterpret_cast<hipStream_t>(stream));
    const uint64_t id = ++next_event_;
    events_[id] = e;
    return id;
  }

  bool event_done(uint64_t id) override {
    auto it = events_.find(id);
    if (it == events_.end()) return true;
    hipError_t rc = hipEventQuery(it->second);
    if (rc == hipErrorNotReady) {
      (void)hipGetLastError();
      return false;
    }
    (void)hipEventDestroy(it->second);
    events_.erase(it);
    return true;
  }

 private:
  hipMemAllocationProp props() const {
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = device_;
    return prop;
  }
  static bool check(hipError_t rc, const char* what, std::string* err) {
    if (rc == hipSuccess) return true;
    if (err) *err = std::string(what) + ": " + hipGetErrorString(rc);
    return false;
  }

  int device_;
  uint64_t base_ = 0;
  size_t va_bytes_ = 0;
  std::vector<hipMemGenericAllocationHandle_t> pages_;
  std::unordered_map<uint64_t, int> mapped_;
  std::unordered_map<uint64_t, hipEvent_t> events_;
  uint64_t next_event_ = 0;
};

}  // namespace

PoolBackend* make_hip_vmm_backend(int device) { return new HipVmmBackend(device); }

}  // namespace host
}  // namespace tch
