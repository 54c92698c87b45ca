// HIP virtual-memory backend of the HBM pool: one reserved address range, physical pages
// created once with hipMemCreate and afterwards only mapped / unmapped, events for frees that
// wait on other streams.  (The reference reaches the same driver facilities through the
// absent mpool submodule; call sites common/cuda_allocator.cc:62-99.)
#include <hip/hip_runtime.h>
#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include <mutex>
#include <unordered_map>
#include <vector>

#include "mem_pool.h"

namespace tch {
int sync_all_streams();   // context.cc: every registered launch queue drained and finished on the device
}

namespace tch {
namespace host {

namespace {

class HipVmmBackend : public PoolBackend {
 public:
  explicit HipVmmBackend(int device) : device_(device) {}

  ~HipVmmBackend() override {
    (void)hipSetDevice(device_);
    (void)hipDeviceSynchronize();
    for (auto& kv : mapped_) (void)hipMemUnmap(reinterpret_cast<void*>(kv.first), page_bytes_);
    for (auto h : pages_) (void)hipMemRelease(h);
    if (base_) (void)hipMemAddressFree(reinterpret_cast<void*>(base_), va_bytes_);
    for (auto& kv : events_) (void)hipEventDestroy(kv.second);
  }

  bool reserve(size_t va_bytes, size_t page_bytes, uint64_t* base, std::string* err) override {
    page_bytes_ = page_bytes;
    if (!check(hipSetDevice(device_), "hipSetDevice", err)) return false;
    hipMemAllocationProp prop = props();
    size_t gran = 0;
    if (!check(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended),
               "hipMemGetAllocationGranularity", err))
      return false;
    if (gran == 0 || page_bytes_ % gran != 0) {
      if (err) *err = "the page size is not a multiple of the device's allocation granularity";
      return false;
    }
    void* p = nullptr;
    if (!check(hipMemAddressReserve(&p, va_bytes, page_bytes_, nullptr, 0), "hipMemAddressReserve", err)) return false;
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
      if (!check(hipMemCreate(&h, page_bytes_, &prop, 0), "hipMemCreate", err)) return false;
      pages_.push_back(h);
    }
    return true;
  }

  bool map(uint64_t va, int page, std::string* err) override {
    if (!check(hipMemMap(reinterpret_cast<void*>(va), page_bytes_, 0, pages_[page], 0), "hipMemMap", err)) return false;
    mapped_[va] = page;
    return true;
  }

  bool set_access(uint64_t va, size_t bytes, std::string* err) override {
    hipMemAccessDesc acc{};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = device_;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    return check(hipMemSetAccess(reinterpret_cast<void*>(va), bytes, &acc, 1), "hipMemSetAccess", err);
  }

  bool unmap(uint64_t va, int n_pages, std::string* err) override {
    // one call over a run of separately mapped neighbours: the driver walks the mappings itself
    if (!check(hipMemUnmap(reinterpret_cast<void*>(va), static_cast<size_t>(n_pages) * page_bytes_), "hipMemUnmap", err))
      return false;
    for (int i = 0; i < n_pages; ++i) mapped_.erase(va + static_cast<uint64_t>(i) * page_bytes_);
    return true;
  }

  int export_fd(int page, std::string* err) override {
    int fd = -1;
    if (!check(hipMemExportToShareableHandle(&fd, pages_[page], hipMemHandleTypePosixFileDescriptor, 0),
               "hipMemExportToShareableHandle", err))
      return -1;
    return fd;
  }

  void quiesce() override {
    // what still waits in a preemptible launch queue is on no stream yet: hand it over and wait for it first
    (void)tch::sync_all_streams();
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
    prop.requestedHandleType = hipMemHandleTypePosixFileDescriptor;   // pages can leave the process as dma-bufs
    return prop;
  }
  static bool check(hipError_t rc, const char* what, std::string* err) {
    if (rc == hipSuccess) return true;
    if (err) *err = std::string(what) + ": " + hipGetErrorString(rc);
    return false;
  }

  int device_;
  uint64_t base_ = 0;
  size_t va_bytes_ = 0, page_bytes_ = kDefaultPageBytes;
  std::vector<hipMemGenericAllocationHandle_t> pages_;
  std::unordered_map<uint64_t, int> mapped_;
  std::unordered_map<uint64_t, hipEvent_t> events_;
  uint64_t next_event_ = 0;
};

}  // namespace

PoolBackend* make_hip_vmm_backend(int device) { return new HipVmmBackend(device); }

// ---- the peer's side: a page that another process created, mapped here from its dma-buf descriptor ----
// hipMemImportFromShareableHandle accepts a descriptor only inside the process that exported it on this
// stack (measured: "invalid argument" in any other process), so the import goes one level down, through
// the runtime's interop call, which maps the dma-buf for the device and returns the address it chose.
namespace {
std::mutex g_hsa_mu;
bool g_hsa_ready = false;
std::vector<hsa_agent_t> g_gpu_agents;

hsa_status_t collect_gpu(hsa_agent_t a, void*) {
  hsa_device_type_t t;
  if (hsa_agent_get_info(a, HSA_AGENT_INFO_DEVICE, &t) == HSA_STATUS_SUCCESS && t == HSA_DEVICE_TYPE_GPU)
    g_gpu_agents.push_back(a);
  return HSA_STATUS_SUCCESS;
}

std::string hsa_error(const char* what, hsa_status_t st) {
  const char* s = nullptr;
  hsa_status_string(st, &s);
  return std::string(what) + ": " + (s ? s : "unknown HSA status");
}
}  // namespace

bool peer_map_descriptor(int device, int fd, size_t expect_bytes, void** ptr, std::string* err) {
  std::lock_guard<std::mutex> lock(g_hsa_mu);
  if (hipSetDevice(device) != hipSuccess) {   // also brings the runtime up in this process
    if (err) *err = "hipSetDevice failed";
    return false;
  }
  if (!g_hsa_ready) {
    hsa_status_t st = hsa_init();
    if (st != HSA_STATUS_SUCCESS) {
      if (err) *err = hsa_error("hsa_init", st);
      return false;
    }
    hsa_iterate_agents(collect_gpu, nullptr);
    g_hsa_ready = true;
  }
  if (device < 0 || device >= static_cast<int>(g_gpu_agents.size())) {
    if (err) *err = "no GPU agent for device " + std::to_string(device);
    return false;
  }
  size_t size = 0, meta_size = 0;
  const void* meta = nullptr;
  void* p = nullptr;
  hsa_status_t st = hsa_amd_interop_map_buffer(1, &g_gpu_agents[device], fd, 0, &size, &p, &meta_size, &meta);
  if (st != HSA_STATUS_SUCCESS) {
    if (err) *err = hsa_error("hsa_amd_interop_map_buffer", st);
    return false;
  }
  if (size < expect_bytes) {
    hsa_amd_interop_unmap_buffer(p);
    if (err) *err = "the imported page is smaller than the pool's page size";
    return false;
  }
  *ptr = p;
  return true;
}

bool peer_unmap(void* ptr, std::string* err) {
  std::lock_guard<std::mutex> lock(g_hsa_mu);
  hsa_status_t st = hsa_amd_interop_unmap_buffer(ptr);
  if (st != HSA_STATUS_SUCCESS) {
    if (err) *err = hsa_error("hsa_amd_interop_unmap_buffer", st);
    return false;
  }
  return true;
}

}  // namespace host
}  // namespace tch
