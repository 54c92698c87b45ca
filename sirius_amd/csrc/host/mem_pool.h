// HBM page pool + caching allocator for the colocated training process.
//
// Replaces common/cuda_allocator.{h,cc} (CUDAMemPool: one PagesPool of 32 MB pages shared
// between training and inference through shared memory, every page carrying its owner; a caching
// allocator for torch with a 2 MB small-block threshold, 1024-byte alignment and a virtual range 8x
// the pool: cuda_allocator.cc:61-99, page size cuda_allocator.h:81-87) and the hook half of
// pytorch/torch_col/csrc/torch_allocator_plugin.cc (deferred free behind events :141-178,
// :383-412; recordStream ignoring the block's own stream :200-229; tagging :322-369).
//
// The allocator those files delegate to (third_party/mpool) is absent from the reference
// tree, so placement policy here is this build's own and is specified completely:
//   * physical pages are created once (hipMemCreate, exportable as dma-buf file descriptors) and
//     only ever mapped / unmapped / re-labelled afterwards -- a handover performs no allocation;
//   * the page table (owner and owning pid of every page) lives in a POSIX shared-memory segment
//     "<prefix>_pages_pool_d<device>" behind a robust process-shared mutex: any process of the same
//     user can attach, claim FREE pages, and give them back (PoolPeer below);
//   * the process that created the pool serves the pages' file descriptors over an abstract unix
//     socket of the same name; a peer maps a page it owns by importing that descriptor
//     (hsa_amd_interop_map_buffer: this stack imports HIP virtual-memory handles only inside the
//     process that made them, the dma-buf itself crosses processes);
//   * two growing segments of virtual address space (small: requests < 2 MB, large: the
//     rest); inside a segment: best fit (smallest free block that fits, lowest offset on
//     ties), split when the remainder is at least one alignment unit, coalesce on free,
//     otherwise grow the segment at its end;
//   * a freed block keeps its pages ("train-local free"); empty_cache() hands every page that
//     lies wholly inside free blocks back as FREE.  Eager mode (the default) unmaps those pages
//     first -- one ranged driver call per run of neighbouring slots -- so that a page marked
//     FREE is mapped nowhere in this process.  Lazy mode leaves the mapping in place (stale)
//     and reuses it if the page is still FREE when the range grows again;
//   * physical pages are taken lowest index first, pages without a stale mapping before pages
//     with one.
// Offsets are therefore a pure function of the alloc / free / empty_cache sequence, and the
// CPU model (NullBackend) and the GPU pool (HipVmmBackend) produce the same ones.
//
// The driver's cost of removing a mapping on MI355X is 0.26 ms per mapping whatever its size
// (2 MB ... 1 GB measured), so the page size sets the price of a real handover: 7.6 ms/GB with
// the reference's 32 MB pages, 1.9 ms/GB with 128 MB pages.  The page size is a parameter of the
// pool (32 MB unless asked otherwise).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <atomic>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "shm.h"

namespace tch {
namespace host {

constexpr size_t kDefaultPageBytes = 32ull << 20;  // CUDAMemPool::PageNbytes
constexpr size_t kSmallBlockBytes = 2ull << 20;    // torch allocator small_block_nbytes (PageNbytes / 16)
constexpr size_t kTrainAlign = 1024;               // torch allocator align_nbytes
constexpr int kVaRangeScale = 8;                   // torch allocator va_range_scale
constexpr int kMaxPoolPages = 16384;               // 512 GB of 32 MB pages

enum PageOwner : uint8_t { kOwnerFree = 0, kOwnerTrain = 1, kOwnerInfer = 2 };

// The shared page table.  Every field behind `mu` except the constants written once by the creator.
struct PageTableLayout {
  ShmHeader header;
  pthread_mutex_t mu;
  int num_pages;
  uint64_t page_bytes;
  int creator_pid;
  int has_device;                      // 0 = CPU model: there are no descriptors to serve
  uint64_t changes;                    // bumped by every change of ownership
  uint8_t owner[kMaxPoolPages];
  int32_t owner_pid[kMaxPoolPages];    // pid of the owning process, 0 for FREE
  // 1 while the pool's creator still maps a page it has handed back (lazy mode: the reply to the other tenant goes
  // out first, the mappings are removed right after it).  A peer that has claimed the page waits for 0 before it
  // maps it, so that a page is never usable by two processes at once.  Written with atomic byte stores.
  uint8_t creator_mapped[kMaxPoolPages];
};

std::string page_table_name(int device);   // "<prefix>_pages_pool_d<device>"

class PoolBackend {
 public:
  virtual ~PoolBackend() = default;
  virtual bool reserve(size_t va_bytes, size_t page_bytes, uint64_t* base, std::string* err) = 0;
  virtual bool create_pages(int n, std::string* err) = 0;
  virtual bool map(uint64_t va, int page, std::string* err) = 0;               // no access rights yet
  virtual bool set_access(uint64_t va, size_t bytes, std::string* err) = 0;    // read/write for the device
  virtual bool unmap(uint64_t va, int n_pages, std::string* err) = 0;          // a run of neighbouring slots
  virtual int export_fd(int page, std::string* err) = 0;                       // dma-buf descriptor, or -1
  // Nothing that was submitted so far may still run or wait to run when pages change hands: drains the software
  // launch queues (what waits there is on no stream yet, a device synchronisation alone does not see it), then
  // waits until the device is idle.
  virtual void quiesce() {}
  // event support for frees that must wait for other streams
  virtual uint64_t record_event(uint64_t stream) = 0;
  virtual bool event_done(uint64_t event) = 0;  // also destroys a finished event
  virtual bool has_device() const { return true; }
};

// CPU model: no device, fake base address, events finish when the test says so.
class NullBackend : public PoolBackend {
 public:
  bool reserve(size_t, size_t page_bytes, uint64_t* base, std::string*) override {
    *base = 0x100000000000ull;
    page_ = page_bytes;
    return true;
  }
  bool create_pages(int, std::string*) override { return true; }
  bool map(uint64_t va, int, std::string* err) override {
    if (fail_map_in > 0 && --fail_map_in == 0) {
      if (err) *err = "the CPU model of the pool was told to refuse this mapping";
      return false;
    }
    ++maps;
    no_access.insert(va);
    return true;
  }
  bool set_access(uint64_t va, size_t bytes, std::string*) override {
    ++access_calls;
    for (auto it = no_access.lower_bound(va); it != no_access.end() && *it < va + bytes;) it = no_access.erase(it);
    return true;
  }
  bool unmap(uint64_t va, int n, std::string*) override {
    unmaps += n;
    ++unmap_calls;
    for (auto it = no_access.lower_bound(va); it != no_access.end() && *it < va + static_cast<uint64_t>(n) * page_;)
      it = no_access.erase(it);
    return true;
  }
  void quiesce() override { ++quiesces; }
  int export_fd(int, std::string* err) override {
    if (err) *err = "the CPU model of the pool has no device memory to export";
    return -1;
  }
  uint64_t record_event(uint64_t) override { return ++next_event; }
  bool event_done(uint64_t e) override { return e <= completed_upto; }
  bool has_device() const override { return false; }
  uint64_t next_event = 0, completed_upto = 0;
  int64_t maps = 0, unmaps = 0, unmap_calls = 0, access_calls = 0, quiesces = 0;
  int fail_map_in = 0;            // test knob: the n-th map from now is refused (0: none)
  std::set<uint64_t> no_access;   // mapped addresses that were never given access rights
  uint64_t page_ = 0;
};

PoolBackend* make_hip_vmm_backend(int device);  // mem_pool_hip.cc

struct PoolStats {
  size_t pool_bytes, page_bytes;
  size_t train_usage;       // bytes held by live training blocks
  size_t train_peak_usage;
  size_t train_all_usage;   // pages mapped into the training allocator x page size
  size_t infer_usage;       // pages labelled inference x page size
  size_t free_pages;
  size_t num_allocs, num_frees, num_maps, num_unmaps;
  size_t num_revives;   // slots that got their page back without a driver call
  size_t stale_pages;   // mappings left in place over pages training no longer owns
  size_t num_unmap_calls;  // driver calls behind num_unmaps (a run of slots is one call)
};

struct PoolOptions {
  size_t page_bytes = kDefaultPageBytes;
  bool lazy_unmap = false;   // hand pages back without unmapping them (see the header comment)
};

class HbmPool {
 public:
  // backend ownership passes to the pool
  static HbmPool* create(int device, size_t pool_bytes, PoolBackend* backend, const PoolOptions& opt, std::string* err);
  ~HbmPool();

  void* alloc(size_t nbytes, uint64_t stream, std::string* err);  // nullptr for nbytes == 0 or on failure
  bool free(void* ptr, std::string* err);
  void record_stream(void* ptr, uint64_t stream);
  size_t process_events();  // reap deferred frees; returns how many blocks were released
  size_t empty_cache();     // FreeTrainLocals; returns bytes handed back as FREE pages
  size_t trim(size_t max_pages);  // remove up to max_pages stale mappings; returns how many
  PoolStats stats();
  uint64_t base() const { return base_; }
  size_t page_bytes() const { return page_bytes_; }
  PoolBackend* backend() { return backend_.get(); }
  int64_t offset_of(const void* ptr) const;
  // owner of every physical page and the slot it is mapped at (live or stale, -1: none); returns pages written
  int page_table(uint8_t* owner_out, int64_t* slot_out, int max_pages);

  // the inference side inside this process (a stand-in peer on a thread): label FREE pages as
  // inference-owned / give them back.  Returns the number of pages actually moved.
  int infer_claim_pages(int n);
  int infer_release_pages(int n);

  // tagging (torch_allocator_plugin.cc:322-369): blocks allocated between tag_model_start and
  // tag_model_end are parameters and are never released by release_interm_memory
  void tag_model_start();
  void tag_model_end();
  bool tag_interm_memory(void* ptr);
  size_t release_interm_memory();  // frees every tagged block still alive; returns bytes
  void untag_interm_memory();
  void register_oom_handler(std::function<void()> fn);
  // Called by empty_cache() before it takes any lock, ahead of the backend's own quiesce: where a runtime that
  // queues launches of its own drains them.  The hook may call back into the pool.
  void set_quiesce_hook(std::function<void()> fn);

 private:
  struct Block {
    size_t size;
    bool allocated;
    uint64_t stream;
  };
  struct Segment {
    uint64_t va_begin = 0, va_limit = 0;  // offsets from base_
    uint64_t frontier = 0;                // offset one past the last block
    std::map<uint64_t, Block> blocks;     // by offset, contiguous from va_begin to frontier
    std::set<std::pair<size_t, uint64_t>> free_index;  // (size, offset)
  };
  struct Deferred {
    uint64_t off;
    std::vector<uint64_t> events;
  };
  HbmPool() = default;
  Segment& segment_for(size_t nbytes) { return nbytes < kSmallBlockBytes ? small_ : large_; }
  Segment* segment_of(uint64_t off) { return off < small_.va_limit ? &small_ : &large_; }
  bool alloc_in(Segment& s, size_t n, uint64_t stream, uint64_t* off_out, std::string* err);
  bool ensure_mapped(uint64_t off, size_t n, std::string* err);
  void free_block(Segment& s, uint64_t off);
  size_t empty_cache_locked();         // takes the table lock
  size_t empty_cache_table_locked();   // table already locked
  int take_free_page(std::string* err);
  void set_owner(int page, PageOwner o);
  void set_creator_mapped(int page, bool mapped) {
    __atomic_store_n(&table_->creator_mapped[page], static_cast<uint8_t>(mapped ? 1 : 0), __ATOMIC_RELEASE);
  }
  void serve_descriptors();   // thread: answers peers that ask for the descriptor of a page they own

  int device_ = 0;
  std::unique_ptr<PoolBackend> backend_;
  uint64_t base_ = 0;
  size_t pool_bytes_ = 0, va_bytes_ = 0, page_bytes_ = kDefaultPageBytes;
  bool lazy_unmap_ = false;
  int num_pages_ = 0;
  std::unique_ptr<ShmSegment> table_seg_;
  PageTableLayout* table_ = nullptr;   // owner[] / owner_pid[] of every physical page, shared
  std::vector<int> slot_page_;     // per VA slot: physical page mapped there, or -1
  std::vector<uint8_t> slot_live_; // per VA slot: 1 while training owns the mapped page, 0 = stale mapping
  std::vector<int64_t> page_slot_; // per physical page: the slot it is mapped at (live or stale), or -1
  size_t n_revive_ = 0;
  Segment small_, large_;
  std::mutex mu_;
  size_t train_usage_ = 0, train_peak_ = 0;
  size_t n_alloc_ = 0, n_free_ = 0, n_map_ = 0, n_unmap_ = 0, n_unmap_calls_ = 0;
  bool tagging_model_ = false;
  std::unordered_set<uint64_t> model_params_, interm_;
  std::unordered_map<uint64_t, std::unordered_set<uint64_t>> stream_sets_;
  std::vector<Deferred> deferred_;
  std::vector<std::function<void()>> oom_handlers_;
  std::function<void()> quiesce_hook_;
  int sweep_dead_owners_table_locked();   // pages of processes that no longer exist go back to FREE; returns how many
  int listen_fd_ = -1;
  std::atomic<bool> serving_{false};
  std::unique_ptr<std::thread> server_;
};

// Another process's view of a pool (the inference side): the shared page table, and device
// mappings of the pages it has claimed.  Reference: the TVM-side allocator over the same
// PagesPool, common/cuda_allocator.cc:86-99.
class PoolPeer {
 public:
  static PoolPeer* attach(int device, std::string* err);
  ~PoolPeer();
  int num_pages() const { return table_->num_pages; }
  size_t page_bytes() const { return table_->page_bytes; }
  int free_pages();
  // FREE -> inference-owned by this process, lowest index first; returns how many, indices in pages_out
  int claim(int n, int* pages_out);
  // inference-owned by this process -> FREE (a page still mapped here is unmapped first)
  int release(const int* pages, int n);
  // device address of a claimed page in this process (imports the creator's descriptor on first use); waits, up
  // to wait_ms, until the pool's creator has removed its own mapping of a page it handed back lazily
  void* map(int page, std::string* err, int wait_ms = 5000);
  // how many of `pages` the pool's creator still maps
  int still_mapped_by_creator(const int* pages, int n);
  bool unmap(int page, std::string* err);

 private:
  PoolPeer() = default;
  int fetch_fd(int page, std::string* err);
  int device_ = 0;
  std::unique_ptr<ShmSegment> seg_;
  PageTableLayout* table_ = nullptr;
  int sock_ = -1;
  std::mutex mu_;
  std::unordered_map<int, void*> mapped_;
};

// process-wide pools by device (CUDAMemPool::Get).  A caller holds a counted reference for as long as it
// is inside the pool: pool_shutdown() on another thread cannot destroy it underneath.
std::shared_ptr<HbmPool> pool(int device);
bool pool_init(int device, size_t pool_bytes, bool use_gpu, const PoolOptions& opt, std::string* err);
void pool_shutdown(int device);
uint64_t pool_generation(int device);  // how many pools this device has had

}  // namespace host
}  // namespace tch
