// HBM page pool + caching allocator for the colocated training process.
//
// Replaces common/cuda_allocator.{h,cc} (CUDAMemPool: one PagesPool of 32 MB pages shared
// between training and inference, a caching allocator for torch with a 2 MB small-block
// threshold, 1024-byte alignment and a virtual range 8x the pool: cuda_allocator.cc:61-85,
// page size cuda_allocator.h:81-87) and the hook half of
// pytorch/torch_col/csrc/torch_allocator_plugin.cc (deferred free behind events :141-178,
// :383-412; recordStream ignoring the block's own stream :200-229; tagging :322-369).
//
// The allocator those files delegate to (third_party/mpool) is absent from the reference
// tree, so placement policy here is this build's own and is specified completely:
//   * physical pages are created once (hipMemCreate) and only ever mapped / unmapped /
//     re-labelled afterwards -- a handover performs no allocation;
//   * two growing segments of virtual address space (small: requests < 2 MB, large: the
//     rest); inside a segment: best fit (smallest free block that fits, lowest offset on
//     ties), split when the remainder is at least one alignment unit, coalesce on free,
//     otherwise grow the segment at its end;
//   * a freed block keeps its pages ("train-local free"); empty_cache() hands every page that
//     lies wholly inside free blocks back as FREE.  That is bookkeeping: the mapping stays in
//     place (stale) and is reused if the page is still FREE when the range grows again;
//   * physical pages are taken lowest index first, pages without a stale mapping before pages
//     with one.
// Offsets are therefore a pure function of the alloc / free / empty_cache sequence, and the
// CPU model (NullBackend) and the GPU pool (HipVmmBackend) produce the same ones.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace tch {
namespace host {

constexpr size_t kPageBytes = 32ull << 20;        // CUDAMemPool::PageNbytes
constexpr size_t kSmallBlockBytes = kPageBytes / 16;  // 2 MB: torch allocator small_block_nbytes
constexpr size_t kTrainAlign = 1024;              // torch allocator align_nbytes
constexpr int kVaRangeScale = 8;                  // torch allocator va_range_scale

enum PageOwner : uint8_t { kOwnerFree = 0, kOwnerTrain = 1, kOwnerInfer = 2 };

class PoolBackend {
 public:
  virtual ~PoolBackend() = default;
  virtual bool reserve(size_t va_bytes, uint64_t* base, std::string* err) = 0;
  virtual bool create_pages(int n, std::string* err) = 0;
  virtual bool map(uint64_t va, int page, std::string* err) = 0;
  virtual bool unmap(uint64_t va, int page, std::string* err) = 0;
  virtual void quiesce() {}  // wait until the device is idle (called once before a round of unmaps)
  // event support for frees that must wait for other streams
  virtual uint64_t record_event(uint64_t stream) = 0;
  virtual bool event_done(uint64_t event) = 0;  // also destroys a finished event
};

// CPU model: no device, fake base address, events finish when the test says so.
class NullBackend : public PoolBackend {
 public:
  bool reserve(size_t, uint64_t* base, std::string*) override {
    *base = 0x100000000000ull;
    return true;
  }
  bool create_pages(int, std::string*) override { return true; }
  bool map(uint64_t, int, std::string*) override { ++maps; return true; }
  bool unmap(uint64_t, int, std::string*) override { ++unmaps; return true; }
  uint64_t record_event(uint64_t) override { return ++next_event; }
  bool event_done(uint64_t e) override { return e <= completed_upto; }
  uint64_t next_event = 0, completed_upto = 0;
  int64_t maps = 0, unmaps = 0;
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
};

class HbmPool {
 public:
  // backend ownership passes to the pool
  static HbmPool* create(int device, size_t pool_bytes, PoolBackend* backend, std::string* err);
  ~HbmPool();

  void* alloc(size_t nbytes, uint64_t stream, std::string* err);  // nullptr for nbytes == 0 or on failure
  bool free(void* ptr, std::string* err);
  void record_stream(void* ptr, uint64_t stream);
  size_t process_events();  // reap deferred frees; returns how many blocks were released
  size_t empty_cache();     // FreeTrainLocals; returns bytes handed back as FREE pages
  size_t trim(size_t max_pages);  // remove up to max_pages stale mappings; returns how many
  PoolStats stats();
  uint64_t base() const { return base_; }
  PoolBackend* backend() { return backend_.get(); }
  int64_t offset_of(const void* ptr) const;

  // the inference side of the pool, as far as a fake peer needs it: label FREE pages as
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
  size_t empty_cache_locked();
  int take_free_page(std::string* err);

  int device_ = 0;
  std::unique_ptr<PoolBackend> backend_;
  uint64_t base_ = 0;
  size_t pool_bytes_ = 0, va_bytes_ = 0;
  int num_pages_ = 0;
  std::vector<uint8_t> owner_;     // per physical page
  std::vector<int> slot_page_;     // per VA slot: physical page mapped there, or -1
  std::vector<uint8_t> slot_live_; // per VA slot: 1 while training owns the mapped page, 0 = stale mapping
  std::vector<int64_t> page_slot_; // per physical page: the slot it is mapped at (live or stale), or -1
  size_t n_revive_ = 0;
  Segment small_, large_;
  std::mutex mu_;
  size_t train_usage_ = 0, train_peak_ = 0;
  size_t n_alloc_ = 0, n_free_ = 0, n_map_ = 0, n_unmap_ = 0;
  bool tagging_model_ = false;
  std::unordered_set<uint64_t> model_params_, interm_;
  std::unordered_map<uint64_t, std::unordered_set<uint64_t>> stream_sets_;
  std::vector<Deferred> deferred_;
  std::vector<std::function<void()>> oom_handlers_;
};

// process-wide pools by device (CUDAMemPool::Get)
HbmPool* pool(int device);
bool pool_init(int device, size_t pool_bytes, bool use_gpu, std::string* err);
void pool_shutdown(int device);
uint64_t pool_generation(int device);  // how many pools this device has had

}  // namespace host
}  // namespace tch
