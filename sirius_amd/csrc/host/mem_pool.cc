#include "mem_pool.h"

#include <algorithm>

#include "shm.h"

namespace tch {
namespace host {

namespace {
std::unique_ptr<HbmPool> g_pools[kMaxDeviceNum];
std::mutex g_pools_mu;
uint64_t g_generation[kMaxDeviceNum] = {};  // bumped per pool_init: tells a stale pointer from a live one

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
}  // namespace

HbmPool* HbmPool::create(int device, size_t pool_bytes, PoolBackend* backend, std::string* err) {
  std::unique_ptr<PoolBackend> be(backend);
  if (pool_bytes < kPageBytes) {
    if (err) *err = "pool must hold at least one 32 MB page";
    return nullptr;
  }
  std::unique_ptr<HbmPool> p(new HbmPool());
  p->device_ = device;
  p->num_pages_ = static_cast<int>(pool_bytes / kPageBytes);
  p->pool_bytes_ = static_cast<size_t>(p->num_pages_) * kPageBytes;
  p->va_bytes_ = p->pool_bytes_ * kVaRangeScale;
  if (!be->reserve(p->va_bytes_, &p->base_, err)) return nullptr;
  if (!be->create_pages(p->num_pages_, err)) return nullptr;
  p->owner_.assign(p->num_pages_, kOwnerFree);
  p->slot_page_.assign(p->va_bytes_ / kPageBytes, -1);
  p->slot_live_.assign(p->va_bytes_ / kPageBytes, 0);
  p->page_slot_.assign(p->num_pages_, -1);
  // one eighth of the range for small blocks, the rest for large ones
  const uint64_t small_bytes = round_up(p->va_bytes_ / 8, kPageBytes);
  p->small_.va_begin = p->small_.frontier = 0;
  p->small_.va_limit = small_bytes;
  p->large_.va_begin = p->large_.frontier = small_bytes;
  p->large_.va_limit = p->va_bytes_;
  p->backend_ = std::move(be);
  return p.release();
}

HbmPool::~HbmPool() = default;

int HbmPool::take_free_page(std::string* err) {
  // lowest index first; a free page that still carries a stale mapping elsewhere is the last
  // resort, and loses that mapping before it is mapped anew (one page, one mapping)
  int stale = -1;
  for (int i = 0; i < num_pages_; ++i) {
    if (owner_[i] != kOwnerFree) continue;
    if (page_slot_[i] < 0) return i;
    if (stale < 0) stale = i;
  }
  if (stale >= 0) {
    const int64_t slot = page_slot_[stale];
    if (!backend_->unmap(base_ + static_cast<uint64_t>(slot) * kPageBytes, stale, err)) return -1;
    ++n_unmap_;
    slot_page_[slot] = -1;
    page_slot_[stale] = -1;
  }
  return stale;
}

bool HbmPool::ensure_mapped(uint64_t off, size_t n, std::string* err) {
  const uint64_t first = off / kPageBytes, last = (off + n - 1) / kPageBytes;
  // a slot whose page was handed back but is still free gets it back without a driver call
  for (uint64_t s = first; s <= last; ++s) {
    const int page = slot_page_[s];
    if (page >= 0 && !slot_live_[s] && owner_[page] == kOwnerFree) {
      owner_[page] = kOwnerTrain;
      slot_live_[s] = 1;
      ++n_revive_;
    }
  }
  // count what is missing before touching anything, so a failure leaves no half-mapped block
  auto count_missing = [&] {
    int m = 0;
    for (uint64_t s = first; s <= last; ++s) m += slot_live_[s] ? 0 : 1;
    return m;
  };
  auto count_free = [&] {
    int f = 0;
    for (int i = 0; i < num_pages_; ++i) f += owner_[i] == kOwnerFree ? 1 : 0;
    return f;
  };
  int missing = count_missing();
  if (missing == 0) return true;
  if (count_free() < missing) {
    // pages cached under free blocks elsewhere may cover the shortfall
    empty_cache_locked();
    missing = count_missing();
    const int free_pages = count_free();
    if (free_pages < missing) {
      if (err) *err = "out of pool memory: need " + std::to_string(missing) + " pages, " + std::to_string(free_pages) + " free";
      return false;
    }
  }
  for (uint64_t s = first; s <= last; ++s) {
    if (slot_live_[s]) continue;
    if (slot_page_[s] >= 0) {
      // the page this slot used to hold now belongs to someone else: drop the stale mapping
      const int old = slot_page_[s];
      if (!backend_->unmap(base_ + s * kPageBytes, old, err)) return false;
      ++n_unmap_;
      page_slot_[old] = -1;
      slot_page_[s] = -1;
    }
    const int page = take_free_page(err);
    if (page < 0) return false;
    if (!backend_->map(base_ + s * kPageBytes, page, err)) return false;
    owner_[page] = kOwnerTrain;
    slot_page_[s] = page;
    page_slot_[page] = static_cast<int64_t>(s);
    slot_live_[s] = 1;
    ++n_map_;
  }
  return true;
}

bool HbmPool::alloc_in(Segment& s, size_t n, uint64_t stream, uint64_t* off_out, std::string* err) {
  auto it = s.free_index.lower_bound({n, 0});
  uint64_t off;
  if (it != s.free_index.end()) {
    off = it->second;
    s.free_index.erase(it);
  } else {
    // grow the segment at its end; a trailing free block is extended rather than left behind
    uint64_t start = s.frontier;
    if (!s.blocks.empty()) {
      auto last = std::prev(s.blocks.end());
      if (!last->second.allocated) {
        start = last->first;
        s.free_index.erase({last->second.size, last->first});
        s.blocks.erase(last);
      }
    }
    const uint64_t new_frontier = round_up(start + n, kPageBytes);
    if (new_frontier > s.va_limit) {
      // put the trailing block back before failing
      if (start < s.frontier) {
        s.blocks[start] = Block{static_cast<size_t>(s.frontier - start), false, 0};
        s.free_index.insert({static_cast<size_t>(s.frontier - start), start});
      }
      if (err) *err = "virtual address range of the training allocator exhausted";
      return false;
    }
    s.frontier = new_frontier;
    s.blocks[start] = Block{static_cast<size_t>(new_frontier - start), false, 0};
    off = start;
  }
  Block& b = s.blocks[off];
  const size_t total = b.size;
  if (total - n >= kTrainAlign) {
    b.size = n;
    s.blocks[off + n] = Block{total - n, false, 0};
    s.free_index.insert({total - n, off + n});
  }
  if (!ensure_mapped(off, s.blocks[off].size, err)) {
    // undo: the block goes back to the free list (coalesced)
    s.blocks[off].allocated = true;
    free_block(s, off);
    return false;
  }
  s.blocks[off].allocated = true;
  s.blocks[off].stream = stream;
  *off_out = off;
  return true;
}

void* HbmPool::alloc(size_t nbytes, uint64_t stream, std::string* err) {
  if (nbytes == 0) return nullptr;  // zero-byte allocations are null (cuda_allocator.cc:129-132)
  std::lock_guard<std::mutex> lock(mu_);
  const size_t n = round_up(nbytes, kTrainAlign);
  uint64_t off = 0;
  if (!alloc_in(segment_for(n), n, stream, &off, err)) {
    for (auto& h : oom_handlers_) h();
    return nullptr;
  }
  train_usage_ += n;
  train_peak_ = std::max(train_peak_, train_usage_);
  ++n_alloc_;
  if (tagging_model_) model_params_.insert(off);
  return reinterpret_cast<void*>(base_ + off);
}

void HbmPool::free_block(Segment& s, uint64_t off) {
  auto it = s.blocks.find(off);
  it->second.allocated = false;
  // coalesce with the next block
  auto next = std::next(it);
  if (next != s.blocks.end() && !next->second.allocated) {
    s.free_index.erase({next->second.size, next->first});
    it->second.size += next->second.size;
    s.blocks.erase(next);
  }
  // and with the previous one
  if (it != s.blocks.begin()) {
    auto prev = std::prev(it);
    if (!prev->second.allocated) {
      s.free_index.erase({prev->second.size, prev->first});
      prev->second.size += it->second.size;
      s.blocks.erase(it);
      it = prev;
    }
  }
  s.free_index.insert({it->second.size, it->first});
}

bool HbmPool::free(void* ptr, std::string* err) {
  if (!ptr) return true;
  std::lock_guard<std::mutex> lock(mu_);
  const uint64_t off = reinterpret_cast<uint64_t>(ptr) - base_;
  Segment* s = segment_of(off);
  auto it = s->blocks.find(off);
  if (it == s->blocks.end() || !it->second.allocated) {
    if (err) *err = "free of a pointer the pool does not own";
    return false;
  }
  auto ss = stream_sets_.find(off);
  if (ss != stream_sets_.end() && !ss->second.empty()) {
    // other streams used the block: hold it until an event on each of them has passed
    Deferred d;
    d.off = off;
    for (uint64_t st : ss->second) d.events.push_back(backend_->record_event(st));
    stream_sets_.erase(ss);
    deferred_.push_back(std::move(d));
    return true;
  }
  stream_sets_.erase(off);
  train_usage_ -= it->second.size;
  ++n_free_;
  model_params_.erase(off);
  interm_.erase(off);
  free_block(*s, off);
  return true;
}

void HbmPool::record_stream(void* ptr, uint64_t stream) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(mu_);
  const uint64_t off = reinterpret_cast<uint64_t>(ptr) - base_;
  Segment* s = segment_of(off);
  auto it = s->blocks.find(off);
  if (it == s->blocks.end() || !it->second.allocated) return;
  if (it->second.stream == stream) return;  // the block's own stream needs no event
  stream_sets_[off].insert(stream);
}

size_t HbmPool::process_events() {
  std::lock_guard<std::mutex> lock(mu_);
  size_t released = 0;
  for (auto it = deferred_.begin(); it != deferred_.end();) {
    auto& ev = it->events;
    ev.erase(std::remove_if(ev.begin(), ev.end(), [&](uint64_t e) { return backend_->event_done(e); }), ev.end());
    if (ev.empty()) {
      Segment* s = segment_of(it->off);
      auto b = s->blocks.find(it->off);
      if (b != s->blocks.end() && b->second.allocated) {
        train_usage_ -= b->second.size;
        ++n_free_;
        model_params_.erase(it->off);
        interm_.erase(it->off);
        free_block(*s, it->off);
        ++released;
      }
      it = deferred_.erase(it);
    } else {
      ++it;
    }
  }
  return released;
}

size_t HbmPool::empty_cache_locked() {
  // Handing a page back is bookkeeping only: the page is relabelled FREE and its mapping into
  // the training range is left in place ("stale").  Tearing a mapping down costs the driver
  // about 0.24 ms per 32 MB page on MI355X -- 47 ms for the 6.5 GB a batch-64 ResNet-152 step
  // gives up -- so it is kept off the handover path: the mapping is reused for free if the
  // page is still FREE when the range grows again, and is only removed when the slot needs a
  // different page, when the page is needed elsewhere, or by trim().
  size_t bytes = 0;
  bool quiesced = false;
  for (Segment* s : {&small_, &large_}) {
    for (auto& kv : s->blocks) {
      if (kv.second.allocated) continue;
      const uint64_t lo = round_up(kv.first, kPageBytes);
      const uint64_t hi = (kv.first + kv.second.size) / kPageBytes * kPageBytes;
      for (uint64_t a = lo; a + kPageBytes <= hi; a += kPageBytes) {
        const uint64_t slot = a / kPageBytes;
        const int page = slot_page_[slot];
        if (page < 0 || !slot_live_[slot]) continue;
        if (!quiesced) {
          // a freed block may still be read by launches in flight on its own stream (frees are
          // stream ordered): nothing may be running when its pages change hands
          backend_->quiesce();
          quiesced = true;
        }
        slot_live_[slot] = 0;
        owner_[page] = kOwnerFree;
        bytes += kPageBytes;
      }
    }
  }
  return bytes;
}

size_t HbmPool::trim(size_t max_pages) {
  std::lock_guard<std::mutex> lock(mu_);
  size_t n = 0;
  for (size_t slot = 0; slot < slot_page_.size() && n < max_pages; ++slot) {
    const int page = slot_page_[slot];
    if (page < 0 || slot_live_[slot]) continue;
    std::string err;
    if (!backend_->unmap(base_ + slot * kPageBytes, page, &err)) continue;
    ++n_unmap_;
    slot_page_[slot] = -1;
    page_slot_[page] = -1;
    ++n;
  }
  return n;
}

size_t HbmPool::empty_cache() {
  process_events();
  std::lock_guard<std::mutex> lock(mu_);
  return empty_cache_locked();
}

PoolStats HbmPool::stats() {
  std::lock_guard<std::mutex> lock(mu_);
  PoolStats st{};
  st.pool_bytes = pool_bytes_;
  st.page_bytes = kPageBytes;
  st.train_usage = train_usage_;
  st.train_peak_usage = train_peak_;
  size_t train_pages = 0, infer_pages = 0, free_pages = 0;
  for (uint8_t o : owner_) {
    train_pages += o == kOwnerTrain;
    infer_pages += o == kOwnerInfer;
    free_pages += o == kOwnerFree;
  }
  st.train_all_usage = train_pages * kPageBytes;
  st.infer_usage = infer_pages * kPageBytes;
  st.free_pages = free_pages;
  st.num_allocs = n_alloc_;
  st.num_frees = n_free_;
  st.num_maps = n_map_;
  st.num_unmaps = n_unmap_;
  st.num_revives = n_revive_;
  for (size_t s = 0; s < slot_page_.size(); ++s) st.stale_pages += slot_page_[s] >= 0 && !slot_live_[s] ? 1 : 0;
  return st;
}

int64_t HbmPool::offset_of(const void* ptr) const {
  const uint64_t a = reinterpret_cast<uint64_t>(ptr);
  if (a < base_ || a >= base_ + va_bytes_) return -1;
  return static_cast<int64_t>(a - base_);
}

int HbmPool::infer_claim_pages(int n) {
  std::lock_guard<std::mutex> lock(mu_);
  int moved = 0;
  for (int i = 0; i < num_pages_ && moved < n; ++i)
    if (owner_[i] == kOwnerFree) {
      owner_[i] = kOwnerInfer;
      ++moved;
    }
  return moved;
}

int HbmPool::infer_release_pages(int n) {
  std::lock_guard<std::mutex> lock(mu_);
  int moved = 0;
  for (int i = num_pages_ - 1; i >= 0 && moved < n; --i)
    if (owner_[i] == kOwnerInfer) {
      owner_[i] = kOwnerFree;
      ++moved;
    }
  return moved;
}

void HbmPool::tag_model_start() {
  std::lock_guard<std::mutex> lock(mu_);
  tagging_model_ = true;
}
void HbmPool::tag_model_end() {
  std::lock_guard<std::mutex> lock(mu_);
  tagging_model_ = false;
}

bool HbmPool::tag_interm_memory(void* ptr) {
  std::lock_guard<std::mutex> lock(mu_);
  const int64_t off = offset_of(ptr);
  if (off < 0) return false;
  Segment* s = segment_of(off);
  auto it = s->blocks.find(off);
  if (it == s->blocks.end() || !it->second.allocated) return false;
  if (model_params_.count(off)) return false;  // parameters are never intermediate memory
  interm_.insert(off);
  return true;
}

size_t HbmPool::release_interm_memory() {
  std::lock_guard<std::mutex> lock(mu_);
  size_t bytes = 0;
  for (uint64_t off : interm_) {
    Segment* s = segment_of(off);
    auto it = s->blocks.find(off);
    if (it == s->blocks.end() || !it->second.allocated) continue;
    bytes += it->second.size;
    train_usage_ -= it->second.size;
    ++n_free_;
    stream_sets_.erase(off);
    free_block(*s, off);
  }
  interm_.clear();
  return bytes;
}

void HbmPool::untag_interm_memory() {
  std::lock_guard<std::mutex> lock(mu_);
  interm_.clear();
}

void HbmPool::register_oom_handler(std::function<void()> fn) {
  std::lock_guard<std::mutex> lock(mu_);
  oom_handlers_.push_back(std::move(fn));
}

HbmPool* pool(int device) {
  if (device < 0 || device >= kMaxDeviceNum) return nullptr;
  return g_pools[device].get();
}

bool pool_init(int device, size_t pool_bytes, bool use_gpu, std::string* err) {
  std::lock_guard<std::mutex> lock(g_pools_mu);
  if (device < 0 || device >= kMaxDeviceNum) {
    if (err) *err = "device id exceeds the supported device count";
    return false;
  }
  if (g_pools[device]) {
    if (err) *err = "pool already initialised for this device";
    return false;
  }
  PoolBackend* be = use_gpu ? make_hip_vmm_backend(device) : new NullBackend();
  g_pools[device].reset(HbmPool::create(device, pool_bytes, be, err));
  if (g_pools[device]) ++g_generation[device];
  return g_pools[device] != nullptr;
}

uint64_t pool_generation(int device) {
  std::lock_guard<std::mutex> lock(g_pools_mu);
  return device >= 0 && device < kMaxDeviceNum ? g_generation[device] : 0;
}

void pool_shutdown(int device) {
  std::lock_guard<std::mutex> lock(g_pools_mu);
  if (device >= 0 && device < kMaxDeviceNum) g_pools[device].reset();
}

}  // namespace host
}  // namespace tch
