#include "mem_pool.h"

#include <errno.h>
#include <poll.h>
#include <signal.h>
#include <string.h>
#include <sys/socket.h>
#include <sys/un.h>
#include <unistd.h>

#include <algorithm>

namespace tch {
namespace host {

namespace {
std::shared_ptr<HbmPool> g_pools[kMaxDeviceNum];
std::mutex g_pools_mu;
uint64_t g_generation[kMaxDeviceNum] = {};  // bumped per pool_init: tells a stale pointer from a live one

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// abstract unix socket "\0<name>": no file to clean up, gone with the last descriptor
socklen_t abstract_addr(const std::string& name, sockaddr_un* a) {
  memset(a, 0, sizeof(*a));
  a->sun_family = AF_UNIX;
  const size_t n = std::min(name.size(), sizeof(a->sun_path) - 2);
  memcpy(a->sun_path + 1, name.data(), n);
  return static_cast<socklen_t>(offsetof(sockaddr_un, sun_path) + 1 + n);
}

// one request of a peer: the descriptor of `page`; the answer is one status word, with the descriptor
// attached (SCM_RIGHTS) when the status is 0
struct FdRequest {
  int32_t page;
};

bool send_status_fd(int sock, int32_t status, int fd) {
  msghdr m{};
  iovec io{&status, sizeof(status)};
  m.msg_iov = &io;
  m.msg_iovlen = 1;
  alignas(cmsghdr) char ctl[CMSG_SPACE(sizeof(int))];
  if (fd >= 0) {
    m.msg_control = ctl;
    m.msg_controllen = sizeof(ctl);
    cmsghdr* h = CMSG_FIRSTHDR(&m);
    h->cmsg_level = SOL_SOCKET;
    h->cmsg_type = SCM_RIGHTS;
    h->cmsg_len = CMSG_LEN(sizeof(int));
    memcpy(CMSG_DATA(h), &fd, sizeof(int));
  }
  return sendmsg(sock, &m, MSG_NOSIGNAL) == static_cast<ssize_t>(sizeof(status));
}

bool recv_status_fd(int sock, int32_t* status, int* fd) {
  msghdr m{};
  iovec io{status, sizeof(*status)};
  m.msg_iov = &io;
  m.msg_iovlen = 1;
  alignas(cmsghdr) char ctl[CMSG_SPACE(sizeof(int))];
  m.msg_control = ctl;
  m.msg_controllen = sizeof(ctl);
  *fd = -1;
  if (recvmsg(sock, &m, 0) != static_cast<ssize_t>(sizeof(*status))) return false;
  for (cmsghdr* h = CMSG_FIRSTHDR(&m); h; h = CMSG_NXTHDR(&m, h))
    if (h->cmsg_level == SOL_SOCKET && h->cmsg_type == SCM_RIGHTS) memcpy(fd, CMSG_DATA(h), sizeof(int));
  return true;
}
}  // namespace

std::string page_table_name(int device) { return default_shm_prefix() + "_pages_pool_d" + std::to_string(device); }

HbmPool* HbmPool::create(int device, size_t pool_bytes, PoolBackend* backend, const PoolOptions& opt, std::string* err) {
  std::unique_ptr<PoolBackend> be(backend);
  const size_t page = opt.page_bytes;
  if (page < kSmallBlockBytes || page % kSmallBlockBytes != 0) {
    if (err) *err = "the page size must be a multiple of 2 MB";
    return nullptr;
  }
  if (pool_bytes < page) {
    if (err) *err = "pool must hold at least one page";
    return nullptr;
  }
  if (pool_bytes / page > static_cast<size_t>(kMaxPoolPages)) {
    if (err) *err = "pool has more pages than the shared page table holds (" + std::to_string(kMaxPoolPages) + ")";
    return nullptr;
  }
  std::unique_ptr<HbmPool> p(new HbmPool());
  p->device_ = device;
  p->page_bytes_ = page;
  p->lazy_unmap_ = opt.lazy_unmap;
  p->num_pages_ = static_cast<int>(pool_bytes / page);
  p->pool_bytes_ = static_cast<size_t>(p->num_pages_) * page;
  p->va_bytes_ = p->pool_bytes_ * kVaRangeScale;
  // The descriptor server's address first: it is taken while the process that made a pool of this name is
  // alive, so a live pool is never taken over; a table left behind by a dead one is replaced.
  sockaddr_un addr;
  const socklen_t len = abstract_addr(page_table_name(device), &addr);
  p->listen_fd_ = socket(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0);
  if (p->listen_fd_ < 0 || bind(p->listen_fd_, reinterpret_cast<sockaddr*>(&addr), len) != 0 ||
      listen(p->listen_fd_, 16) != 0) {
    if (err) *err = "a pool named " + page_table_name(device) + " is served by another process (" + strerror(errno) + ")";
    return nullptr;
  }
  p->table_seg_.reset(ShmSegment::open(page_table_name(device), sizeof(PageTableLayout), true, true, err));
  if (!p->table_seg_) return nullptr;
  if (!p->table_seg_->created()) {
    if (err) *err = "a page table named " + page_table_name(device) + " already exists";
    return nullptr;
  }
  p->table_ = static_cast<PageTableLayout*>(p->table_seg_->base());
  init_shared_mutex(&p->table_->mu);
  p->table_->num_pages = p->num_pages_;
  p->table_->page_bytes = page;
  p->table_->creator_pid = static_cast<int>(getpid());
  p->table_->has_device = be->has_device() ? 1 : 0;
  if (!be->reserve(p->va_bytes_, page, &p->base_, err)) return nullptr;
  if (!be->create_pages(p->num_pages_, err)) return nullptr;
  p->slot_page_.assign(p->va_bytes_ / page, -1);
  p->slot_live_.assign(p->va_bytes_ / page, 0);
  p->page_slot_.assign(p->num_pages_, -1);
  // one eighth of the range for small blocks, the rest for large ones
  const uint64_t small_bytes = round_up(p->va_bytes_ / 8, page);
  p->small_.va_begin = p->small_.frontier = 0;
  p->small_.va_limit = small_bytes;
  p->large_.va_begin = p->large_.frontier = small_bytes;
  p->large_.va_limit = p->va_bytes_;
  p->backend_ = std::move(be);
  p->serving_.store(true);
  HbmPool* raw = p.get();
  p->server_.reset(new std::thread([raw] { raw->serve_descriptors(); }));
  p->table_seg_->mark_ready();
  return p.release();
}

HbmPool::~HbmPool() {
  serving_.store(false);
  if (server_) server_->join();
  if (listen_fd_ >= 0) close(listen_fd_);
}

void HbmPool::set_owner(int page, PageOwner o) {
  table_->owner[page] = o;
  table_->owner_pid[page] = o == kOwnerFree ? 0 : static_cast<int32_t>(getpid());
  table_->changes++;
}

void HbmPool::serve_descriptors() {
  std::vector<pollfd> fds;
  fds.push_back({listen_fd_, POLLIN, 0});
  while (serving_.load()) {
    const int n = poll(fds.data(), fds.size(), 50);
    if (n <= 0) continue;
    if (fds[0].revents & POLLIN) {
      const int c = accept4(listen_fd_, nullptr, nullptr, SOCK_CLOEXEC);
      if (c >= 0) fds.push_back({c, POLLIN, 0});
    }
    for (size_t i = 1; i < fds.size();) {
      if (!(fds[i].revents & (POLLIN | POLLHUP | POLLERR))) {
        ++i;
        continue;
      }
      FdRequest rq{};
      const ssize_t got = recv(fds[i].fd, &rq, sizeof(rq), MSG_DONTWAIT);
      if (got != static_cast<ssize_t>(sizeof(rq))) {   // closed or broken: drop the peer
        close(fds[i].fd);
        fds.erase(fds.begin() + i);
        continue;
      }
      // the descriptor of a page goes only to the process the table names as its owner
      ucred cred{};
      socklen_t cl = sizeof(cred);
      getsockopt(fds[i].fd, SOL_SOCKET, SO_PEERCRED, &cred, &cl);
      int32_t status = -1;
      int fd = -1;
      if (rq.page >= 0 && rq.page < num_pages_) {
        bool owned;
        {
          ShmLock t(&table_->mu);
          owned = table_->owner[rq.page] == kOwnerInfer && table_->owner_pid[rq.page] == static_cast<int32_t>(cred.pid);
        }
        if (owned) {
          std::string err;
          fd = backend_->export_fd(rq.page, &err);
          status = fd >= 0 ? 0 : -2;
        }
      }
      send_status_fd(fds[i].fd, status, fd);
      if (fd >= 0) close(fd);
      ++i;
    }
  }
  for (size_t i = 1; i < fds.size(); ++i) close(fds[i].fd);
}

int HbmPool::take_free_page(std::string* err) {
  // lowest index first; a free page that still carries a stale mapping elsewhere is the last
  // resort, and loses that mapping before it is mapped anew (one page, one mapping)
  // (called with the table locked)
  int stale = -1;
  for (int i = 0; i < num_pages_; ++i) {
    if (table_->owner[i] != kOwnerFree) continue;
    if (page_slot_[i] < 0) return i;
    if (stale < 0) stale = i;
  }
  if (stale >= 0) {
    const int64_t slot = page_slot_[stale];
    if (!backend_->unmap(base_ + static_cast<uint64_t>(slot) * page_bytes_, 1, err)) return -1;
    ++n_unmap_;
    ++n_unmap_calls_;
    slot_page_[slot] = -1;
    page_slot_[stale] = -1;
    set_creator_mapped(stale, false);
  }
  return stale;
}

bool HbmPool::ensure_mapped(uint64_t off, size_t n, std::string* err) {
  const uint64_t first = off / page_bytes_, last = (off + n - 1) / page_bytes_;
  {
    bool all_live = true;
    for (uint64_t s = first; s <= last && all_live; ++s) all_live = slot_live_[s] != 0;
    if (all_live) return true;   // the common case touches no shared state
  }
  // ownership changes from here on: the table is locked against the other processes
  ShmLock table_lock(&table_->mu);
  // a slot whose page was handed back but is still free gets it back without a driver call
  for (uint64_t s = first; s <= last; ++s) {
    const int page = slot_page_[s];
    if (page >= 0 && !slot_live_[s] && table_->owner[page] == kOwnerFree) {
      set_owner(page, kOwnerTrain);
      set_creator_mapped(page, false);   // training's again: nobody waits for this mapping to go
      slot_live_[s] = 1;
      ++n_revive_;
    }
  }
  // count what is missing before touching anything: running out of pages is found before the first driver call
  auto count_missing = [&] {
    int m = 0;
    for (uint64_t s = first; s <= last; ++s) m += slot_live_[s] ? 0 : 1;
    return m;
  };
  auto count_free = [&] {
    int f = 0;
    for (int i = 0; i < num_pages_; ++i) f += table_->owner[i] == kOwnerFree ? 1 : 0;
    return f;
  };
  int missing = count_missing();
  if (missing == 0) return true;
  // a peer that died without detaching still owns its pages in the table: they come back first
  if (count_free() < missing) sweep_dead_owners_table_locked();
  if (count_free() < missing) {
    // pages cached under free blocks elsewhere may cover the shortfall
    empty_cache_table_locked();
    missing = count_missing();
    const int free_pages = count_free();
    if (free_pages < missing) {
      if (err) *err = "out of pool memory: need " + std::to_string(missing) + " pages, " + std::to_string(free_pages) + " free";
      return false;
    }
  }
  // access rights are set once per run of newly mapped neighbours (the driver call costs the same for
  // one page and for a hundred)
  uint64_t run_first = 0, run_len = 0;
  auto close_run = [&]() -> bool {
    if (run_len == 0) return true;
    const bool ok = backend_->set_access(base_ + run_first * page_bytes_, run_len * page_bytes_, err);
    run_len = 0;
    return ok;
  };
  // A driver call that fails in the middle leaves the slots mapped so far live and owned by training (the caller
  // frees the block, and the next request over them takes the fast path above): they must not be left without
  // access rights, so the open run is closed before the failure is reported.
  auto fail = [&]() -> bool {
    std::string ignored;
    if (run_len) (void)backend_->set_access(base_ + run_first * page_bytes_, run_len * page_bytes_, &ignored);
    run_len = 0;
    return false;
  };
  for (uint64_t s = first; s <= last; ++s) {
    if (slot_live_[s]) {
      if (!close_run()) return false;
      continue;
    }
    if (slot_page_[s] >= 0) {
      // the page this slot used to hold now belongs to someone else: drop the stale mapping
      const int old = slot_page_[s];
      if (!backend_->unmap(base_ + s * page_bytes_, 1, err)) return fail();
      ++n_unmap_;
      ++n_unmap_calls_;
      page_slot_[old] = -1;
      slot_page_[s] = -1;
      set_creator_mapped(old, false);
    }
    const int page = take_free_page(err);
    if (page < 0) return fail();
    if (!backend_->map(base_ + s * page_bytes_, page, err)) return fail();
    set_owner(page, kOwnerTrain);
    slot_page_[s] = page;
    page_slot_[page] = static_cast<int64_t>(s);
    slot_live_[s] = 1;
    ++n_map_;
    if (run_len == 0) run_first = s;
    ++run_len;
  }
  return close_run();
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
    const uint64_t new_frontier = round_up(start + n, page_bytes_);
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
  ShmLock table_lock(&table_->mu);
  return empty_cache_table_locked();
}

size_t HbmPool::empty_cache_table_locked() {
  // Every page that lies wholly inside free blocks goes back as FREE.  Eager mode removes the page's
  // mapping first, so that what the table calls FREE is mapped nowhere in this process and another
  // process may take it: one driver call per run of neighbouring slots (0.26 ms per mapping in the run on
  // MI355X, whatever the page size).  Lazy mode relabels only: the mapping stays (stale), is reused for
  // free if the page is still FREE when the range grows again, and is removed when the slot needs
  // another page, when the page is needed elsewhere, or by trim().
  std::vector<uint64_t> slots;
  for (Segment* s : {&small_, &large_}) {
    for (auto& kv : s->blocks) {
      if (kv.second.allocated) continue;
      const uint64_t lo = round_up(kv.first, page_bytes_);
      const uint64_t hi = (kv.first + kv.second.size) / page_bytes_ * page_bytes_;
      for (uint64_t a = lo; a + page_bytes_ <= hi; a += page_bytes_) {
        const uint64_t slot = a / page_bytes_;
        if (slot_page_[slot] >= 0 && slot_live_[slot]) slots.push_back(slot);
      }
    }
  }
  if (slots.empty()) return 0;
  // a freed block may still be read by launches in flight on its own stream (frees are stream
  // ordered): nothing may be running when its pages change hands
  backend_->quiesce();
  std::sort(slots.begin(), slots.end());
  if (!lazy_unmap_) {
    for (size_t i = 0; i < slots.size();) {
      size_t j = i + 1;
      while (j < slots.size() && slots[j] == slots[j - 1] + 1) ++j;
      std::string err;
      if (backend_->unmap(base_ + slots[i] * page_bytes_, static_cast<int>(j - i), &err)) {
        n_unmap_ += j - i;
        ++n_unmap_calls_;
        for (size_t k = i; k < j; ++k) {
          page_slot_[slot_page_[slots[k]]] = -1;
          set_owner(slot_page_[slots[k]], kOwnerFree);
          slot_page_[slots[k]] = -1;
          slot_live_[slots[k]] = 0;
        }
      } else {
        // the driver refused: these pages stay with training (nothing was handed over)
        for (size_t k = i; k < j; ++k) slots[k] = UINT64_MAX;
      }
      i = j;
    }
    size_t bytes = 0;
    for (uint64_t sl : slots) bytes += sl == UINT64_MAX ? 0 : page_bytes_;
    return bytes;
  }
  for (uint64_t slot : slots) {
    slot_live_[slot] = 0;
    set_creator_mapped(slot_page_[slot], true);   // before the page shows as FREE: a claimer must see the flag
    set_owner(slot_page_[slot], kOwnerFree);
  }
  return slots.size() * page_bytes_;
}

size_t HbmPool::trim(size_t max_pages) {
  std::lock_guard<std::mutex> lock(mu_);
  size_t n = 0;
  for (size_t slot = 0; slot < slot_page_.size() && n < max_pages;) {
    if (slot_page_[slot] < 0 || slot_live_[slot]) {
      ++slot;
      continue;
    }
    size_t end = slot + 1;
    while (end < slot_page_.size() && end - slot < max_pages - n && slot_page_[end] >= 0 && !slot_live_[end]) ++end;
    std::string err;
    if (backend_->unmap(base_ + slot * page_bytes_, static_cast<int>(end - slot), &err)) {
      n_unmap_ += end - slot;
      ++n_unmap_calls_;
      for (size_t k = slot; k < end; ++k) {
        set_creator_mapped(slot_page_[k], false);
        page_slot_[slot_page_[k]] = -1;
        slot_page_[k] = -1;
      }
      n += end - slot;
    }
    slot = end;
  }
  return n;
}

size_t HbmPool::empty_cache() {
  process_events();
  // Before any lock: a launch that still waits in a software launch queue is on no stream yet, so the device
  // synchronisation inside the locked part would not see it, and it may refer to a block freed since (frees are
  // stream ordered).  Draining here also keeps the wait out of the cross-process table lock: the quiesce that
  // follows under the locks finds an idle device.
  std::function<void()> hook;
  {
    std::lock_guard<std::mutex> lock(mu_);
    hook = quiesce_hook_;
  }
  if (hook) hook();
  backend_->quiesce();
  std::lock_guard<std::mutex> lock(mu_);
  return empty_cache_locked();
}

void HbmPool::set_quiesce_hook(std::function<void()> fn) {
  std::lock_guard<std::mutex> lock(mu_);
  quiesce_hook_ = std::move(fn);
}

int HbmPool::sweep_dead_owners_table_locked() {
  // The robust mutex covers a process that dies holding the table's lock; this covers one that dies holding
  // PAGES (killed, crashed, or gone without detaching): its mappings went with it, the labels stay.  kill(pid, 0)
  // says ESRCH for a pid that names no process.
  const int32_t me = static_cast<int32_t>(getpid());
  int freed = 0;
  for (int i = 0; i < num_pages_; ++i) {
    if (table_->owner[i] != kOwnerInfer) continue;
    const int32_t pid = table_->owner_pid[i];
    if (pid == me || pid <= 0) continue;
    if (kill(static_cast<pid_t>(pid), 0) != 0 && errno == ESRCH) {
      table_->owner[i] = kOwnerFree;
      table_->owner_pid[i] = 0;
      table_->changes++;
      ++freed;
    }
  }
  return freed;
}

PoolStats HbmPool::stats() {
  std::lock_guard<std::mutex> lock(mu_);
  PoolStats st{};
  st.pool_bytes = pool_bytes_;
  st.page_bytes = page_bytes_;
  st.train_usage = train_usage_;
  st.train_peak_usage = train_peak_;
  size_t train_pages = 0, infer_pages = 0, free_pages = 0;
  {
    ShmLock table_lock(&table_->mu);
    sweep_dead_owners_table_locked();
    for (int i = 0; i < num_pages_; ++i) {
      const uint8_t o = table_->owner[i];
      train_pages += o == kOwnerTrain;
      infer_pages += o == kOwnerInfer;
      free_pages += o == kOwnerFree;
    }
  }
  st.train_all_usage = train_pages * page_bytes_;
  st.infer_usage = infer_pages * page_bytes_;
  st.free_pages = free_pages;
  st.num_allocs = n_alloc_;
  st.num_frees = n_free_;
  st.num_maps = n_map_;
  st.num_unmaps = n_unmap_;
  st.num_revives = n_revive_;
  st.num_unmap_calls = n_unmap_calls_;
  for (size_t s = 0; s < slot_page_.size(); ++s) st.stale_pages += slot_page_[s] >= 0 && !slot_live_[s] ? 1 : 0;
  return st;
}

int64_t HbmPool::offset_of(const void* ptr) const {
  const uint64_t a = reinterpret_cast<uint64_t>(ptr);
  if (a < base_ || a >= base_ + va_bytes_) return -1;
  return static_cast<int64_t>(a - base_);
}

int HbmPool::page_table(uint8_t* owner_out, int64_t* slot_out, int max_pages) {
  std::lock_guard<std::mutex> lock(mu_);
  ShmLock table_lock(&table_->mu);
  const int n = std::min(max_pages, num_pages_);
  for (int i = 0; i < n; ++i) {
    if (owner_out) owner_out[i] = table_->owner[i];
    if (slot_out) slot_out[i] = page_slot_[i];
  }
  return n;
}

int HbmPool::infer_claim_pages(int n) {
  std::lock_guard<std::mutex> lock(mu_);
  ShmLock table_lock(&table_->mu);
  int moved = 0;
  for (int i = 0; i < num_pages_ && moved < n; ++i)
    if (table_->owner[i] == kOwnerFree) {
      set_owner(i, kOwnerInfer);
      ++moved;
    }
  return moved;
}

int HbmPool::infer_release_pages(int n) {
  std::lock_guard<std::mutex> lock(mu_);
  ShmLock table_lock(&table_->mu);
  const int32_t me = static_cast<int32_t>(getpid());
  int moved = 0;
  for (int i = num_pages_ - 1; i >= 0 && moved < n; --i)
    if (table_->owner[i] == kOwnerInfer && table_->owner_pid[i] == me) {
      set_owner(i, kOwnerFree);
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

std::shared_ptr<HbmPool> pool(int device) {
  if (device < 0 || device >= kMaxDeviceNum) return nullptr;
  std::lock_guard<std::mutex> lock(g_pools_mu);
  return g_pools[device];
}

bool pool_init(int device, size_t pool_bytes, bool use_gpu, const PoolOptions& opt, std::string* err) {
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
  g_pools[device].reset(HbmPool::create(device, pool_bytes, be, opt, err));
  if (g_pools[device]) ++g_generation[device];
  return g_pools[device] != nullptr;
}

uint64_t pool_generation(int device) {
  std::lock_guard<std::mutex> lock(g_pools_mu);
  return device >= 0 && device < kMaxDeviceNum ? g_generation[device] : 0;
}

void pool_shutdown(int device) {
  // out of the table first; the pool itself goes when the last caller inside it has left
  std::shared_ptr<HbmPool> last;
  {
    std::lock_guard<std::mutex> lock(g_pools_mu);
    if (device >= 0 && device < kMaxDeviceNum) last.swap(g_pools[device]);
  }
}

// ---------------------------------------------------------------------------
// PoolPeer: the page table and the pages as another process sees them
// ---------------------------------------------------------------------------

bool peer_map_descriptor(int device, int fd, size_t expect_bytes, void** ptr, std::string* err);   // mem_pool_hip.cc
bool peer_unmap(void* ptr, std::string* err);

PoolPeer* PoolPeer::attach(int device, std::string* err) {
  std::unique_ptr<PoolPeer> p(new PoolPeer());
  p->device_ = device;
  p->seg_.reset(ShmSegment::open(page_table_name(device), sizeof(PageTableLayout), false, false, err));
  if (!p->seg_) return nullptr;
  p->table_ = static_cast<PageTableLayout*>(p->seg_->base());
  sockaddr_un addr;
  const socklen_t len = abstract_addr(page_table_name(device), &addr);
  p->sock_ = socket(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0);
  if (p->sock_ < 0 || connect(p->sock_, reinterpret_cast<sockaddr*>(&addr), len) != 0) {
    if (err) *err = std::string("descriptor server of the pool's creator: ") + strerror(errno);
    return nullptr;
  }
  return p.release();
}

PoolPeer::~PoolPeer() {
  std::vector<int> mine;
  {
    std::lock_guard<std::mutex> lock(mu_);
    for (auto& kv : mapped_) {
      std::string err;
      peer_unmap(kv.second, &err);
    }
    mapped_.clear();
  }
  // whatever this process still owns goes back
  if (table_) {
    ShmLock t(&table_->mu);
    const int32_t me = static_cast<int32_t>(getpid());
    for (int i = 0; i < table_->num_pages; ++i)
      if (table_->owner[i] == kOwnerInfer && table_->owner_pid[i] == me) {
        table_->owner[i] = kOwnerFree;
        table_->owner_pid[i] = 0;
        table_->changes++;
      }
  }
  if (sock_ >= 0) close(sock_);
}

int PoolPeer::free_pages() {
  ShmLock t(&table_->mu);
  int n = 0;
  for (int i = 0; i < table_->num_pages; ++i) n += table_->owner[i] == kOwnerFree;
  return n;
}

int PoolPeer::claim(int n, int* pages_out) {
  ShmLock t(&table_->mu);
  const int32_t me = static_cast<int32_t>(getpid());
  int got = 0;
  for (int i = 0; i < table_->num_pages && got < n; ++i)
    if (table_->owner[i] == kOwnerFree) {
      table_->owner[i] = kOwnerInfer;
      table_->owner_pid[i] = me;
      table_->changes++;
      if (pages_out) pages_out[got] = i;
      ++got;
    }
  return got;
}

int PoolPeer::release(const int* pages, int n) {
  const int32_t me = static_cast<int32_t>(getpid());
  int done = 0;
  for (int k = 0; k < n; ++k) {
    const int page = pages[k];
    if (page < 0 || page >= table_->num_pages) continue;
    std::string err;
    unmap(page, &err);   // nothing of a page given back stays mapped here
    ShmLock t(&table_->mu);
    if (table_->owner[page] == kOwnerInfer && table_->owner_pid[page] == me) {
      table_->owner[page] = kOwnerFree;
      table_->owner_pid[page] = 0;
      table_->changes++;
      ++done;
    }
  }
  return done;
}

int PoolPeer::fetch_fd(int page, std::string* err) {
  FdRequest rq{page};
  if (send(sock_, &rq, sizeof(rq), MSG_NOSIGNAL) != static_cast<ssize_t>(sizeof(rq))) {
    if (err) *err = std::string("asking the pool's creator for a page descriptor: ") + strerror(errno);
    return -1;
  }
  int32_t status = -1;
  int fd = -1;
  if (!recv_status_fd(sock_, &status, &fd)) {
    if (err) *err = "the pool's creator closed the descriptor channel";
    return -1;
  }
  if (status != 0 || fd < 0) {
    if (fd >= 0) close(fd);
    if (err) *err = status == -1 ? "the page table does not name this process as the owner of page " + std::to_string(page)
                                 : "the pool's creator could not export page " + std::to_string(page);
    return -1;
  }
  return fd;
}

int PoolPeer::still_mapped_by_creator(const int* pages, int n) {
  int cnt = 0;
  for (int k = 0; k < n; ++k)
    if (pages[k] >= 0 && pages[k] < table_->num_pages)
      cnt += __atomic_load_n(&table_->creator_mapped[pages[k]], __ATOMIC_ACQUIRE) ? 1 : 0;
  return cnt;
}

void* PoolPeer::map(int page, std::string* err, int wait_ms) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = mapped_.find(page);
  if (it != mapped_.end()) return it->second;
  if (page < 0 || page >= table_->num_pages) {
    if (err) *err = "no such page";
    return nullptr;
  }
  // a page handed back lazily is FREE (and claimable) before its old mapping is gone: wait for that
  for (int waited_us = 0; __atomic_load_n(&table_->creator_mapped[page], __ATOMIC_ACQUIRE); waited_us += 50) {
    if (waited_us >= wait_ms * 1000) {
      if (err) *err = "page " + std::to_string(page) + " is still mapped by the process that handed it back";
      return nullptr;
    }
    usleep(50);
  }
  if (!table_->has_device) {
    if (err) *err = "this pool is the CPU model: its pages have no device memory";
    return nullptr;
  }
  const int fd = fetch_fd(page, err);
  if (fd < 0) return nullptr;
  void* ptr = nullptr;
  const bool ok = peer_map_descriptor(device_, fd, table_->page_bytes, &ptr, err);
  close(fd);
  if (!ok) return nullptr;
  mapped_[page] = ptr;
  return ptr;
}

bool PoolPeer::unmap(int page, std::string* err) {
  std::lock_guard<std::mutex> lock(mu_);
  auto it = mapped_.find(page);
  if (it == mapped_.end()) return true;
  const bool ok = peer_unmap(it->second, err);
  mapped_.erase(it);
  return ok;
}

}  // namespace host
}  // namespace tch
