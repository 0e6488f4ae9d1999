// Library plumbing: last-error slot, per-stream scratch arena, buffer knobs.
#include <atomic>
#include <chrono>
#include <thread>
#include <map>
#include <mutex>

#include "common.h"

namespace mnt {

static thread_local std::string g_last_error;

void set_last_error(const std::string &message) { g_last_error = message; }

static std::mutex g_arena_mutex;
static std::map<std::pair<int, hipStream_t>, Arena *> g_arenas;

Arena &Arena::of(hipStream_t stream) {
  int device = 0;
  MNT_HIP(hipGetDevice(&device));
  std::lock_guard<std::mutex> lock(g_arena_mutex);
  auto key = std::make_pair(device, stream);
  auto it = g_arenas.find(key);
  if (it == g_arenas.end()) it = g_arenas.emplace(key, new Arena(stream)).first;
  return *it->second;
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

void Arena::add_page(size_t bytes) {
  Page page;
  page.size = align_up(bytes, 256);
  page.used = 0;
  MNT_HIP(hipMalloc(reinterpret_cast<void **>(&page.base), page.size));
  pages_.push_back(page);
}

void *Arena::alloc(size_t bytes) {
  bytes = align_up(bytes ? bytes : 1, 256);
  for (size_t p = cursor_; p < pages_.size(); ++p) {
    if (p != cursor_) pages_[p].used = 0;
    if (pages_[p].used + bytes <= pages_[p].size) {
      void *ptr = pages_[p].base + pages_[p].used;
      pages_[p].used += bytes;
      cursor_ = p;
      return ptr;
    }
  }
  size_t want = static_cast<size_t>(static_cast<double>(bytes) * (1.0 + (growth_ > 0 ? growth_ : 0)));
  size_t pages = (want + page_size_ - 1) / page_size_;
  add_page(pages * page_size_);
  cursor_ = pages_.size() - 1;
  pages_[cursor_].used = bytes;
  return pages_[cursor_].base;
}

Arena::Mark Arena::mark() const {
  if (pages_.empty()) return Mark{0, 0};
  return Mark{cursor_, pages_[cursor_].used};
}

void Arena::release(const Mark &m) {
  if (pages_.empty()) return;
  for (size_t p = m.page + 1; p < pages_.size(); ++p) pages_[p].used = 0;
  cursor_ = m.page;
  if (cursor_ < pages_.size()) pages_[cursor_].used = m.used;
}

void Arena::preallocate(size_t bytes) {
  size_t have = 0;
  for (const auto &p : pages_) have = p.size > have ? p.size : have;
  if (have >= bytes) return;
  add_page(align_up(bytes, page_size_));
}

void Arena::free_all(bool synchronise) {
  if (synchronise) MNT_HIP(hipStreamSynchronize(stream_));
  for (auto &p : pages_) MNT_HIP(hipFree(p.base));
  pages_.clear();
  cursor_ = 0;
  for (int slot = 0; slot < 2; ++slot) {
    if (persistent_[slot]) {
      MNT_HIP(hipFree(persistent_[slot]));
      persistent_[slot] = nullptr;
      persistent_size_[slot] = 0;
    }
  }
  pending.valid = false;
  map_state_valid = false;
  zero_bitmap_words = 0;
}

void Arena::reset_device() {
  int device = 0;
  MNT_HIP(hipGetDevice(&device));
  std::lock_guard<std::mutex> lock(g_arena_mutex);
  for (auto it = g_arenas.begin(); it != g_arenas.end();) {
    if (it->first.first != device) {
      ++it;
      continue;
    }
    Arena *arena = it->second;
    arena->free_all(false);               // the caller has waited for the whole device; the stream may be gone
    if (arena->pinned_ != nullptr) {
      MNT_HIP(hipHostFree(arena->pinned_));
      arena->pinned_ = nullptr;
      arena->pinned_device_ = nullptr;
    }
    delete arena;
    it = g_arenas.erase(it);
  }
}

size_t Arena::total() const {
  size_t t = 0;
  for (const auto &p : pages_) t += p.size;
  return t;
}

size_t Arena::used() const {
  size_t t = 0;
  for (size_t p = 0; p < pages_.size() && p <= cursor_; ++p) t += pages_[p].used;
  return t;
}

void *Arena::pinned() {
  if (!pinned_) {
    MNT_HIP(hipHostMalloc(&pinned_, kPinnedBytes, hipHostMallocMapped | hipHostMallocCoherent));
    memset(pinned_, 0, kPinnedBytes);
    MNT_HIP(hipHostGetDevicePointer(&pinned_device_, pinned_, 0));
  }
  return pinned_;
}

void *Arena::pinned_device() {
  pinned();
  return pinned_device_;
}

unsigned long long *Arena::flag_device(int slot) {
  return reinterpret_cast<unsigned long long *>(static_cast<char *>(pinned_device()) + kFlagOffset +
                                                static_cast<size_t>(slot) * 64);
}

static std::atomic<long long> g_host_waits{0}, g_host_wait_ns{0};

void Arena::wait_flag(int slot, unsigned long long sequence) {
  volatile unsigned long long *flag = reinterpret_cast<volatile unsigned long long *>(
      static_cast<char *>(pinned()) + kFlagOffset + static_cast<size_t>(slot) * 64);
  const auto start = std::chrono::steady_clock::now();
  struct Tally {
    std::chrono::steady_clock::time_point since;
    ~Tally() {
      g_host_waits.fetch_add(1, std::memory_order_relaxed);
      g_host_wait_ns.fetch_add(std::chrono::duration_cast<std::chrono::nanoseconds>(
                                   std::chrono::steady_clock::now() - since).count(),
                               std::memory_order_relaxed);
    }
  } tally{start};
  unsigned spins = 0;
  while (*flag != sequence) {
    if ((++spins & 0x3FFFu) == 0) {
      const auto waited = std::chrono::steady_clock::now() - start;
      if (waited > std::chrono::seconds(2)) {
        MNT_HIP(hipStreamSynchronize(stream_));
        MNT_CHECK(*flag == sequence, "a kernel finished without signalling its completion flag");
        break;
      }
    }
    __builtin_ia32_pause();
  }
  std::atomic_thread_fence(std::memory_order_acquire);
}

void *Arena::persistent(int slot, size_t bytes) {
  if (bytes > persistent_size_[slot]) {
    if (persistent_[slot]) {
      MNT_HIP(hipStreamSynchronize(stream_));
      MNT_HIP(hipFree(persistent_[slot]));
    }
    persistent_size_[slot] = align_up(bytes + bytes / 4, 1 << 20);
    MNT_HIP(hipMalloc(&persistent_[slot], persistent_size_[slot]));
    if (slot == 0) zero_bitmap_words = 0;
  }
  return persistent_[slot];
}

// ---- stage profiler -------------------------------------------------------

static bool g_profile_on = false;
static std::vector<std::pair<const char *, hipEvent_t>> g_marks;
static std::vector<hipEvent_t> g_event_pool;
static constexpr size_t kMaxMarks = 4096;

static std::thread::id g_profile_thread;

int compute_units() {
  static std::atomic<int> known[64];
  int device = 0;
  MNT_HIP(hipGetDevice(&device));
  const int slot = device & 63;
  int units = known[slot].load(std::memory_order_relaxed);
  if (units == 0) {
    MNT_HIP(hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device));
    units = units > 0 ? units : 256;
    known[slot].store(units, std::memory_order_relaxed);
  }
  return units;
}

void profile_mark(const char *label, hipStream_t stream) {
  // marks are kept for the thread that turned profiling on: the look-ahead
  // worker runs the same entry points on another stream at the same time
  if (!g_profile_on || std::this_thread::get_id() != g_profile_thread || g_marks.size() >= kMaxMarks) return;
  hipEvent_t event;
  if (!g_event_pool.empty()) {
    event = g_event_pool.back();
    g_event_pool.pop_back();
  } else {
    MNT_HIP(hipEventCreate(&event));
  }
  MNT_HIP(hipEventRecord(event, stream));
  g_marks.emplace_back(label, event);
}

static void profile_clear() {
  for (auto &m : g_marks) g_event_pool.push_back(m.second);
  g_marks.clear();
}

}  // namespace mnt

using namespace mnt;

extern "C" {

int mnt_abi_version(void) { return 1; }

const char *mnt_last_error(void) { return g_last_error.c_str(); }

int mnt_buffer_preallocate(void *stream, size_t bytes) {
  return guarded([&] { Arena::of(static_cast<hipStream_t>(stream)).preallocate(bytes); });
}

int mnt_buffer_free(void *stream) {
  return guarded([&] { Arena::of(static_cast<hipStream_t>(stream)).free_all(); });
}

int mnt_buffer_set_growth(void *stream, float growth) {
  return guarded([&] { Arena::of(static_cast<hipStream_t>(stream)).set_growth(growth); });
}

int mnt_buffer_set_page_size(void *stream, size_t bytes) {
  return guarded([&] { Arena::of(static_cast<hipStream_t>(stream)).set_page_size(bytes); });
}

size_t mnt_buffer_total_size(void *stream) {
  size_t value = 0;
  guarded([&] { value = Arena::of(static_cast<hipStream_t>(stream)).total(); });
  return value;
}

size_t mnt_buffer_used_size(void *stream) {
  size_t value = 0;
  guarded([&] { value = Arena::of(static_cast<hipStream_t>(stream)).used(); });
  return value;
}

int mnt_profile_enable(int on) {
  return guarded([&] {
    profile_clear();
    g_profile_thread = std::this_thread::get_id();
    g_profile_on = on != 0;
  });
}

int mnt_profile_read(int capacity, float *ms_out, char *labels_out, int label_stride,
                     int *count_out) {
  return guarded([&] {
    MNT_CHECK(ms_out != nullptr && labels_out != nullptr && count_out != nullptr && label_stride > 1,
              "bad argument");
    int count = 0;
    if (!g_marks.empty()) MNT_HIP(hipEventSynchronize(g_marks.back().second));
    for (size_t i = 1; i < g_marks.size() && count < capacity; ++i) {
      float ms = 0.0f;
      MNT_HIP(hipEventElapsedTime(&ms, g_marks[i - 1].second, g_marks[i].second));
      ms_out[count] = ms;
      snprintf(labels_out + static_cast<size_t>(count) * label_stride, label_stride, "%s",
               g_marks[i].first);
      ++count;
    }
    *count_out = count;
    profile_clear();
  });
}

int mnt_reset_error(void) {
  (void)hipGetLastError();
  g_last_error.clear();
  return 0;
}

int mnt_host_wait_stats(int64_t *waits_out, int64_t *nanoseconds_out, int reset) {
  return guarded([&] {
    if (waits_out != nullptr) *waits_out = g_host_waits.load(std::memory_order_relaxed);
    if (nanoseconds_out != nullptr) *nanoseconds_out = g_host_wait_ns.load(std::memory_order_relaxed);
    if (reset) {
      g_host_waits.store(0, std::memory_order_relaxed);
      g_host_wait_ns.store(0, std::memory_order_relaxed);
    }
  });
}

int mnt_device_reset(void) {
  return guarded([&] {
    if (mnt_lookahead_finish(nullptr) != 0) throw Error{mnt_last_error()};
    MNT_HIP(hipDeviceSynchronize());
    Arena::reset_device();
    (void)hipGetLastError();
    g_last_error.clear();
  });
}

}  // extern "C"
