// Shared host-side plumbing of libminuet_hip: error reporting, the per-stream
// scratch arena, launch geometry and small device helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/minuet_hip.h"

namespace mnt {

// ---------------------------------------------------------------- errors ----

struct Error {
  std::string message;
};

void set_last_error(const std::string &message);

[[noreturn]] inline void fail(const char *file, int line, const char *fmt, ...) {
  char body[768];
  va_list args;
  va_start(args, fmt);
  vsnprintf(body, sizeof(body), fmt, args);
  va_end(args);
  char full[1024];
  const char *base = strrchr(file, '/');
  snprintf(full, sizeof(full), "[Minuet] [%s (%d)] %s", base ? base + 1 : file, line, body);
  throw Error{full};
}

#define MNT_FAIL(...) ::mnt::fail(__FILE__, __LINE__, __VA_ARGS__)
#define MNT_CHECK(cond, ...)                 \
  do {                                       \
    if (!(cond)) MNT_FAIL(__VA_ARGS__);      \
  } while (0)
#define MNT_HIP(expr)                                                          \
  do {                                                                         \
    hipError_t status_ = (expr);                                               \
    if (status_ != hipSuccess)                                                 \
      MNT_FAIL("%s failed: %s", #expr, hipGetErrorString(status_));            \
  } while (0)

// One caller thread per stream at a time: the scratch arena of a stream, the
// state its two-phase entry points hand from call to call and its pinned
// block have no locks of their own.  A library call takes the arena of every
// stream it touches for the calling thread until it returns (calls nest: an
// entry point may go through others); a thread that enters the library on a
// stream another thread is inside of gets an error instead of a data race.
// (The reference is called with the interpreter lock held,
// csrc/minuet/torch/common.h:17-21; a ctypes call releases that lock.)
void enter_call();
void leave_call();

struct CallDepth {
  CallDepth() { enter_call(); }
  ~CallDepth() { leave_call(); }
};

// Wraps the body of every extern "C" entry point.
template <typename Fn>
inline int guarded(Fn &&fn) {
  CallDepth depth;
  try {
    fn();
    return 0;
  } catch (const Error &e) {
    set_last_error(e.message);
    return 1;
  } catch (const std::exception &e) {
    set_last_error(std::string("[Minuet] ") + e.what());
    return 2;
  }
}

// ----------------------------------------------------------------- arena ----

// Per-stream LIFO scratch arena over hipMalloc pages.  Everything a call
// borrows is released when its Scope ends; memory is reused by later work on
// the same stream, which is ordered after the earlier work.
class Arena {
 public:
  // The arena of `stream` on the current device, taken for the calling thread
  // until its outermost library call returns (see enter_call); fails when
  // another thread holds it.
  static Arena &of(hipStream_t stream);
  // Keeps / gives up the arena for the calling thread across calls
  // (mnt_stream_acquire / mnt_stream_release).
  static void pin(hipStream_t stream);
  static void unpin(hipStream_t stream);
  // Gives back everything the library holds on the current device: the arenas
  // of all its streams (pages, persistent blocks, pinned staging blocks).
  static void reset_device();

  struct Mark {
    size_t page;
    size_t used;
  };

  void *alloc(size_t bytes);
  Mark mark() const;
  void release(const Mark &m);
  void preallocate(size_t bytes);
  void free_all(bool synchronise = true);
  size_t total() const;
  size_t used() const;
  void set_growth(float g) { growth_ = g; }
  void set_page_size(size_t b) { page_size_ = b ? b : page_size_; }

  // Pinned host staging block (64 KiB) for small read-backs and uploads.
  static constexpr size_t kPinnedBytes = 64 * 1024;
  void *pinned();
  // Device-side address of the same block (kernels may write results there).
  void *pinned_device();
  // Completion handshake through the pinned block: a kernel ends by storing a
  // fresh sequence number into flag word `slot` (after its results, with a
  // system-scope release); wait_flag spins on that word on the host, which
  // is several times quicker than a stream synchronisation.  After two
  // seconds it falls back to hipStreamSynchronize so that a failed kernel
  // surfaces as an error instead of a hang.
  static constexpr size_t kFlagOffset = 512;      // 8 words of 64 bytes each
  static constexpr size_t kPlanOffset = 1024;     // mirrored sizes / order
  unsigned long long next_sequence() { return ++sequence_; }
  unsigned long long *flag_device(int slot);
  void wait_flag(int slot, unsigned long long sequence);
  // Long-lived device blocks that survive scopes (state of the two-phase entry
  // points; slot 0: target coordinates, slot 1: kernel-map build).  Grows to
  // at least `bytes`; 0 returns the current block.
  void *persistent(int slot, size_t bytes);

  hipStream_t stream() const { return stream_; }

  // State handed from mnt_target_coordinates_count to ..._fill.
  struct Pending {
    bool valid = false;
    int64_t count = 0, n = 0, num_batches = 0;
    int ndim = 0, coord_dtype = 0, index_dtype = 0;
    const void *batch_dims = nullptr;
    alignas(8) unsigned char blob[256] = {0};
  } pending;

  // The target bitmap in persistent block 0 is left all zero by the kernel
  // that walks it: the words from the block's start on that are known to be
  // zero (0 after anything else has written there, or after the block moved).
  long long zero_bitmap_words = 0;
  long long zero_bitmap_words_after = 0;   // what the count becomes once the walk of the build under way is launched

  // State handed from mnt_kernel_map_query to mnt_kernel_map_emit.
  bool map_state_valid = false;
  alignas(8) unsigned char map_state[64] = {0};

 private:
  struct Page {
    char *base;
    size_t size;
    size_t used;
  };
  explicit Arena(hipStream_t s) : stream_(s) {}
  void add_page(size_t bytes);
  friend void leave_call();

  hipStream_t stream_;
  std::vector<Page> pages_;
  size_t cursor_ = 0;
  size_t page_size_ = size_t(8) << 20;
  float growth_ = 1.0f;
  void *pinned_ = nullptr;
  void *pinned_device_ = nullptr;
  unsigned long long sequence_ = 0;
  void *persistent_[2] = {nullptr, nullptr};
  size_t persistent_size_[2] = {0, 0};
  // guarded by the registry's mutex
  bool held_ = false, pinned_by_thread_ = false;
  unsigned long long holder_ = 0;            // token of the thread inside a call / that pinned it
};

class Scope {
 public:
  explicit Scope(hipStream_t stream) : arena_(Arena::of(stream)), mark_(arena_.mark()) {}
  ~Scope() { arena_.release(mark_); }
  template <typename T>
  T *alloc(size_t count) {
    return static_cast<T *>(arena_.alloc(count * sizeof(T)));
  }
  Arena &arena() { return arena_; }

 private:
  Arena &arena_;
  Arena::Mark mark_;
};

// ------------------------------------------------------------- profiling ----

// Records a timestamp event on `stream` when stage profiling is on (see
// mnt_profile_enable); the interval since the previous mark is reported under
// `label`, which must be a string literal.
void profile_mark(const char *label, hipStream_t stream);

// ---------------------------------------------------------------- launch ----

// Compute units of the current device (asked for once per device).
int compute_units();

inline int64_t div_ceil(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline unsigned grid_for(int64_t items, int block, int64_t cap = (int64_t(1) << 20)) {
  int64_t g = div_ceil(items, block);
  if (g < 1) g = 1;
  if (g > cap) g = cap;
  return static_cast<unsigned>(g);
}

inline void check_launch(const char *what) {
  hipError_t status = hipGetLastError();
  if (status != hipSuccess) MNT_FAIL("launch of %s failed: %s", what, hipGetErrorString(status));
}

inline int int_size(int dtype) {
  MNT_CHECK(dtype == MNT_INT32 || dtype == MNT_INT64, "unsupported integer dtype code %d", dtype);
  return dtype == MNT_INT32 ? 4 : 8;
}

inline int float_size(int dtype) {
  MNT_CHECK(dtype == MNT_FLOAT32 || dtype == MNT_FLOAT16 || dtype == MNT_BFLOAT16,
            "unsupported float dtype code %d", dtype);
  return dtype == MNT_FLOAT32 ? 4 : 2;
}

// Packing frame of voxel keys: field k of a row holds c[k] - lo[k] shifted left
// by shift[k]; field 0 is the batch id when batches are present.  Fields are
// wide enough that adding any kernel offset never borrows from or carries
// into a neighbouring field, so key(q + delta) == key(q) + key_delta(delta).
struct Frame {
  long long lo[MNT_MAX_NDIM];
  int shift[MNT_MAX_NDIM];
  int width[MNT_MAX_NDIM];
  int batch_shift;
  int batch_width;
  int ndim;
  int total_bits;
};

}  // namespace mnt
