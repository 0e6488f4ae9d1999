// Building a pass's coordinate levels and kernel maps ahead of the layers that
// ask for them: a worker thread walks a list of requests (what the previous
// pass asked for) through the library's own entry points on a stream of its
// own, while the caller's thread goes on enqueueing layers.  The reference
// builds every map at the first layer that needs it
// (minuet/nn/convolutions.py:58-173), so its host thread alternates between
// map building and layer launches; here the two run side by side.
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <thread>

#include "common.h"

namespace mnt {
namespace {

constexpr int kPending = -1;

struct Level {
  const void *coords = nullptr;
  int64_t n = 0;
  const void *batch_dims = nullptr;
  bool known = false;            // row count and coordinates exist
  bool bounds_known = false;
  int64_t bounds[8] = {0};
};

struct Session {
  std::vector<mnt_lookahead_item> items;
  std::vector<Level> levels;
  std::vector<int> status;                 // kPending, 0 = built, > 0 = failed
  std::vector<int64_t> size;
  std::vector<std::string> message;
  std::vector<hipEvent_t> built;           // recorded on the worker's stream after each item
  int ndim = 0, coord_dtype = 0, index_dtype = 0, device = 0;
  int64_t num_batches = 1;
  int64_t *bounds_out = nullptr;
  int32_t *bounds_known_out = nullptr;
  hipEvent_t inputs_ready = nullptr;       // recorded on the caller's stream at the start
  hipEvent_t session_end = nullptr;        // recorded on the worker's stream behind the last item, built or failed
  bool end_recorded = false;
};

// The worker outlives main(): what it waits on is never destroyed.
std::mutex &g_mutex = *new std::mutex;
std::condition_variable &g_wake = *new std::condition_variable;
std::condition_variable &g_progress = *new std::condition_variable;
bool g_worker_started = false;
bool g_job_posted = false;                 // a session waits for the worker
bool g_busy = false;                       // the worker is inside a session
bool g_active = false;                     // a session exists (started, not finished)
Session &g_session = *new Session;
hipStream_t g_stream[16] = {nullptr};      // the worker's stream, per device
std::vector<hipEvent_t> &g_event_pool = *new std::vector<hipEvent_t>;

hipEvent_t take_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e;
  MNT_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  return e;
}

void derive_bounds(const Level &source, const int64_t *stride, int ndim, Level &target) {
  // floor(c / s) * s is monotone: the extremes map to the extremes
  for (int k = 0; k < 4; ++k) {
    target.bounds[k] = source.bounds[k];
    target.bounds[4 + k] = source.bounds[4 + k];
  }
  for (int k = 0; k < ndim; ++k) {
    const int64_t s = stride[k];
    auto floor_to = [s](int64_t v) { return (v >= 0 ? v / s : -((-v + s - 1) / s)) * s; };
    target.bounds[k] = floor_to(source.bounds[k]);
    target.bounds[4 + k] = floor_to(source.bounds[4 + k]);
  }
  target.bounds_known = true;
}

// One item through the entry point a caller would use; throws on failure.
void build_item(Session &s, int index, hipStream_t stream) {
  const mnt_lookahead_item &item = s.items[index];
  const int num_levels = static_cast<int>(s.levels.size());
  const int num_items = static_cast<int>(s.items.size());
  auto need_level = [&](int level) -> Level & {
    MNT_CHECK(level >= 0 && level < num_levels, "item %d names level %d of %d", index, level, num_levels);
    MNT_CHECK(s.levels[level].known, "item %d needs level %d, which no earlier item has built", index, level);
    return s.levels[level];
  };
  auto need_dense = [&](int dense) -> const mnt_lookahead_item & {
    MNT_CHECK(dense >= 0 && dense < index && dense < num_items && s.items[dense].kind == MNT_AHEAD_DENSE,
              "item %d needs a dense map built by an earlier item", index);
    MNT_CHECK(s.status[dense] == 0, "item %d needs item %d, which failed", index, dense);
    return s.items[dense];
  };
  auto must = [&](int status) {
    if (status != 0) throw Error{mnt_last_error()};
  };
  const bool batched = s.levels[0].batch_dims != nullptr;
  switch (item.kind) {
    case MNT_AHEAD_COORDS: {
      Level &source = need_level(item.source_level);
      MNT_CHECK(item.target_level > 0 && item.target_level < num_levels && !s.levels[item.target_level].known,
                "item %d builds level %d, which is out of range or exists", index, item.target_level);
      MNT_CHECK(source.n > 0, "level %d is empty", item.source_level);
      MNT_CHECK(item.capacity >= source.n, "item %d: room for %lld rows, level %d has %lld", index,
                (long long)item.capacity, item.source_level, (long long)source.n);
      MNT_CHECK(item.out0 != nullptr && (!batched || item.out1 != nullptr), "item %d: null output", index);
      int64_t count = 0;
      must(mnt_target_coordinates(source.coords, source.n, s.ndim, s.coord_dtype, item.stride,
                                  source.batch_dims, s.num_batches, s.index_dtype,
                                  source.bounds_known ? source.bounds : nullptr, item.out0, item.capacity,
                                  item.out1, &count, stream));
      Level &target = s.levels[item.target_level];
      target.coords = item.out0;
      target.n = count;
      target.batch_dims = batched ? item.out1 : nullptr;
      target.known = true;
      if (source.bounds_known) derive_bounds(source, item.stride, s.ndim, target);
      s.size[index] = count;
      break;
    }
    case MNT_AHEAD_DENSE: {
      Level &source = need_level(item.source_level);
      Level &target = need_level(item.target_level);
      MNT_CHECK(item.offsets != nullptr && item.num_offsets > 0 && item.out0 != nullptr,
                "item %d: null operand", index);
      MNT_CHECK(item.capacity >= item.num_offsets * target.n, "item %d: room for %lld map entries, needs %lld",
                index, (long long)item.capacity, (long long)(item.num_offsets * target.n));
      int64_t bounds[16] = {0};
      must(mnt_kernel_map_dense(source.coords, source.n, target.coords, target.n, item.offsets,
                                item.num_offsets, s.ndim, s.coord_dtype, source.batch_dims,
                                target.batch_dims, s.num_batches, s.index_dtype,
                                source.bounds_known ? source.bounds : nullptr,
                                target.bounds_known ? target.bounds : nullptr, bounds,
                                static_cast<int32_t *>(item.out0), stream));
      if (source.n > 0 && target.n > 0) {
        memcpy(source.bounds, bounds, sizeof(source.bounds));
        source.bounds_known = true;
        memcpy(target.bounds, bounds + 8, sizeof(target.bounds));
        target.bounds_known = true;
      }
      s.size[index] = target.n;
      break;
    }
    case MNT_AHEAD_TABLES: {
      const mnt_lookahead_item &dense = need_dense(item.dense_item);
      const int64_t S = s.levels[dense.source_level].n, T = s.levels[dense.target_level].n;
      const int64_t O = dense.num_offsets;
      MNT_CHECK(item.host0 != nullptr && item.host1 != nullptr && item.out0 != nullptr && item.out1 != nullptr,
                "item %d: null output", index);
      must(mnt_kernel_map_tables(static_cast<const int32_t *>(dense.out0), S, T, O, item.reorder, item.host0,
                                 item.host1, stream));
      int64_t pairs = 0;
      for (int64_t o = 0; o < O; ++o) pairs += item.host0[o];
      const bool lists = item.out2 != nullptr && item.out3 != nullptr;
      if (lists && pairs > item.capacity) {
        // the emit half must still run to close the two-phase call; it takes no lists then
        must(mnt_kernel_map_emit(static_cast<int32_t *>(item.out0), static_cast<int32_t *>(item.out1), nullptr,
                                 nullptr, static_cast<int32_t *>(item.out4), static_cast<int32_t *>(item.out5),
                                 stream));
        MNT_FAIL("item %d: room for %lld pairs, the map has %lld", index, (long long)item.capacity,
                 (long long)pairs);
      }
      must(mnt_kernel_map_emit(static_cast<int32_t *>(item.out0), static_cast<int32_t *>(item.out1),
                               lists ? static_cast<int32_t *>(item.out2) : nullptr,
                               lists ? static_cast<int32_t *>(item.out3) : nullptr,
                               static_cast<int32_t *>(item.out4), static_cast<int32_t *>(item.out5), stream));
      s.size[index] = pairs;
      break;
    }
    case MNT_AHEAD_INVERT: {
      const mnt_lookahead_item &dense = need_dense(item.dense_item);
      const int64_t S = s.levels[dense.source_level].n, T = s.levels[dense.target_level].n;
      MNT_CHECK(item.out0 != nullptr && item.capacity >= dense.num_offsets * S,
                "item %d: room for %lld map entries, needs %lld", index, (long long)item.capacity,
                (long long)(dense.num_offsets * S));
      must(mnt_kernel_map_invert(static_cast<const int32_t *>(dense.out0), dense.num_offsets, T, S,
                                 static_cast<int32_t *>(item.out0), stream));
      s.size[index] = S;
      break;
    }
    default:
      MNT_FAIL("item %d has unknown kind %d", index, item.kind);
  }
}

void run_session(Session &s) {
  hipStream_t stream = nullptr;
  bool usable = true;
  std::string setup_error;
  try {
    MNT_HIP(hipSetDevice(s.device));
    if (g_stream[s.device] == nullptr) {
      MNT_HIP(hipStreamCreateWithFlags(&g_stream[s.device], hipStreamNonBlocking));
    }
    stream = g_stream[s.device];
    MNT_HIP(hipStreamWaitEvent(stream, s.inputs_ready, 0));
  } catch (const Error &e) {
    usable = false;
    setup_error = e.message;
  }
  const int count = static_cast<int>(s.items.size());
  for (int i = 0; i < count; ++i) {
    int status = 0;
    std::string message;
    if (!usable) {
      status = 1;
      message = setup_error;
    } else {
      try {
        build_item(s, i, stream);
        MNT_HIP(hipEventRecord(s.built[i], stream));
      } catch (const Error &e) {
        status = 1;
        message = e.message;
      } catch (const std::exception &e) {
        status = 2;
        message = std::string("[Minuet] ") + e.what();
      }
    }
    {
      std::lock_guard<std::mutex> lock(g_mutex);
      s.status[i] = status;
      s.message[i] = message;
    }
    g_progress.notify_all();
  }
  // Whatever the items enqueued, failed ones included, lies before this event:
  // an item that fails half-way records no event of its own, yet its kernels
  // may still be writing the session's buffers.
  if (usable && hipEventRecord(s.session_end, stream) == hipSuccess) {
    std::lock_guard<std::mutex> lock(g_mutex);
    s.end_recorded = true;
  }
  if (s.bounds_out != nullptr && s.bounds_known_out != nullptr) {
    for (size_t l = 0; l < s.levels.size(); ++l) {
      memcpy(s.bounds_out + 8 * l, s.levels[l].bounds, 8 * sizeof(int64_t));
      s.bounds_known_out[l] = s.levels[l].bounds_known ? 1 : 0;
    }
  }
}

void worker_main() {
  for (;;) {
    {
      std::unique_lock<std::mutex> lock(g_mutex);
      g_wake.wait(lock, [] { return g_job_posted; });
      g_job_posted = false;
      g_busy = true;
    }
    run_session(g_session);
    {
      std::lock_guard<std::mutex> lock(g_mutex);
      g_busy = false;
    }
    g_progress.notify_all();
  }
}

}  // namespace
}  // namespace mnt

using namespace mnt;

extern "C" int mnt_lookahead_start(const void *coords, int64_t n, int ndim, int coord_dtype,
                                   const void *batch_dims, int64_t num_batches, int index_dtype,
                                   const int64_t *bounds_host, const mnt_lookahead_item *items,
                                   int num_items, int num_levels, int64_t *bounds_out,
                                   int32_t *bounds_known_out, void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MNT_CHECK(ndim >= 1 && ndim <= MNT_MAX_NDIM, "ndim must be in [1, %d] but found %d", MNT_MAX_NDIM, ndim);
    MNT_CHECK(coords != nullptr && n > 0 && n <= INT32_MAX, "the cloud needs 1 .. 2^31 - 1 rows, found %lld",
              (long long)n);
    MNT_CHECK(items != nullptr && num_items > 0 && num_items <= 4096 && num_levels >= 1 && num_levels <= 64,
              "bad item list (%d items, %d levels)", num_items, num_levels);
    int_size(coord_dtype);
    int_size(index_dtype);
    if (batch_dims == nullptr) num_batches = 1;
    MNT_CHECK(num_batches >= 1, "num_batches must be positive");
    int device = 0;
    MNT_HIP(hipGetDevice(&device));
    MNT_CHECK(device >= 0 && device < 16, "device %d is beyond the 16 the look-ahead keeps a stream for", device);
    std::unique_lock<std::mutex> lock(g_mutex);
    MNT_CHECK(!g_active, "a look-ahead session is running: finish it first");
    Session &s = g_session;
    s.items.assign(items, items + num_items);
    s.levels.assign(num_levels, Level());
    s.levels[0].coords = coords;
    s.levels[0].n = n;
    s.levels[0].batch_dims = batch_dims;
    s.levels[0].known = true;
    if (bounds_host != nullptr) {
      memcpy(s.levels[0].bounds, bounds_host, 8 * sizeof(int64_t));
      s.levels[0].bounds_known = true;
    }
    s.status.assign(num_items, kPending);
    s.size.assign(num_items, 0);
    s.message.assign(num_items, std::string());
    while (static_cast<int>(s.built.size()) < num_items) s.built.push_back(take_event());
    s.ndim = ndim;
    s.coord_dtype = coord_dtype;
    s.index_dtype = index_dtype;
    s.device = device;
    s.num_batches = num_batches;
    s.bounds_out = bounds_out;
    s.bounds_known_out = bounds_known_out;
    if (s.inputs_ready == nullptr) s.inputs_ready = take_event();
    if (s.session_end == nullptr) s.session_end = take_event();
    s.end_recorded = false;
    MNT_HIP(hipEventRecord(s.inputs_ready, stream));
    if (!g_worker_started) {
      std::thread(worker_main).detach();
      g_worker_started = true;
    }
    g_active = true;
    g_job_posted = true;
    lock.unlock();
    g_wake.notify_one();
  });
}

extern "C" int mnt_lookahead_wait(int item, void *stream_, int64_t *size_out) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    std::unique_lock<std::mutex> lock(g_mutex);
    MNT_CHECK(g_active, "no look-ahead session is running");
    Session &s = g_session;
    MNT_CHECK(item >= 0 && item < static_cast<int>(s.items.size()), "item %d of %d", item,
              static_cast<int>(s.items.size()));
    g_progress.wait(lock, [&] { return s.status[item] != kPending; });
    if (s.status[item] != 0) throw Error{s.message[item]};
    if (size_out != nullptr) *size_out = s.size[item];
    hipEvent_t built = s.built[item];
    lock.unlock();
    MNT_HIP(hipStreamWaitEvent(stream, built, 0));
  });
}

extern "C" int mnt_lookahead_finish(void *stream_) {
  return guarded([&] {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    std::unique_lock<std::mutex> lock(g_mutex);
    if (!g_active) return;
    g_progress.wait(lock, [] { return !g_job_posted && !g_busy; });
    Session &s = g_session;
    // the caller's stream waits for everything the worker enqueued, the
    // kernels of items that failed after their first launch included
    hipEvent_t last = s.end_recorded ? s.session_end : nullptr;
    g_active = false;
    lock.unlock();
    if (last != nullptr) MNT_HIP(hipStreamWaitEvent(stream, last, 0));
  });
}
