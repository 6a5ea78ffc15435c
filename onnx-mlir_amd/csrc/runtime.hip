// C-ABI runtime of the MI355X accelerator for onnx-mlir's int8 path:
// accelerator life cycle, OMTensor marshalling, GPU residency and the op
// entry points declared in include/om_mi355x.h.
//
// An entry point receives OMTensor wrappers exactly as KrnlCallOpLowering
// builds them (src/Conversion/KrnlToLLVM/KrnlCall.cpp:34-102).  A tensor whose
// data pointer is GPU memory is used in place; a host tensor is staged into a
// per-thread pool of GPU buffers (inputs copied in before the kernels, outputs
// copied back after them, one stream synchronisation per call).  Host buffers
// declared constant are uploaded once; a constant matmul right-hand side is
// also packed and column-summed once.
//
// There is no CPU implementation behind these entry points: without a gfx950
// device they fail (errno, stderr, om_mi355x_last_error).

#include <errno.h>
#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <time.h>

#include <algorithm>
#include <condition_variable>
#include <functional>
#include <map>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "om_kernels.h"
#include "om_mi355x.h"

using namespace om;

// ---------------------------------------------------------------------------
// Scratch of om_mi355x_DynamicQuantizeLinearNoAlloc, the entry point that
// allocates nothing: the per-block partial minima / maxima, the arrival
// counter and the tagged slots that DynamicQuantizeLinear's kernels exchange
// their results through live in this array instead of in memory from
// hipMalloc.  Every GPU the library runs on holds its own copy until the
// process ends.  The name below is only a host-side handle: the address a
// kernel or a memory operation needs comes from hipGetSymbolAddress, once per
// device (resolve_scratch), and only that address is ever used.
// Layout: f32 partial_min[kNoAllocBlocks], f32 partial_max[kNoAllocBlocks],
// 64 counter words ([0] arrivals of the two-launch path, [8] "the one-launch
// kernel gave up" flag), u64 slots[2 * kNoAllocBlocks].
// ---------------------------------------------------------------------------
constexpr int kNoAllocBlocks = 512;
constexpr size_t kNoAllocScratchBytes =
    sizeof(float) * 2 * kNoAllocBlocks + 256 +
    sizeof(unsigned long long) * 2 * kNoAllocBlocks; // 12,544 bytes
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// ---------------------------------------------------------------------------
// errors
// ---------------------------------------------------------------------------
namespace {

// The compiler options that change this path's arithmetic (OM_MI355X_QUANT_*).
// In the reference they are a property of each compiled model
// (src/Compiler/CompilerPasses.cpp:298-301), so here they are a property of
// each op: om_mi355x_SetQuantMode leaves its mode in t_quant_mode_next, the
// next QuantizeLinear / DequantizeLinear / DynamicQuantizeLinear / fused-layer
// entry point of the thread takes it (QuantModeScope) and leaves 0 behind.  An
// op that no SetQuantMode call precedes therefore always computes the default
// form, whatever ran on the thread before it.
thread_local int t_quant_mode_next = 0;
// Mode of the entry point that is running on this thread; 0 outside one.
thread_local int t_quant_mode = 0;
struct QuantModeScope {
  QuantModeScope() {
    t_quant_mode = t_quant_mode_next;
    t_quant_mode_next = 0;
  }
  ~QuantModeScope() { t_quant_mode = 0; }
};
thread_local std::string t_last_error;
thread_local std::string t_last_error_returned;

void fail(int err, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  t_last_error = buf;
  fprintf(stderr, "om_mi355x: %s\n", buf);
  errno = err;
}

#define HIP_OK(expr)                                                           \
  do {                                                                         \
    hipError_t e_ = (expr);                                                    \
    if (e_ != hipSuccess) {                                                    \
      fail(EIO, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_),        \
          __FILE__, __LINE__);                                                 \
      return false;                                                            \
    }                                                                          \
  } while (0)

// ---------------------------------------------------------------------------
// device state
// ---------------------------------------------------------------------------
pthread_mutex_t g_init_mutex = PTHREAD_MUTEX_INITIALIZER;
bool g_device_ok = false;
std::string g_device_why;

std::mutex g_mem_mutex;
// GPU allocations handed out by om_mi355x_malloc: start -> bytes.
std::map<uintptr_t, size_t> g_user_allocs;
// Host buffers declared constant, and their GPU copies.
std::unordered_set<const void *> g_constants;
struct DevCopy {
  void *dev;
  size_t bytes;
};
std::unordered_map<const void *, DevCopy> g_const_copies;
// Zero points in GPU memory that were declared constant and have been read
// back once: (bytes, whether every one of them is zero).
std::unordered_map<const void *, std::pair<size_t, bool>> g_const_zero;
// Packed right-hand sides of constant B, keyed by B's data pointer.
struct PackedB {
  int8_t *bp;
  int32_t *colsum;
  int64_t K, N;
  bool is_unsigned;
};
std::unordered_map<const void *, PackedB> g_packed;
// GPU blocks that left a cache while work on some stream may still read them
// (a constant re-declared with another shape); freed by om_mi355x_ClearCache
// after the device has drained.
std::vector<void *> g_retired;

// Host buffers backed by GPU memory (om_mi355x_KeepOnDevice): start address ->
// (GPU copy, bytes).  Guarded by g_mem_mutex.
struct Backing {
  void *dev;
  size_t bytes;    // size of the host buffer
  size_t capacity; // size of the GPU block (what the pool files it under)
  hipStream_t stream; // stream of the thread that declared it
};
std::map<uintptr_t, Backing> g_backed;

// Device address of `scratch` on each GPU, resolved with that GPU current
// (each GPU has its own copy of the array at its own address), and the
// host-side state that goes with it.  Guarded by g_scratch_mutex.
constexpr int kMaxDevices = 16;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};
unsigned g_scratch_epoch[kMaxDevices] = {};   // launch number of k_dql_grid
bool g_scratch_no_grid[kMaxDevices] = {};     // one-launch kernel switched off
bool g_scratch_used[kMaxDevices] = {};
bool g_scratch_unchecked[kMaxDevices] = {}; // launched since its flag was last fetched
std::thread::id g_scratch_launcher[kMaxDevices]; // by this thread: the one whose synchronisation fetches it

// Call with device `dev` current.
bool resolve_scratch(int dev) {
  if (dev < 0 || dev >= kMaxDevices)
    return false;
  std::lock_guard<std::mutex> lk(g_scratch_mutex);
  if (g_scratch_ptr[dev])
    return true;
  void *p = nullptr;
  const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !p) {
    (void)hipGetLastError();
    return false;
  }
  g_scratch_ptr[dev] = p;
  return true;
}

bool probe_device() {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count < 1) {
    (void)hipGetLastError();
    g_device_why = "no HIP device visible";
    return false;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) {
    (void)hipGetLastError();
    g_device_why = "hipGetDeviceProperties failed";
    return false;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    g_device_why = std::string("device 0 is ") + prop.gcnArchName +
                   ", the kernels are built for gfx950 only";
    return false;
  }
  if (hipSetDevice(0) != hipSuccess) {
    (void)hipGetLastError();
    g_device_why = "hipSetDevice(0) failed";
    return false;
  }
  if (!resolve_scratch(0)) {
    g_device_why = "hipGetSymbolAddress(scratch) failed";
    return false;
  }
  return true;
}

// ---------------------------------------------------------------------------
// Large copies between pageable host memory and the GPU
// ---------------------------------------------------------------------------
// A direct hipMemcpy on pageable memory reaches a third of the link rate.  A
// lane moves every step-th piece of a buffer through page-locked slots of its
// own: the DMA of one piece runs while the CPU copies the neighbouring piece
// between its slot and the host buffer.  One core copies about 34 GB/s and the
// link carries 56 GB/s, so the calling thread's lane is joined by lanes run by
// helper threads (OM_MI355X_COPY_THREADS, default 2, 0 = none).
struct CopyLane {
  static constexpr int kSlots = 3;
  static constexpr size_t kSlotBytes = (size_t)4 << 20;
  hipStream_t stream = nullptr;
  void *slot[kSlots] = {nullptr, nullptr, nullptr};
  hipEvent_t ev[kSlots] = {nullptr, nullptr, nullptr};
  hipEvent_t done = nullptr; // end of this lane's last to_device()
  bool ready = false;

  // `borrowed`: the stream to issue on; null = a stream of the lane's own.
  bool init(hipStream_t borrowed) {
    if (ready)
      return true;
    void *p = nullptr;
    if (hipHostMalloc(&p, kSlots * kSlotBytes, hipHostMallocDefault) !=
        hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    bool good = true;
    for (int i = 0; i < kSlots && good; ++i)
      good = hipEventCreateWithFlags(&ev[i], hipEventDisableTiming) ==
             hipSuccess;
    good = good && hipEventCreateWithFlags(&done, hipEventDisableTiming) ==
                       hipSuccess;
    if (good && !borrowed)
      good = hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) ==
             hipSuccess;
    else
      stream = borrowed;
    if (!good) {
      (void)hipGetLastError();
      for (int i = 0; i < kSlots; ++i)
        if (ev[i]) {
          (void)hipEventDestroy(ev[i]);
          ev[i] = nullptr;
        }
      if (done) {
        (void)hipEventDestroy(done);
        done = nullptr;
      }
      (void)hipHostFree(p);
      return false;
    }
    for (int i = 0; i < kSlots; ++i)
      slot[i] = (char *)p + (size_t)i * kSlotBytes;
    ready = true;
    return true;
  }

  // Pieces first, first+step, ... of `bytes` (piece <= kSlotBytes each), from
  // GPU memory into host memory.  Queued on the lane's stream; returns when
  // this lane's share of the host buffer is complete.
  hipError_t to_host(char *host, const char *dev, size_t bytes, size_t piece,
      size_t first, size_t step) {
    const size_t n = (bytes + piece - 1) / piece;
    const size_t mine = first < n ? (n - first + step - 1) / step : 0;
    auto offset = [&](size_t k) { return (first + k * step) * piece; };
    auto length = [&](size_t k) {
      return offset(k) + piece <= bytes ? piece : bytes - offset(k);
    };
    auto drain = [&](size_t k) -> hipError_t {
      hipError_t e = hipEventSynchronize(ev[k % kSlots]);
      if (e == hipSuccess)
        memcpy(host + offset(k), slot[k % kSlots], length(k));
      return e;
    };
    for (size_t k = 0; k < mine; ++k) {
      const int sl = (int)(k % kSlots);
      hipError_t e = hipMemcpyAsync(slot[sl], dev + offset(k), length(k),
          hipMemcpyDeviceToHost, stream);
      if (e == hipSuccess)
        e = hipEventRecord(ev[sl], stream);
      if (e == hipSuccess && k + 1 >= (size_t)kSlots)
        e = drain(k + 1 - kSlots);
      if (e != hipSuccess)
        return e;
    }
    for (size_t k = (mine >= (size_t)kSlots ? mine - kSlots + 1 : 0); k < mine;
         ++k) {
      hipError_t e = drain(k);
      if (e != hipSuccess)
        return e;
    }
    return hipSuccess;
  }

  // The same pieces from host memory into GPU memory.  Returns when the host
  // buffer has been read; the DMAs are queued on the lane's stream and `done`
  // is recorded behind the last of them.
  hipError_t to_device(char *dev, const char *host, size_t bytes, size_t piece,
      size_t first, size_t step) {
    const size_t n = (bytes + piece - 1) / piece;
    for (size_t k = 0, i = first; i < n; ++k, i += step) {
      const int sl = (int)(k % kSlots);
      const size_t off = i * piece;
      const size_t len = off + piece <= bytes ? piece : bytes - off;
      // The slot may still feed an earlier DMA (an event that was never
      // recorded counts as complete).
      hipError_t e = hipEventSynchronize(ev[sl]);
      if (e != hipSuccess)
        return e;
      memcpy(slot[sl], host + off, len);
      e = hipMemcpyAsync(dev + off, slot[sl], len, hipMemcpyHostToDevice,
          stream);
      if (e == hipSuccess)
        e = hipEventRecord(ev[sl], stream);
      if (e != hipSuccess)
        return e;
    }
    return hipEventRecord(done, stream);
  }
};

// A helper thread with a lane of its own.  Helpers are created once, never
// destroyed (they sleep on their condition variable until the process ends)
// and serve one calling thread at a time.
struct CopyHelper {
  std::mutex m;
  std::condition_variable cv;
  std::function<hipError_t(CopyLane &)> job;
  bool pending = false, finished = true;
  hipError_t result = hipSuccess;
  CopyLane lane;

  void loop() {
    (void)hipSetDevice(0);
    std::unique_lock<std::mutex> lk(m);
    for (;;) {
      cv.wait(lk, [&] { return pending; });
      pending = false;
      std::function<hipError_t(CopyLane &)> j = std::move(job);
      lk.unlock();
      hipError_t e = lane.init(nullptr) ? j(lane) : hipErrorOutOfMemory;
      lk.lock();
      result = e;
      finished = true;
      cv.notify_all();
    }
  }
  void start(std::function<hipError_t(CopyLane &)> j) {
    std::lock_guard<std::mutex> lk(m);
    job = std::move(j);
    pending = true;
    finished = false;
    cv.notify_all();
  }
  hipError_t wait() {
    std::unique_lock<std::mutex> lk(m);
    cv.wait(lk, [&] { return finished; });
    return result;
  }
};

struct CopyHelpers {
  std::mutex in_use; // held by the calling thread that employs the helpers
  std::vector<CopyHelper *> list;
};

CopyHelpers *copy_helpers() {
  static CopyHelpers *set = [] {
    CopyHelpers *s = new CopyHelpers; // lives until the process ends
    long want = 2;
    if (const char *v = getenv("OM_MI355X_COPY_THREADS"))
      want = strtol(v, nullptr, 10);
    for (long i = 0; i < want && i < 4; ++i) {
      CopyHelper *h = new CopyHelper;
      try {
        std::thread(&CopyHelper::loop, h).detach();
      } catch (...) {
        delete h;
        break;
      }
      s->list.push_back(h);
    }
    return s;
  }();
  return set;
}

// Per-thread execution context: one stream (default priority), the scratch of
// DynamicQuantizeLinear, a pool of reusable GPU buffers and timer events.
// Buffers of the pool are only ever used by work on this stream, so handing a
// buffer to the next call without waiting is safe: stream order serialises
// the uses.
struct Ctx {
  bool ready = false;
  hipStream_t stream = nullptr;
  DqlScratch dql = {nullptr, nullptr, nullptr, 0, 0, nullptr, 0, kDqlMaxBlocks};
  float *dql_scale = nullptr; // scale / zero point of the fused path
  uint8_t *dql_zp = nullptr;
  std::multimap<size_t, void *> pool;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  // Large copies from and to pageable host memory (see CopyLane).
  // Below these sizes a plain copy is faster (measured: 4 MiB in 0.22 ms
  // plain against 0.25 ms in pieces, 4 MiB out 0.33 against 0.26 ms).
  static constexpr size_t kStagedIn = (size_t)8 << 20;
  static constexpr size_t kStagedOut = (size_t)4 << 20;
  CopyLane lane;             // the calling thread's lane, on `stream`
  hipEvent_t fork_ev = nullptr; // where the helpers' streams join `stream`

  bool init() {
    if (ready)
      return true;
    OMInitAccelMI355X();
    if (!g_device_ok) {
      fail(EIO, "accelerator unavailable: %s", g_device_why.c_str());
      return false;
    }
    HIP_OK(hipSetDevice(0));
    HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    void *p = nullptr;
    HIP_OK(hipMalloc(&p, sizeof(float) * 2 * kDqlMaxBlocks + 256 +
                             sizeof(unsigned long long) * 2 * kDqlMaxBlocks));
    dql.partial_min = (float *)p;
    dql.partial_max = dql.partial_min + kDqlMaxBlocks;
    dql.counter = (unsigned *)(dql.partial_max + kDqlMaxBlocks);
    dql_scale = (float *)(dql.counter + 16);
    dql_zp = (uint8_t *)(dql.counter + 32);
    dql.grid_slots = (unsigned long long *)((char *)dql.counter + 256);
    HIP_OK(hipMemset(dql.counter, 0,
        256 + sizeof(unsigned long long) * 2 * kDqlMaxBlocks));
    dql.max_blocks = kDqlMaxBlocks;
    dql.grid_blocks = dql_grid_blocks();
    dql.spin_limit = 1u << 20; // about a second of polling
    if (const char *v = getenv("OM_MI355X_DQL_SPIN_LIMIT"))
      dql.spin_limit = (unsigned)strtoul(v, nullptr, 10);
    HIP_OK(hipEventCreate(&ev0));
    HIP_OK(hipEventCreate(&ev1));
    ready = true;
    return true;
  }

  // Call after the stream has been synchronised.  The one-launch
  // DynamicQuantizeLinear kernel raises a flag if its grid barrier ever timed
  // out (its output is then missing); report that and stop using the kernel.
  // Whether a one-launch kernel of this thread gave up since the last check
  // (call after the stream has been synchronised).  If so the flag is
  // cleared and the one-launch kernel is not used again by this thread.
  // Whether the one-launch kernel raised its flag since the last look.  The
  // flag is only fetched (a blocking 4-byte copy, tens of microseconds) when
  // such a kernel has been launched since.
  bool dql_unchecked = false;
  bool dql_gave_up() {
    if (!ready || dql.grid_blocks == 0 || !dql_unchecked)
      return false;
    dql_unchecked = false;
    unsigned flag = 0;
    if (hipMemcpy(&flag, dql.counter + 8, sizeof(flag),
            hipMemcpyDeviceToHost) != hipSuccess)
      return false;
    if (!flag)
      return false;
    (void)hipMemset(dql.counter, 0, 256);
    dql.grid_blocks = 0;
    return true;
  }
  bool dql_barrier_ok() {
    if (!dql_gave_up())
      return true;
    fail(EIO, "DynamicQuantizeLinear: the blocks of the one-launch kernel "
              "timed out waiting for one another (grid barrier); its output "
              "was not written");
    return false;
  }

  bool stage_ready() {
    if (!fork_ev && hipEventCreateWithFlags(&fork_ev, hipEventDisableTiming) !=
                        hipSuccess) {
      (void)hipGetLastError();
      fork_ev = nullptr;
      return false;
    }
    return lane.init(stream);
  }

  // One large buffer (kStagedIn / kStagedOut) between pageable host memory and
  // GPU memory, split into pieces that go round-robin to this thread's lane
  // and to the helpers (if no other thread employs them).  In stream order
  // with the work queued on `stream` before and after; returns when the host
  // buffer is complete (to_host) or has been read (to_device).
  hipError_t copy_staged(void *host, void *dev, size_t bytes, bool to_host) {
    // Measured on 2 ... 1024 MiB: 1 MiB pieces are best up to 16 MiB (more
    // pieces than lanes, so that DMA and CPU copies overlap), 2 MiB beyond.
    const size_t piece = bytes < ((size_t)16 << 20)    ? (size_t)1 << 20
                         : bytes < ((size_t)256 << 20) ? (size_t)2 << 20
                                                       : CopyLane::kSlotBytes;
    const size_t n = (bytes + piece - 1) / piece;
    CopyHelpers *hs = copy_helpers();
    std::unique_lock<std::mutex> use(hs->in_use, std::try_to_lock);
    size_t nh = 0;
    if (use.owns_lock() && n >= 2)
      nh = std::min(hs->list.size(), n - 1);
    const size_t lanes = 1 + nh;
    hipError_t e = hipSuccess;
    if (nh) {
      e = hipEventRecord(fork_ev, stream);
      if (e != hipSuccess)
        return e;
    }
    char *h = (char *)host, *d = (char *)dev;
    hipEvent_t fork = fork_ev;
    for (size_t i = 0; i < nh; ++i)
      hs->list[i]->start([=](CopyLane &l) -> hipError_t {
        // Behind everything the calling thread has queued so far (the
        // kernels that write the data, or the last use of the GPU buffer).
        hipError_t r = hipStreamWaitEvent(l.stream, fork, 0);
        if (r != hipSuccess)
          return r;
        return to_host ? l.to_host(h, d, bytes, piece, i + 1, lanes)
                       : l.to_device(d, h, bytes, piece, i + 1, lanes);
      });
    e = to_host ? lane.to_host(h, d, bytes, piece, 0, lanes)
                : lane.to_device(d, h, bytes, piece, 0, lanes);
    for (size_t i = 0; i < nh; ++i) {
      hipError_t r = hs->list[i]->wait();
      if (r == hipSuccess && !to_host)
        r = hipStreamWaitEvent(stream, hs->list[i]->lane.done, 0);
      if (e == hipSuccess)
        e = r;
    }
    return e;
  }

  void *take(size_t bytes) {
    if (bytes == 0)
      bytes = 16;
    bytes = (bytes + 255) & ~(size_t)255;
    auto it = pool.lower_bound(bytes);
    if (it != pool.end() && it->first <= bytes * 2) {
      void *p = it->second;
      taken[p] = it->first;
      pool_bytes -= it->first;
      pool.erase(it);
      return p;
    }
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) {
      // Give cached buffers back to the driver and retry once.
      for (auto &kv : pool)
        (void)hipFree(kv.second);
      pool.clear();
      pool_bytes = 0;
      e = hipMalloc(&p, bytes);
    }
    if (e != hipSuccess) {
      fail(EIO, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
      return nullptr;
    }
    taken[p] = bytes;
    return p;
  }
  void give(void *p) {
    auto it = taken.find(p);
    if (it == taken.end())
      return;
    adopt(p, it->second);
    taken.erase(it);
  }
  // A pool block whose ownership leaves the pool (a backing that outlives the
  // call); adopt() files such a block back.
  void *take_owned(size_t bytes, size_t *capacity) {
    void *p = take(bytes);
    if (!p)
      return nullptr;
    auto it = taken.find(p);
    *capacity = it->second;
    taken.erase(it);
    return p;
  }
  // Idle blocks are kept for reuse up to kPoolCap bytes per host thread; past
  // that (shapes that keep changing) a block goes back to the driver, after
  // the work that may still use it.
  static constexpr size_t kPoolCap = (size_t)16 << 30;
  size_t pool_bytes = 0;
  void adopt(void *p, size_t capacity) {
    if (pool_bytes + capacity > kPoolCap) {
      (void)hipStreamSynchronize(stream);
      (void)hipFree(p);
      return;
    }
    pool.emplace(capacity, p);
    pool_bytes += capacity;
  }
  void drop_pool() {
    for (auto &kv : pool)
      (void)hipFree(kv.second);
    pool.clear();
    pool_bytes = 0;
  }
  std::unordered_map<void *, size_t> taken;

  // A context lives as long as its host thread.  When the thread ends, what
  // it holds on the GPU goes back to the driver: the idle pool blocks, the
  // scratch, the page-locked copy slots, the events and the stream (after the
  // work queued on it).  Buffers handed out by om_mi355x_malloc and backings
  // declared with om_mi355x_KeepOnDevice are not the thread's and stay.
  ~Ctx() {
    if (!ready)
      return;
    ready = false;
    (void)hipStreamSynchronize(stream);
    {
      // Backings declared by this thread no longer have a stream to wait for.
      std::lock_guard<std::mutex> lk(g_mem_mutex);
      for (auto &kv : g_backed)
        if (kv.second.stream == stream)
          kv.second.stream = nullptr;
    }
    dql_forget_stream(stream);
    drop_pool();
    for (auto &kv : taken)
      (void)hipFree(kv.first);
    taken.clear();
    if (dql.partial_min)
      (void)hipFree(dql.partial_min);
    if (lane.ready) {
      (void)hipHostFree(lane.slot[0]);
      for (int i = 0; i < CopyLane::kSlots; ++i)
        (void)hipEventDestroy(lane.ev[i]);
      (void)hipEventDestroy(lane.done);
    }
    if (fork_ev)
      (void)hipEventDestroy(fork_ev);
    if (ev0)
      (void)hipEventDestroy(ev0);
    if (ev1)
      (void)hipEventDestroy(ev1);
    (void)hipStreamDestroy(stream);
    (void)hipGetLastError();
  }
};

thread_local Ctx t_ctx;

// GPU address that stands for host address p, if p lies in a buffer declared
// with om_mi355x_KeepOnDevice; null otherwise.
void *backed_lookup(const void *p) {
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  if (g_backed.empty())
    return nullptr;
  auto it = g_backed.upper_bound((uintptr_t)p);
  if (it == g_backed.begin())
    return nullptr;
  --it;
  const uintptr_t off = (uintptr_t)p - it->first;
  if (off >= it->second.bytes)
    return nullptr;
  return (char *)it->second.dev + off;
}

bool is_device_ptr(const void *p) {
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    auto it = g_user_allocs.upper_bound((uintptr_t)p);
    if (it != g_user_allocs.begin()) {
      --it;
      if ((uintptr_t)p < it->first + it->second)
        return true;
    }
  }
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return attr.type == hipMemoryTypeDevice;
}

// ---------------------------------------------------------------------------
// tensor views
// ---------------------------------------------------------------------------
struct View {
  void *data = nullptr;
  int dtype = 0;
  int64_t rank = 0;
  const int64_t *shape = nullptr;
  int64_t numel = 0;
  size_t bytes = 0;
};

size_t dtype_bytes(int dt) {
  switch (dt) {
  case OM_MI355X_TYPE_FLOAT:
  case OM_MI355X_TYPE_INT32:
    return 4;
  case OM_MI355X_TYPE_UINT8:
  case OM_MI355X_TYPE_INT8:
    return 1;
  default:
    return 0;
  }
}

bool view_of(const OMTensor *t, const char *name, View &v) {
  if (!t) {
    fail(EINVAL, "%s: tensor is NULL", name);
    return false;
  }
  v.data = omTensorGetDataPtr(t);
  v.dtype = omTensorGetDataType(t);
  v.rank = omTensorGetRank(t);
  v.shape = omTensorGetShape(t);
  const int64_t *strides = omTensorGetStrides(t);
  v.numel = 1;
  if (v.rank < 0 || (v.rank > 0 && (!v.shape || !strides))) {
    fail(EINVAL, "%s: tensor has no shape", name);
    return false;
  }
  for (int64_t i = 0; i < v.rank; ++i) {
    // a dimension that was never resolved (-1) or a product beyond 2^62
    if (v.shape[i] < 0 ||
        (v.shape[i] > 0 && v.numel > ((int64_t)1 << 62) / v.shape[i])) {
      fail(EINVAL, "%s: dimension %lld is %lld", name, (long long)i,
          (long long)v.shape[i]);
      return false;
    }
    v.numel *= v.shape[i];
  }
  // Row-major contiguous is what memref.alloc and the entry-point wrapper
  // produce (src/Runtime/OMTensor.inc:185-192); anything else is refused.
  int64_t expect = 1;
  for (int64_t i = v.rank - 1; i >= 0; --i) {
    if (v.shape[i] != 1 && strides[i] != expect) {
      fail(EINVAL, "%s: tensor is not row-major contiguous", name);
      return false;
    }
    expect *= v.shape[i];
  }
  if (dtype_bytes(v.dtype) == 0) {
    fail(EINVAL, "%s: unsupported element type %d", name, v.dtype);
    return false;
  }
  v.bytes = (size_t)v.numel * dtype_bytes(v.dtype);
  if (v.numel > 0 && !v.data) {
    fail(EINVAL, "%s: data pointer is NULL", name);
    return false;
  }
  return true;
}

// One entry-point invocation: resolves tensors to GPU pointers, remembers
// which host outputs need copying back and which pool buffers to return.
// ---------------------------------------------------------------------------
// Timing support.  Entry points normally return as soon as their kernels are
// queued when all tensors live on the GPU.  Two environment variables change
// that, for measurements:
//   OM_MI355X_SYNC=1         every entry point waits for its kernels, so that
//                            the before / after instrumentation points the
//                            compiler puts around each ONNX op
//                            (src/Runtime/OMInstrument.c:156-170) bracket the
//                            op's real duration;
//   OM_MI355X_PERF_REPORT=1  the same, and the runtime prints its own lines in
//                            that format, "==PERF-REPORT==, <op>, <entry
//                            point>, before|after, <seconds since the last
//                            line>, <seconds since the first line>", to the
//                            file named by ONNX_MLIR_INSTRUMENT_FILE or to
//                            stdout (as OMInstrument.c:290-300 does).
bool env_flag(const char *name) {
  const char *v = getenv(name);
  return v && v[0] && v[0] != '0';
}
bool sync_every_call() {
  static const bool on = env_flag("OM_MI355X_SYNC");
  return on;
}
bool report_enabled() {
  static const bool on = env_flag("OM_MI355X_PERF_REPORT");
  return on;
}
double now_seconds() {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
void report_line(const char *op, const char *when, double t) {
  static std::mutex m;
  static FILE *out = nullptr;
  static double t_first = 0.0, t_last = 0.0;
  std::lock_guard<std::mutex> lk(m);
  if (!out) {
    const char *name = getenv("ONNX_MLIR_INSTRUMENT_FILE");
    out = (name && name[0]) ? fopen(name, "w") : nullptr;
    if (!out)
      out = stdout;
    t_first = t_last = t;
  }
  fprintf(out, "==PERF-REPORT==, onnx.%s, om_mi355x_%s, %s, %.6f, %.6f\n", op, op,
      when, t - t_last, t - t_first);
  fflush(out);
  t_last = t;
}

struct Call {
  Ctx &c;
  bool ok = true;
  bool touched_host = false;
  bool used_dql = false; // launched DynamicQuantizeLinear (see dql_barrier_ok)
  struct Back {
    void *host;
    void *dev;
    size_t bytes;
  };
  std::vector<Back> backs;
  std::vector<void *> temps;

  const char *op;
  double t_begin = 0.0;

  Call(Ctx &ctx, const char *op_name) : c(ctx), op(op_name) {
    ok = c.init();
    if (ok && report_enabled()) {
      t_begin = now_seconds();
      report_line(op, "before", t_begin);
    }
  }

  void *temp(size_t bytes) {
    void *p = c.take(bytes);
    if (!p)
      ok = false;
    else
      temps.push_back(p);
    return p;
  }

  // keep_constant: a host buffer declared constant gets a GPU copy that stays
  // (false: it is staged like any other host tensor, for this call only).
  const void *in(const View &v, bool keep_constant = true) {
    if (!ok || v.numel == 0)
      return v.data;
    if (void *d = backed_lookup(v.data))
      return d;
    if (is_device_ptr(v.data))
      return v.data;
    bool constant = false;
    if (keep_constant) {
      std::lock_guard<std::mutex> lk(g_mem_mutex);
      constant = g_constants.count(v.data) != 0;
      if (constant) {
        auto it = g_const_copies.find(v.data);
        if (it != g_const_copies.end() && it->second.bytes == v.bytes)
          return it->second.dev;
      }
    }
    void *d = nullptr;
    if (constant) {
      if (hipMalloc(&d, v.bytes ? v.bytes : 16) != hipSuccess) {
        fail(EIO, "hipMalloc(%zu) for a constant failed", v.bytes);
        ok = false;
        return nullptr;
      }
      if (hipMemcpy(d, v.data, v.bytes, hipMemcpyHostToDevice) != hipSuccess) {
        fail(EIO, "upload of a constant failed");
        ok = false;
        return nullptr;
      }
      std::lock_guard<std::mutex> lk(g_mem_mutex);
      auto ins = g_const_copies.emplace(v.data, DevCopy{d, v.bytes});
      if (!ins.second) { // another thread won, or the size changed
        if (ins.first->second.bytes == v.bytes) {
          (void)hipFree(d);
          return ins.first->second.dev;
        }
        g_retired.push_back(ins.first->second.dev); // may still be in use
        ins.first->second = DevCopy{d, v.bytes};
      }
      return d;
    }
    d = temp(v.bytes);
    if (!d)
      return nullptr;
    hipError_t e;
    if (v.bytes >= Ctx::kStagedIn && c.stage_ready())
      e = c.copy_staged(v.data, d, v.bytes, false);
    else
      e = hipMemcpyAsync(d, v.data, v.bytes, hipMemcpyHostToDevice, c.stream);
    if (e != hipSuccess) {
      fail(EIO, "host-to-device copy failed: %s", hipGetErrorString(e));
      ok = false;
      return nullptr;
    }
    touched_host = true;
    return d;
  }

  void *out(const View &v) {
    if (!ok || v.numel == 0)
      return v.data;
    if (void *d = backed_lookup(v.data))
      return d;
    if (is_device_ptr(v.data))
      return v.data;
    void *d = temp(v.bytes);
    if (!d)
      return nullptr;
    backs.push_back(Back{v.data, d, v.bytes});
    touched_host = true;
    return d;
  }

  void check(hipError_t e, const char *what) {
    if (e != hipSuccess) {
      fail(EIO, "%s failed: %s", what, hipGetErrorString(e));
      ok = false;
    }
  }

  void finish() {
    if (ok) {
      for (const Back &b : backs) {
        hipError_t e;
        if (b.bytes >= Ctx::kStagedOut && c.stage_ready())
          e = c.copy_staged(b.host, b.dev, b.bytes, true);
        else
          e = hipMemcpyAsync(
              b.host, b.dev, b.bytes, hipMemcpyDeviceToHost, c.stream);
        if (e != hipSuccess) {
          fail(EIO, "device-to-host copy failed: %s", hipGetErrorString(e));
          ok = false;
          break;
        }
      }
    }
    if ((touched_host || sync_every_call() || report_enabled()) && c.ready) {
      hipError_t e = hipStreamSynchronize(c.stream);
      if (e != hipSuccess && ok)
        fail(EIO, "stream synchronisation failed: %s", hipGetErrorString(e));
      else if (used_dql && !c.dql_barrier_ok())
        ok = false;
    }
    for (void *p : temps)
      c.give(p);
    temps.clear();
    if (report_enabled() && c.ready)
      report_line(op, "after", now_seconds());
  }
};

bool is_q8(int dt) {
  return dt == OM_MI355X_TYPE_UINT8 || dt == OM_MI355X_TYPE_INT8;
}

// DynamicQuantizeLinear on GPU pointers, as part of `call`.  When the call is
// going to wait for its kernels anyway (a host tensor is involved, or one of
// the timing modes is on), the wait happens here, and if the blocks of the
// one-launch kernel gave up waiting for one another the two-launch path runs
// right away: the outputs are correct when the entry point returns.  A call
// on GPU tensors only returns without waiting; there a give-up is reported
// (EIO) at the thread's next synchronisation.
void run_dql(Call &call, const float *dx, int64_t n, uint8_t *dy, float *ds,
    uint8_t *dz, bool y_shift) {
  Ctx &c = call.c;
  const int mode = t_quant_mode;
  if (mode != 0) { // never the one-launch kernel: nothing to check afterwards
    call.check(launch_dynamic_quantize(
                   c.stream, c.dql, dx, n, dy, ds, dz, y_shift, mode),
        "DynamicQuantizeLinear");
    return;
  }
  c.dql_unchecked = c.dql.grid_blocks != 0;
  call.check(
      launch_dynamic_quantize(c.stream, c.dql, dx, n, dy, ds, dz, y_shift),
      "DynamicQuantizeLinear");
  if (!call.ok || c.dql.grid_blocks == 0)
    return;
  if (!(call.touched_host || sync_every_call() || report_enabled())) {
    call.used_dql = true;
    return;
  }
  const hipError_t e = hipStreamSynchronize(c.stream);
  if (e != hipSuccess) {
    call.check(e, "stream synchronisation");
    return;
  }
  if (c.dql_gave_up()) { // grid_blocks is 0 from here on: two launches
    fprintf(stderr,
        "om_mi355x: DynamicQuantizeLinear: the blocks of the one-launch "
        "kernel timed out waiting for one another; redone with two launches, "
        "which this thread uses from now on\n");
    call.check(
        launch_dynamic_quantize(c.stream, c.dql, dx, n, dy, ds, dz, y_shift),
        "DynamicQuantizeLinear (two launches)");
  }
}

// The "gave up" flag of the static scratch on device `dev`, after a
// synchronisation; reports and clears it.
bool noalloc_barrier_ok() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return true;
  void *sp;
  {
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    if (!g_scratch_used[dev] || g_scratch_no_grid[dev] ||
        !g_scratch_unchecked[dev] ||
        g_scratch_launcher[dev] != std::this_thread::get_id())
      return true;
    g_scratch_unchecked[dev] = false;
    sp = g_scratch_ptr[dev];
  }
  unsigned *counter = (unsigned *)((char *)sp + sizeof(float) * 2 * kNoAllocBlocks);
  unsigned flag = 0;
  if (hipMemcpy(&flag, counter + 8, sizeof(flag), hipMemcpyDeviceToHost) !=
          hipSuccess ||
      !flag)
    return true;
  (void)hipMemset(counter, 0, 256);
  {
    std::lock_guard<std::mutex> lk(g_scratch_mutex);
    g_scratch_no_grid[dev] = true;
  }
  fail(EIO, "DynamicQuantizeLinearNoAlloc: the blocks of the one-launch "
            "kernel timed out waiting for one another (grid barrier); its "
            "output was not written");
  return false;
}

// Splits `shape` around `axis` for a scale of `scale_numel` entries.
bool axis_split(const View &x, int64_t scale_numel, int64_t axis,
    const char *op, int64_t &outer, int64_t &channels, int64_t &inner) {
  if (scale_numel == 1) {
    outer = 1;
    channels = 1;
    inner = x.numel;
    return true;
  }
  if (axis < 0)
    axis += x.rank;
  if (axis < 0 || axis >= x.rank) {
    fail(EINVAL, "%s: axis out of range", op);
    return false;
  }
  if (x.shape[axis] != scale_numel) {
    fail(EINVAL, "%s: scale has %lld entries, dimension %lld has %lld", op,
        (long long)scale_numel, (long long)axis, (long long)x.shape[axis]);
    return false;
  }
  outer = 1;
  inner = 1;
  for (int64_t i = 0; i < axis; ++i)
    outer *= x.shape[i];
  for (int64_t i = axis + 1; i < x.rank; ++i)
    inner *= x.shape[i];
  channels = scale_numel;
  return true;
}

// Shape of a matrix product as onnx.MatMul defines it
// (src/Dialect/ONNX/ONNXOps/Math/MatMul.cpp:200-292, numpy's matmul rules).
//  - B [K, N] (or [K], taken as [K, 1]): the leading dimensions of A
//    [.., M, K] are folded into M; one product.
//  - B [.., K, N] with leading (batch) dimensions: A is [.., M, K] (or [K],
//    taken as [1, K]), the batch dimensions of A and B are broadcast against
//    each other, and there is one M x K x N product per batch entry:
//    a_batch[i] / b_batch[i] are the matrices of A / B that entry i multiplies.
struct MatmulShape {
  int64_t M = 0, K = 0, N = 0;
  int64_t batches = 1;
  int64_t a_mats = 1, b_mats = 1; // matrices held by A and by B
  std::vector<int64_t> a_batch, b_batch;
};

bool matmul_dims(const View &a, const View &b, const char *op, bool allow_batched_b,
    MatmulShape &sh) {
  if (a.rank < 1 || b.rank < 1) {
    fail(EINVAL, "%s: A and B need at least one dimension", op);
    return false;
  }
  sh.K = a.shape[a.rank - 1];
  const int64_t bk = b.rank >= 2 ? b.shape[b.rank - 2] : b.shape[0];
  if (bk != sh.K) {
    fail(EINVAL, "%s: inner dimensions differ (%lld vs %lld)", op,
        (long long)sh.K, (long long)bk);
    return false;
  }
  sh.N = b.rank >= 2 ? b.shape[b.rank - 1] : 1;
  if (b.rank <= 2) {
    sh.M = 1;
    for (int64_t i = 0; i + 1 < a.rank; ++i)
      sh.M *= a.shape[i];
    sh.a_batch.assign(1, 0);
    sh.b_batch.assign(1, 0);
    return true;
  }
  if (!allow_batched_b) {
    fail(EINVAL, "%s: expected a 2-D B [K,N]", op);
    return false;
  }
  sh.M = a.rank >= 2 ? a.shape[a.rank - 2] : 1;
  const int64_t ar = a.rank >= 2 ? a.rank - 2 : 0, br = b.rank - 2;
  const int64_t r = ar > br ? ar : br;
  std::vector<int64_t> dims(r), astr(r, 0), bstr(r, 0);
  int64_t am = 1, bm = 1;
  for (int64_t i = r - 1; i >= 0; --i) { // right-aligned, as numpy broadcasts
    const int64_t ai = i - (r - ar), bi = i - (r - br);
    const int64_t ad = ai >= 0 ? a.shape[ai] : 1, bd = bi >= 0 ? b.shape[bi] : 1;
    if (ad != bd && ad != 1 && bd != 1) {
      fail(EINVAL, "%s: batch dimensions %lld and %lld do not broadcast", op,
          (long long)ad, (long long)bd);
      return false;
    }
    dims[i] = ad == 1 ? bd : ad;
    astr[i] = ad == 1 ? 0 : am;
    bstr[i] = bd == 1 ? 0 : bm;
    am *= ad;
    bm *= bd;
  }
  sh.a_mats = am;
  sh.b_mats = bm;
  sh.batches = 1;
  for (int64_t d : dims)
    sh.batches *= d;
  if (sh.batches > ((int64_t)1 << 20)) {
    fail(EINVAL, "%s: more than 2^20 batch entries", op);
    return false;
  }
  sh.a_batch.resize((size_t)sh.batches);
  sh.b_batch.resize((size_t)sh.batches);
  for (int64_t e = 0; e < sh.batches; ++e) {
    int64_t rest = e, ai = 0, bi = 0;
    for (int64_t i = r - 1; i >= 0; --i) {
      const int64_t c = rest % dims[i];
      rest /= dims[i];
      ai += c * astr[i];
      bi += c * bstr[i];
    }
    sh.a_batch[(size_t)e] = ai;
    sh.b_batch[(size_t)e] = bi;
  }
  return true;
}

// Packed form of B: from the cache when B was declared constant, otherwise
// packed into pool buffers for this call only.
bool packed_b(Call &call, const View &b, int64_t K, int64_t N,
    const int8_t *&bp, const int32_t *&colsum) {
  const bool uns = b.dtype == OM_MI355X_TYPE_UINT8;
  const int64_t Kpad = round_up(K > 0 ? K : 1, kGemmBK);
  const int64_t Npad = round_up(N, kGemmBN);
  bool constant;
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    constant = g_constants.count(b.data) != 0;
    if (constant) {
      auto it = g_packed.find(b.data);
      if (it != g_packed.end() && it->second.K == K && it->second.N == N &&
          it->second.is_unsigned == uns) {
        bp = it->second.bp;
        colsum = it->second.colsum;
        return true;
      }
    }
  }
  // A constant B is only ever read here, to be packed: its plain copy on the
  // GPU lasts for this call, the packed form is the one that stays.
  const void *db = call.in(b, /*keep_constant=*/false);
  if (!call.ok)
    return false;
  int8_t *pbp;
  int32_t *pcs;
  if (constant) {
    void *p = nullptr, *q = nullptr;
    if (hipMalloc(&p, (size_t)Kpad * Npad) != hipSuccess ||
        hipMalloc(&q, (size_t)Npad * 4) != hipSuccess) {
      fail(EIO, "hipMalloc for a packed constant failed");
      call.ok = false;
      return false;
    }
    pbp = (int8_t *)p;
    pcs = (int32_t *)q;
  } else {
    pbp = (int8_t *)call.temp((size_t)Kpad * Npad);
    pcs = (int32_t *)call.temp((size_t)Npad * 4);
    if (!call.ok)
      return false;
  }
  call.check(launch_pack_b(call.c.stream, db, uns, K, N, pbp, pcs), "pack B");
  if (!call.ok)
    return false;
  if (constant) {
    // Other threads use their own streams: make the packed data final first.
    call.check(hipStreamSynchronize(call.c.stream), "pack B synchronise");
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    auto ins = g_packed.emplace(b.data, PackedB{pbp, pcs, K, N, uns});
    if (!ins.second) {
      PackedB &have = ins.first->second;
      if (have.K == K && have.N == N && have.is_unsigned == uns) {
        // Another thread packed the same constant first and may already be
        // computing with its buffers: keep those, drop the ones made here
        // (nothing but this thread's finished pack kernel has touched them).
        (void)hipFree(pbp);
        (void)hipFree(pcs);
        bp = have.bp;
        colsum = have.colsum;
        return true;
      }
      // The same address declared constant with another shape: the old
      // buffers may still be read by work in flight on any stream, so they
      // are only retired here and freed when the cache is cleared.
      g_retired.push_back(have.bp);
      g_retired.push_back(have.colsum);
      have = PackedB{pbp, pcs, K, N, uns};
    }
  }
  bp = pbp;
  colsum = pcs;
  return true;
}

// A zero point has one entry, or one per row / column of a matrix (`per`), or
// -- with batched operands, as [.., M, 1] / [.., 1, N] -- one per row / column
// of every matrix of its tensor (`per * mats`).
// Whether a zero point is known to be all zeros: then it stands for no zero
// point at all (the corrections it enters are multiplied by zero), and for
// the right-hand side of a product that spares the kernels the row sums of A
// -- symmetric int8 weights, the common case of QLinearMatMul, whose
// b_zero_point is a required operand.  Host memory is looked at; GPU memory
// only if it was declared constant, once (a blocking copy), and remembered
// until om_mi355x_UnmarkConstant.
bool zero_point_is_zero(const View &v) {
  if (v.numel == 0 || v.bytes == 0 || v.bytes > ((size_t)1 << 20))
    return false;
  const uint8_t *p = (const uint8_t *)v.data;
  auto all_zero = [&](const uint8_t *h) {
    for (size_t i = 0; i < v.bytes; ++i)
      if (h[i])
        return false;
    return true;
  };
  void *backing = backed_lookup(v.data);
  if (!backing && !is_device_ptr(v.data))
    return all_zero(p);
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    if (!g_constants.count(v.data))
      return false;
    auto it = g_const_zero.find(v.data);
    if (it != g_const_zero.end() && it->second.first == v.bytes)
      return it->second.second;
  }
  std::vector<uint8_t> h(v.bytes);
  if (hipMemcpy(h.data(), backing ? backing : v.data, v.bytes,
          hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  const bool zero = all_zero(h.data());
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  g_const_zero[v.data] = std::make_pair(v.bytes, zero);
  return zero;
}

bool zp_len_ok(const View *zp, int64_t per, int64_t mats, const char *op,
    const char *name, int64_t &len) {
  if (!zp) {
    len = 0;
    return true;
  }
  if (zp->numel == 1)
    len = 1;
  else if (zp->numel == per || zp->numel == per * mats)
    len = zp->numel;
  else {
    fail(EINVAL, "%s: %s has %lld entries, expected 1 or %lld", op, name,
        (long long)zp->numel, (long long)per);
    return false;
  }
  return true;
}

// Shared body of MatMulInteger, MatMulIntegerDequant and QLinearMatMul.
struct MatmulSpec {
  const char *op;
  Epilogue epi;
  const OMTensor *y, *a, *b, *a_zp, *b_zp;
  const OMTensor *a_scale = nullptr, *b_scale = nullptr, *y_scale = nullptr,
                 *y_zp = nullptr, *bias = nullptr;
  NarrowMode narrow = kWrap;
  bool relu = false; // kEpiF32: onnx.Relu on the result
  bool gelu = false; // kEpiF32: onnx.Gelu (approximate "none") on the result
};

// The `activation` argument of the fused entry points: 0 = none, 1 = Relu,
// 2 = Gelu.
bool activation_ok(int64_t activation, const char *op, bool &relu, bool &gelu) {
  if (activation < 0 || activation > 2) {
    fail(EINVAL, "%s: activation %lld is not 0 (none), 1 (Relu) or 2 (Gelu)", op,
        (long long)activation);
    return false;
  }
  relu = activation == 1;
  gelu = activation == 2;
  return true;
}

// Optional bias of the f32 epilogue: f32, one value or one per column.
bool bias_ok(const OMTensor *bias_t, int64_t N, const char *op, View &bias) {
  if (!bias_t)
    return true;
  if (!view_of(bias_t, "bias", bias))
    return false;
  if (bias.dtype != OM_MI355X_TYPE_FLOAT || (bias.numel != 1 && bias.numel != N)) {
    fail(EINVAL, "%s: bias must be f32, scalar or [N]", op);
    return false;
  }
  return true;
}

void run_matmul(const MatmulSpec &sp) {
  View y, a, b, azp, bzp, as, bs, ys, yzp, bias;
  if (!view_of(sp.y, "y", y) || !view_of(sp.a, "a", a) ||
      !view_of(sp.b, "b", b))
    return;
  if (sp.a_zp && !view_of(sp.a_zp, "a_zero_point", azp))
    return;
  if (sp.b_zp && !view_of(sp.b_zp, "b_zero_point", bzp))
    return;
  if (!is_q8(a.dtype) || !is_q8(b.dtype)) {
    fail(EINVAL, "%s: A and B must be uint8 or int8", sp.op);
    return;
  }
  if ((sp.a_zp && azp.dtype != a.dtype) || (sp.b_zp && bzp.dtype != b.dtype)) {
    fail(EINVAL, "%s: a zero point's type differs from its tensor's", sp.op);
    return;
  }
  MatmulShape sh;
  // The fused epilogue of a linear layer keeps its 2-D weights; the ONNX ops
  // themselves take batched right-hand sides.
  if (!matmul_dims(a, b, sp.op, sp.epi != kEpiF32, sh))
    return;
  const int64_t M = sh.M, K = sh.K, N = sh.N;
  if (y.numel != sh.batches * M * N) {
    fail(EINVAL, "%s: output has %lld elements, expected %lld", sp.op,
        (long long)y.numel, (long long)(sh.batches * M * N));
    return;
  }
  const int want_y = sp.epi == kEpiI32   ? OM_MI355X_TYPE_INT32
                     : sp.epi == kEpiF32 ? OM_MI355X_TYPE_FLOAT
                                         : 0;
  if ((want_y && y.dtype != want_y) || (!want_y && !is_q8(y.dtype))) {
    fail(EINVAL, "%s: output element type %d is wrong", sp.op, y.dtype);
    return;
  }
  int64_t azl, bzl;
  if (!zp_len_ok(sp.a_zp ? &azp : nullptr, M, sh.a_mats, sp.op, "a_zero_point", azl) ||
      !zp_len_ok(sp.b_zp ? &bzp : nullptr, N, sh.b_mats, sp.op, "b_zero_point", bzl))
    return;
  if (sp.epi != kEpiI32) {
    if (!view_of(sp.a_scale, "a_scale", as) ||
        !view_of(sp.b_scale, "b_scale", bs))
      return;
    if (as.dtype != OM_MI355X_TYPE_FLOAT || bs.dtype != OM_MI355X_TYPE_FLOAT ||
        as.numel != 1 || (bs.numel != 1 && bs.numel != N)) {
      fail(EINVAL, "%s: scales must be f32, a_scale scalar, b_scale scalar "
                   "or [N]", sp.op);
      return;
    }
  }
  if (!bias_ok(sp.bias, N, sp.op, bias))
    return;
  if (sp.epi == kEpiQ8) {
    if (!view_of(sp.y_scale, "y_scale", ys) ||
        !view_of(sp.y_zp, "y_zero_point", yzp))
      return;
    if (ys.dtype != OM_MI355X_TYPE_FLOAT || ys.numel != 1 ||
        yzp.numel != 1 || yzp.dtype != y.dtype) {
      fail(EINVAL, "%s: y_scale must be an f32 scalar and y_zero_point a "
                   "scalar of the output type", sp.op);
      return;
    }
  }
  if (M == 0 || N == 0 || sh.batches == 0)
    return;

  Call call(t_ctx, sp.op);
  if (!call.ok)
    return;
  const bool a_uns = a.dtype == OM_MI355X_TYPE_UINT8;
  const bool b_uns = b.dtype == OM_MI355X_TYPE_UINT8;
  GemmArgs g = {};
  g.A = call.in(a);
  g.a_unsigned = a_uns;
  g.a_preshifted = false;
  g.b_unsigned = b_uns;
  g.M = M;
  g.K = K;
  g.N = N;
  const int32_t *colsum = nullptr;
  // One right-hand side: packed once (cached for a constant).  Batched: the
  // matrices of B are packed one after the other into buffers of this call.
  const int64_t Kpad = round_up(K > 0 ? K : 1, kGemmBK);
  const int64_t Npad = round_up(N, kGemmBN);
  const size_t bp_bytes = (size_t)Kpad * Npad;
  int8_t *bp_all = nullptr;
  int32_t *cs_all = nullptr;
  if (b.rank <= 2) {
    if (!packed_b(call, b, K, N, g.Bp, colsum)) {
      call.finish();
      return;
    }
  } else {
    const uint8_t *db = (const uint8_t *)call.in(b);
    bp_all = (int8_t *)call.temp(bp_bytes * (size_t)sh.b_mats);
    cs_all = (int32_t *)call.temp((size_t)Npad * 4 * (size_t)sh.b_mats);
    for (int64_t i = 0; call.ok && i < sh.b_mats; ++i)
      call.check(launch_pack_b(call.c.stream, db + (size_t)i * K * N, b_uns, K, N,
                     bp_all + (size_t)i * bp_bytes, cs_all + (size_t)i * Npad),
          "pack B");
    if (!call.ok) {
      call.finish();
      return;
    }
  }
  g.colsum = colsum;
  const uint8_t *d_azp = sp.a_zp ? (const uint8_t *)call.in(azp) : nullptr;
  const uint8_t *d_bzp = sp.b_zp ? (const uint8_t *)call.in(bzp) : nullptr;
  if (d_bzp && !b_uns && zero_point_is_zero(bzp)) {
    d_bzp = nullptr; // B carries no offset
    bzl = 0;
  }
  g.a_zp = d_azp;
  g.a_zp_len = azl;
  g.b_zp = d_bzp;
  g.b_zp_len = bzl;
  g.epi = sp.epi;
  if (sp.epi != kEpiI32) {
    g.a_scale = (const float *)call.in(as);
    g.b_scale = (const float *)call.in(bs);
    g.b_scale_len = bs.numel;
  }
  if (sp.bias) {
    g.bias = (const float *)call.in(bias);
    g.bias_len = bias.numel;
  }
  g.relu = sp.relu;
  g.gelu = sp.gelu;
  if (sp.epi == kEpiQ8) {
    g.y_scale = (const float *)call.in(ys);
    g.y_zp = call.in(yzp);
    g.y_unsigned = y.dtype == OM_MI355X_TYPE_UINT8;
    g.narrow = sp.narrow;
  }
  g.out = call.out(y);
  if (b.rank <= 2) {
    if (call.ok && gemm_pads_rows(M, K, g.A)) {
      // few rows of an awkward length or alignment: aligned copies whose tail
      // holds the zero point, multiplied over the padded length
      void *padded = call.temp((size_t)M * round_up(K, 16));
      if (call.ok)
        call.check(launch_pad_rows(call.c.stream, g.A, M, K, d_azp, azl,
                       /*stored_minus_128=*/false, padded),
            "pad rows");
      g.A = padded;
      g.K = round_up(K, 16);
    }
    if (call.ok)
      call.check(launch_gemm(call.c.stream, g), sp.op);
    call.finish();
    return;
  }
  // One product per batch entry, queued one after the other.
  const uint8_t *d_a = (const uint8_t *)g.A;
  char *d_y = (char *)g.out;
  const size_t y_es = sp.epi == kEpiQ8 ? 1 : 4;
  for (int64_t e = 0; call.ok && e < sh.batches; ++e) {
    const int64_t ai = sh.a_batch[(size_t)e], bi = sh.b_batch[(size_t)e];
    GemmArgs ge = g;
    ge.A = d_a + (size_t)ai * M * K;
    ge.Bp = bp_all + (size_t)bi * bp_bytes;
    ge.colsum = cs_all + (size_t)bi * Npad;
    // zero points given per matrix ([.., M, 1] / [.., 1, N]) move with it
    if (azl > M) {
      ge.a_zp = d_azp + (size_t)ai * M;
      ge.a_zp_len = M;
    }
    if (bzl > N) {
      ge.b_zp = d_bzp + (size_t)bi * N;
      ge.b_zp_len = N;
    }
    ge.out = d_y + (size_t)e * M * N * y_es;
    call.check(launch_gemm(call.c.stream, ge), sp.op);
  }
  call.finish();
}

} // namespace

// ---------------------------------------------------------------------------
// accelerator life cycle
// ---------------------------------------------------------------------------
extern "C" {

long OMIsInitAccelMI355X = 0;

void OMInitAccelMI355X(void) {
  if (!OMIsInitAccelMI355X) {
    pthread_mutex_lock(&g_init_mutex);
    if (!OMIsInitAccelMI355X) {
      g_device_ok = probe_device();
      OMIsInitAccelMI355X = 1;
    }
    pthread_mutex_unlock(&g_init_mutex);
  }
}

uint64_t OMInitCompatibleAccelMI355X(uint64_t versionNum) {
  OMInitAccelMI355X();
  // A model runs here when it was compiled for this major version or an
  // older minor one, and device 0 is a gfx950.
  const uint64_t major = (versionNum >> 16) & 0xFF;
  const uint64_t mine_major = (OM_MI355X_VERSION >> 16) & 0xFF;
  if (major != mine_major ||
      (versionNum & 0xFFFF) > (OM_MI355X_VERSION & 0xFFFF)) {
    fprintf(stderr,
        "om_mi355x: model needs runtime version 0x%llx, this runtime is "
        "0x%llx\n",
        (unsigned long long)versionNum,
        (unsigned long long)OM_MI355X_VERSION);
    errno = EPERM;
    return 0;
  }
  if (!g_device_ok) {
    fprintf(stderr,
        "om_mi355x: this model was compiled for the MI355X accelerator: %s\n",
        g_device_why.c_str());
    errno = EPERM;
    return 0;
  }
  return 1;
}

void OMShutdownAccelMI355X(void) {
  if (OMIsInitAccelMI355X) {
    pthread_mutex_lock(&g_init_mutex);
    OMIsInitAccelMI355X = 0;
    pthread_mutex_unlock(&g_init_mutex);
  }
}

void om_mi355x_SetQuantMode(OMTensor *anchor, int64_t mode) {
  (void)anchor;
  if (mode < 0 || mode > (OM_MI355X_QUANT_RECIPROCAL | OM_MI355X_QUANT_NO_ZERO_POINT)) {
    fail(EINVAL, "om_mi355x_SetQuantMode: mode %lld is not a combination of "
                 "OM_MI355X_QUANT_RECIPROCAL and OM_MI355X_QUANT_NO_ZERO_POINT",
        (long long)mode);
    return;
  }
  t_quant_mode_next = (int)mode;
}

int64_t om_mi355x_GetQuantMode(void) { return t_quant_mode_next; }

// ---------------------------------------------------------------------------
// ops
// ---------------------------------------------------------------------------
void om_mi355x_QuantizeLinear(OMTensor *y_t, const OMTensor *x_t,
    const OMTensor *scale_t, const OMTensor *zp_t, int64_t axis,
    int64_t saturate) {
  const QuantModeScope quant_mode_of_this_op;
  (void)saturate;
  View y, x, sc, zp;
  if (!view_of(y_t, "y", y) || !view_of(x_t, "x", x) ||
      !view_of(scale_t, "y_scale", sc))
    return;
  if (zp_t && !view_of(zp_t, "y_zero_point", zp))
    return;
  if (x.dtype != OM_MI355X_TYPE_FLOAT || sc.dtype != OM_MI355X_TYPE_FLOAT ||
      !is_q8(y.dtype) || y.numel != x.numel ||
      (zp_t && (zp.dtype != y.dtype || zp.numel != sc.numel))) {
    fail(EINVAL, "QuantizeLinear: expected f32 x and scale, ui8/i8 y with a "
                 "zero point of y's type and the scale's shape");
    return;
  }
  int64_t outer, channels, inner;
  if (!axis_split(x, sc.numel, axis, "QuantizeLinear", outer, channels, inner))
    return;
  if (x.numel == 0)
    return;
  Call call(t_ctx, "QuantizeLinear");
  if (!call.ok)
    return;
  const int mode = t_quant_mode;
  const float *dx = (const float *)call.in(x);
  const float *ds = (const float *)call.in(sc);
  // without zero points the one given only decides the output type
  // (src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:231-237)
  const void *dz = (zp_t && !(mode & OM_MI355X_QUANT_NO_ZERO_POINT))
                       ? call.in(zp)
                       : nullptr;
  void *dy = call.out(y);
  if (call.ok)
    call.check(launch_quantize(call.c.stream, dx, outer, channels, inner, ds,
                   dz, y.dtype == OM_MI355X_TYPE_INT8, dy,
                   (mode & OM_MI355X_QUANT_RECIPROCAL) != 0),
        "QuantizeLinear");
  call.finish();
}

void om_mi355x_DequantizeLinear(OMTensor *y_t, const OMTensor *x_t,
    const OMTensor *scale_t, const OMTensor *zp_t, int64_t axis) {
  const QuantModeScope quant_mode_of_this_op;
  View y, x, sc, zp;
  if (!view_of(y_t, "y", y) || !view_of(x_t, "x", x) ||
      !view_of(scale_t, "x_scale", sc))
    return;
  if (zp_t && !view_of(zp_t, "x_zero_point", zp))
    return;
  const bool x_ok = is_q8(x.dtype) || x.dtype == OM_MI355X_TYPE_INT32;
  if (!x_ok || y.dtype != OM_MI355X_TYPE_FLOAT ||
      sc.dtype != OM_MI355X_TYPE_FLOAT || y.numel != x.numel ||
      (zp_t && (zp.dtype != x.dtype || zp.numel != sc.numel))) {
    fail(EINVAL, "DequantizeLinear: expected ui8/i8/i32 x, f32 scale and y, a "
                 "zero point of x's type and the scale's shape");
    return;
  }
  int64_t outer, channels, inner;
  if (!axis_split(
          x, sc.numel, axis, "DequantizeLinear", outer, channels, inner))
    return;
  if (x.numel == 0)
    return;
  Call call(t_ctx, "DequantizeLinear");
  if (!call.ok)
    return;
  const void *dx = call.in(x);
  const float *ds = (const float *)call.in(sc);
  // (src/Conversion/ONNXToKrnl/Math/Elementwise.cpp:1453)
  const void *dz = (zp_t && !(t_quant_mode & OM_MI355X_QUANT_NO_ZERO_POINT))
                       ? call.in(zp)
                       : nullptr;
  float *dy = (float *)call.out(y);
  const QKind kind = x.dtype == OM_MI355X_TYPE_UINT8  ? kU8
                     : x.dtype == OM_MI355X_TYPE_INT8 ? kI8
                                                      : kI32;
  if (call.ok)
    call.check(launch_dequantize(call.c.stream, dx, kind, outer, channels,
                   inner, ds, dz, dy),
        "DequantizeLinear");
  call.finish();
}

void om_mi355x_DynamicQuantizeLinear(OMTensor *y_t, OMTensor *scale_t,
    OMTensor *zp_t, const OMTensor *x_t) {
  const QuantModeScope quant_mode_of_this_op;
  View y, sc, zp, x;
  if (!view_of(y_t, "y", y) || !view_of(scale_t, "y_scale", sc) ||
      !view_of(zp_t, "y_zero_point", zp) || !view_of(x_t, "x", x))
    return;
  if (x.dtype != OM_MI355X_TYPE_FLOAT || y.dtype != OM_MI355X_TYPE_UINT8 ||
      sc.dtype != OM_MI355X_TYPE_FLOAT || zp.dtype != OM_MI355X_TYPE_UINT8 ||
      sc.numel != 1 || zp.numel != 1 || y.numel != x.numel) {
    fail(EINVAL, "DynamicQuantizeLinear: expected f32 x, ui8 y of x's shape, "
                 "scalar f32 scale and scalar ui8 zero point");
    return;
  }
  // No elements: scale and zero point are still results (0 and 0: the range
  // is widened to include 0, DynamicQuantizeLinear.cpp:64-83).
  Call call(t_ctx, "DynamicQuantizeLinear");
  if (!call.ok)
    return;
  const float *dx = (const float *)call.in(x);
  uint8_t *dy = (uint8_t *)call.out(y);
  float *ds = (float *)call.out(sc);
  uint8_t *dz = (uint8_t *)call.out(zp);
  if (call.ok)
    run_dql(call, dx, x.numel, dy, ds, dz, false);
  call.finish();
}

void om_mi355x_DynamicQuantizeLinearNoAlloc(OMTensor *y_t, OMTensor *scale_t,
    OMTensor *zp_t, const OMTensor *x_t) {
  const QuantModeScope quant_mode_of_this_op;
  const char *op = "DynamicQuantizeLinearNoAlloc";
  View y, sc, zp, x;
  if (!view_of(y_t, "y", y) || !view_of(scale_t, "y_scale", sc) ||
      !view_of(zp_t, "y_zero_point", zp) || !view_of(x_t, "x", x))
    return;
  if (x.dtype != OM_MI355X_TYPE_FLOAT || y.dtype != OM_MI355X_TYPE_UINT8 ||
      sc.dtype != OM_MI355X_TYPE_FLOAT || zp.dtype != OM_MI355X_TYPE_UINT8 ||
      sc.numel != 1 || zp.numel != 1 || y.numel != x.numel) {
    fail(EINVAL, "%s: expected f32 x, ui8 y of x's shape, scalar f32 scale "
                 "and scalar ui8 zero point", op);
    return;
  }
  if (x.numel > OM_MI355X_NOALLOC_MAX_ELEMENTS) {
    fail(EINVAL, "%s: x has %lld elements, the limit of this entry point is "
                 "%lld", op, (long long)x.numel,
        (long long)OM_MI355X_NOALLOC_MAX_ELEMENTS);
    return;
  }
  // Creating the thread's stream allocates, so it must exist already.
  Ctx &c = t_ctx;
  if (!c.ready) {
    fail(EINVAL, "%s: this thread has no stream yet; call "
                 "om_mi355x_synchronize() (or any other entry point) on it "
                 "once, outside the region that must not allocate", op);
    return;
  }
  // Every tensor must be GPU memory already: staging a host tensor would take
  // a buffer from the pool, which may allocate.
  const View *all[4] = {&y, &sc, &zp, &x};
  void *dev_ptr[4];
  for (int i = 0; i < 4; ++i) {
    dev_ptr[i] = all[i]->data;
    if (all[i]->numel == 0)
      continue; // never dereferenced
    void *d = backed_lookup(all[i]->data);
    if (!d && is_device_ptr(all[i]->data))
      d = all[i]->data;
    if (!d) {
      fail(EINVAL, "%s: every tensor must be in GPU memory", op);
      return;
    }
    dev_ptr[i] = d;
  }
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || !resolve_scratch(dev)) {
    (void)hipGetLastError();
    fail(EIO, "%s: the scratch array has no address on this device", op);
    return;
  }
  // From here on `sp`, the array's address on this device, stands for it.
  std::lock_guard<std::mutex> lk(g_scratch_mutex);
  char *const sp = (char *)g_scratch_ptr[dev];
  DqlScratch s;
  s.partial_min = (float *)sp;
  s.partial_max = s.partial_min + kNoAllocBlocks;
  s.counter = (unsigned *)(s.partial_max + kNoAllocBlocks);
  s.grid_slots = (unsigned long long *)((char *)s.counter + 256);
  s.max_blocks = kNoAllocBlocks;
  // The one-launch kernel tags its exchange slots with a launch number that
  // is a kernel argument, and asks another stream whether it is idle: neither
  // survives being recorded into a graph and replayed.  Should this thread's
  // stream be under capture, the two-launch form is recorded instead (fill
  // kernel, minimum / maximum with an arrival counter, quantize), which
  // carries no such state.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(c.stream, &capture) != hipSuccess) {
    (void)hipGetLastError();
    capture = hipStreamCaptureStatusNone;
  }
  s.grid_blocks = (g_scratch_no_grid[dev] || capture != hipStreamCaptureStatusNone)
                      ? 0
                      : std::min(c.dql.grid_blocks, kNoAllocBlocks);
  s.spin_limit = c.dql.spin_limit;
  s.epoch = g_scratch_epoch[dev];
  g_scratch_used[dev] = true;
  g_scratch_unchecked[dev] = true;
  g_scratch_launcher[dev] = std::this_thread::get_id();
  // The array keeps what the last call left.  The slots need no clearing
  // (they carry the launch number); the arrival counter of the two-launch
  // path must start at zero and would not be if an earlier launch had been
  // cut short.  A fill kernel, not a memset: the caller may be recording a
  // graph.  The "gave up" flag (word 8) is left for the next synchronisation
  // to report.
  hipError_t e = launch_fill_u32(c.stream, (uint32_t *)s.counter, 8, 0u);
  if (e == hipSuccess)
    e = launch_dynamic_quantize(c.stream, s, (const float *)dev_ptr[3],
        x.numel, (uint8_t *)dev_ptr[0], (float *)dev_ptr[1],
        (uint8_t *)dev_ptr[2], false, t_quant_mode);
  g_scratch_epoch[dev] = s.epoch;
  if (e != hipSuccess)
    fail(EIO, "%s failed: %s", op, hipGetErrorString(e));
}

void om_mi355x_MatMulInteger(OMTensor *y, const OMTensor *a,
    const OMTensor *b, const OMTensor *a_zp, const OMTensor *b_zp) {
  MatmulSpec sp = {"MatMulInteger", kEpiI32, y, a, b, a_zp, b_zp};
  run_matmul(sp);
}

void om_mi355x_MatMulIntegerDequant(OMTensor *y, const OMTensor *a,
    const OMTensor *b, const OMTensor *a_zp, const OMTensor *b_zp,
    const OMTensor *a_scale, const OMTensor *b_scale, const OMTensor *bias,
    int64_t activation) {
  MatmulSpec sp = {"MatMulIntegerDequant", kEpiF32, y, a, b, a_zp, b_zp};
  if (!activation_ok(activation, sp.op, sp.relu, sp.gelu))
    return;
  sp.a_scale = a_scale;
  sp.b_scale = b_scale;
  sp.bias = bias;
  run_matmul(sp);
}

void om_mi355x_QLinearMatMul(OMTensor *y, const OMTensor *a,
    const OMTensor *a_scale, const OMTensor *a_zp, const OMTensor *b,
    const OMTensor *b_scale, const OMTensor *b_zp, const OMTensor *y_scale,
    const OMTensor *y_zp, int64_t narrow_mode) {
  if (!a_zp || !b_zp || !y_zp) {
    fail(EINVAL, "QLinearMatMul: zero points are required operands");
    return;
  }
  MatmulSpec sp = {"QLinearMatMul", kEpiQ8, y, a, b, a_zp, b_zp};
  sp.a_scale = a_scale;
  sp.b_scale = b_scale;
  sp.y_scale = y_scale;
  sp.y_zp = y_zp;
  sp.narrow = narrow_mode ? kSaturate : kWrap;
  run_matmul(sp);
}

} // extern "C"

namespace {
// The fused layer, with or without the limits of x handed in and those of y
// handed out (om_mi355x_DynQuantMatMulDequantLimits).
void dyn_quant_matmul_dequant(const char *op, OMTensor *y_t,
    OMTensor *ylim_t, const OMTensor *x_t, const OMTensor *xlim_t,
    const OMTensor *b_t, const OMTensor *bzp_t, const OMTensor *bscale_t,
    const OMTensor *bias_t, int64_t activation) {
  const QuantModeScope quant_mode_of_this_op;
  View y, x, b, bzp, bs, bias, ylim, xlim;
  bool relu, gelu;
  if (!activation_ok(activation, op, relu, gelu))
    return;
  if (!view_of(y_t, "y", y) || !view_of(x_t, "x", x) ||
      !view_of(b_t, "b", b) || !view_of(bscale_t, "b_scale", bs))
    return;
  if (bzp_t && !view_of(bzp_t, "b_zero_point", bzp))
    return;
  if ((ylim_t && !view_of(ylim_t, "y_limits", ylim)) ||
      (xlim_t && !view_of(xlim_t, "x_limits", xlim)))
    return;
  if ((ylim_t && (ylim.dtype != OM_MI355X_TYPE_FLOAT || ylim.numel != 2)) ||
      (xlim_t && (xlim.dtype != OM_MI355X_TYPE_FLOAT || xlim.numel != 2))) {
    fail(EINVAL, "%s: limits are f32 tensors of two elements (minimum, "
                 "maximum)", op);
    return;
  }
  if (x.dtype != OM_MI355X_TYPE_FLOAT || y.dtype != OM_MI355X_TYPE_FLOAT ||
      !is_q8(b.dtype) || bs.dtype != OM_MI355X_TYPE_FLOAT ||
      (bzp_t && bzp.dtype != b.dtype)) {
    fail(EINVAL, "%s: expected f32 x and y, ui8/i8 b, f32 b_scale", op);
    return;
  }
  MatmulShape sh;
  if (!matmul_dims(x, b, op, false, sh))
    return;
  const int64_t M = sh.M, K = sh.K, N = sh.N;
  int64_t bzl;
  if (!zp_len_ok(bzp_t ? &bzp : nullptr, N, 1, op, "b_zero_point", bzl))
    return;
  if (y.numel != M * N || (bs.numel != 1 && bs.numel != N)) {
    fail(EINVAL, "%s: output or b_scale shape is wrong", op);
    return;
  }
  if (!bias_ok(bias_t, N, op, bias))
    return;
  if (M == 0 || N == 0)
    return;
  Call call(t_ctx, op);
  if (!call.ok)
    return;
  const float *dx = (const float *)call.in(x);
  const float *d_xlim = xlim_t ? (const float *)call.in(xlim, false) : nullptr;
  void *dy = call.out(y); // before the quantization: it decides whether to wait
  float *d_ylim = ylim_t ? (float *)call.out(ylim) : nullptr;
  const int32_t *colsum = nullptr;
  const int8_t *bp = nullptr;
  if (!call.ok || !packed_b(call, b, K, N, bp, colsum)) {
    call.finish();
    return;
  }
  const void *d_bzp = bzp_t ? call.in(bzp) : nullptr;
  const float *d_bs = (const float *)call.in(bs);
  const float *d_bias = bias_t ? (const float *)call.in(bias) : nullptr;
  // in_kernel: the GEMM kernel quantizes the rows itself (a few rows: every
  // block on its own; up to one round of 32-row blocks: the blocks agree on
  // minimum and maximum through the exchange slots).  Otherwise
  // DynamicQuantizeLinear is a launch of its own and the quantized
  // activations stay on the GPU, stored as (u8 - 128) so that the GEMM stages
  // them without a per-byte fix-up.
  auto run = [&](bool in_kernel) -> hipError_t {
    int64_t padded_k = 0;
    GemmArgs g = {};
    g.out = dy;
    g.y_limits = d_ylim;
    g.dql = &call.c.dql;
    if (in_kernel) {
      g.X = dx;
      g.x_limits = d_xlim;
    } else {
      uint8_t *aq = (uint8_t *)call.temp((size_t)M * K);
      if (call.ok && d_xlim)
        // minimum and maximum are known: one pass, no reduction
        call.check(launch_quantize_from_limits(call.c.stream, dx, M * K, d_xlim,
                       aq, call.c.dql_scale, call.c.dql_zp, true, t_quant_mode),
            "quantize");
      else if (call.ok)
        run_dql(call, dx, M * K, aq, call.c.dql_scale, call.c.dql_zp, true);
      g.A = aq;
      if (call.ok && gemm_pads_rows(M, K, aq)) {
        // (see run_matmul) the quantized rows are stored minus 128
        void *padded = call.temp((size_t)M * round_up(K, 16));
        if (call.ok)
          call.check(launch_pad_rows(call.c.stream, aq, M, K, call.c.dql_zp, 1,
                         /*stored_minus_128=*/true, padded),
              "pad rows");
        g.A = padded;
        padded_k = round_up(K, 16);
      }
      if (!call.ok)
        return hipSuccess; // already reported
    }
    g.a_unsigned = true;
    g.a_preshifted = true;
    g.b_unsigned = b.dtype == OM_MI355X_TYPE_UINT8;
    g.M = M;
    g.K = padded_k ? padded_k : K;
    g.N = N;
    g.Bp = bp;
    g.colsum = colsum;
    g.a_zp = call.c.dql_zp;
    g.a_zp_len = 1;
    g.b_zp = d_bzp;
    g.b_zp_len = bzl;
    g.epi = kEpiF32;
    g.a_scale = call.c.dql_scale;
    g.b_scale = d_bs;
    g.b_scale_len = bs.numel;
    g.bias = d_bias;
    g.bias_len = bias_t ? bias.numel : 0;
    g.relu = relu;
    g.gelu = gelu;
    return launch_gemm(call.c.stream, g);
  };
  const int kind = (call.ok && t_quant_mode == 0 && call.c.dql.grid_blocks >= 0)
                       ? gemm_quantizes_rows(M, K, N, dx)
                       : 0;
  // Blocks that wait for one another (more rows than one block quantizes for
  // itself, and limits of x that are not known) raise the same flag as
  // DynamicQuantizeLinear's one-launch kernel when they give up; checked like
  // that kernel's.
  const bool exchanges = kind == 2 && !d_xlim;
  const bool in_kernel = kind == 1 || (kind == 2 && (d_xlim || call.c.dql.grid_blocks > 0));
  hipError_t e = hipSuccess;
  if (call.ok) {
    e = run(in_kernel);
    if (e == hipErrorNotReady && exchanges) // the exchange is taken or off
      e = run(false);
    else if (e == hipSuccess && exchanges) {
      call.c.dql_unchecked = true;
      if (!(call.touched_host || sync_every_call() || report_enabled()))
        call.used_dql = true;
      else {
        e = hipStreamSynchronize(call.c.stream);
        if (e == hipSuccess && call.c.dql_gave_up()) {
          fprintf(stderr,
              "om_mi355x: %s: the blocks of the one-launch "
              "kernel timed out waiting for one another; redone with two launches "
              "for the quantization and one for the product, which this thread "
              "uses from now on\n", op);
          e = run(false);
        }
      }
    }
    if (call.ok)
      call.check(e, op);
  }
  call.finish();
}
} // namespace

extern "C" {

void om_mi355x_DynQuantMatMulDequant(OMTensor *y_t, const OMTensor *x_t,
    const OMTensor *b_t, const OMTensor *bzp_t, const OMTensor *bscale_t,
    const OMTensor *bias_t, int64_t activation) {
  dyn_quant_matmul_dequant("DynQuantMatMulDequant", y_t, nullptr, x_t, nullptr,
      b_t, bzp_t, bscale_t, bias_t, activation);
}

void om_mi355x_DynQuantMatMulDequantLimits(OMTensor *y_t, OMTensor *ylim_t,
    const OMTensor *x_t, const OMTensor *xlim_t, const OMTensor *b_t,
    const OMTensor *bzp_t, const OMTensor *bscale_t, const OMTensor *bias_t,
    int64_t activation) {
  dyn_quant_matmul_dequant("DynQuantMatMulDequantLimits", y_t, ylim_t, x_t,
      xlim_t, b_t, bzp_t, bscale_t, bias_t, activation);
}

// ---------------------------------------------------------------------------
// residency, memory, measurement
// ---------------------------------------------------------------------------
void om_mi355x_MarkConstant(const OMTensor *t) {
  if (!t)
    return;
  const void *p = omTensorGetDataPtr(t);
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  g_constants.insert(p);
}

void om_mi355x_UnmarkConstant(const OMTensor *t) {
  if (!t)
    return;
  const void *p = omTensorGetDataPtr(t);
  void *drop[3] = {nullptr, nullptr, nullptr};
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    g_constants.erase(p);
    g_const_zero.erase(p);
    auto c = g_const_copies.find(p);
    if (c != g_const_copies.end()) {
      drop[0] = c->second.dev;
      g_const_copies.erase(c);
    }
    auto k = g_packed.find(p);
    if (k != g_packed.end()) {
      drop[1] = k->second.bp;
      drop[2] = k->second.colsum;
      g_packed.erase(k);
    }
  }
  if (drop[0] || drop[1]) {
    (void)hipDeviceSynchronize(); // work on any stream may still read them
    for (void *d : drop)
      if (d)
        (void)hipFree(d);
  }
}

// The GPU blocks come from the calling thread's pool and go back to it, so a
// model that declares and releases the same buffers on every inference
// allocates only during the first one.  Work that uses a block is queued on
// the declaring thread's stream; a release from that thread needs no wait
// (the next user of the block is ordered behind it on the same stream), a
// release from another thread waits for that stream first.
void om_mi355x_KeepOnDevice(const OMTensor *t) {
  View v;
  if (!t || !view_of(t, "tensor", v) || v.bytes == 0)
    return;
  if (!t_ctx.init())
    return;
  if (is_device_ptr(v.data))
    return; // already GPU memory: nothing to back
  Backing old = {nullptr, 0, 0, nullptr};
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    auto it = g_backed.find((uintptr_t)v.data);
    if (it != g_backed.end()) {
      if (it->second.bytes == v.bytes)
        return;
      old = it->second; // same address, other size: a buffer that was freed
      g_backed.erase(it); // and allocated again without a release
    }
  }
  if (old.dev) {
    if (old.stream && old.stream != t_ctx.stream)
      (void)hipStreamSynchronize(old.stream);
    t_ctx.adopt(old.dev, old.capacity);
  }
  size_t capacity = 0;
  void *d = t_ctx.take_owned(v.bytes, &capacity);
  if (!d)
    return;
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  g_backed[(uintptr_t)v.data] = Backing{d, v.bytes, capacity, t_ctx.stream};
}

void om_mi355x_Release(const OMTensor *t) {
  if (!t)
    return;
  const void *p = omTensorGetDataPtr(t);
  Backing b;
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    auto it = g_backed.find((uintptr_t)p);
    if (it == g_backed.end())
      return;
    b = it->second;
    g_backed.erase(it);
  }
  if (t_ctx.ready && b.stream == t_ctx.stream) {
    t_ctx.adopt(b.dev, b.capacity);
    return;
  }
  if (b.stream)
    (void)hipStreamSynchronize(b.stream);
  (void)hipFree(b.dev);
}

void om_mi355x_ClearCache(void) {
  // Cached buffers may be in use on any thread's stream.
  if (t_ctx.ready)
    (void)hipDeviceSynchronize();
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  for (void *p : g_retired)
    (void)hipFree(p);
  g_retired.clear();
  for (auto &kv : g_const_copies)
    (void)hipFree(kv.second.dev);
  g_const_copies.clear();
  for (auto &kv : g_packed) {
    (void)hipFree(kv.second.bp);
    (void)hipFree(kv.second.colsum);
  }
  g_packed.clear();
  g_constants.clear();
  g_const_zero.clear();
  for (auto &kv : g_backed)
    (void)hipFree(kv.second.dev);
  g_backed.clear();
  t_ctx.drop_pool();
}

void *om_mi355x_malloc(size_t bytes) {
  if (!t_ctx.init())
    return nullptr;
  void *p = nullptr;
  hipError_t e = hipMalloc(&p, bytes ? bytes : 16);
  if (e != hipSuccess) {
    fail(EIO, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_mem_mutex);
  g_user_allocs[(uintptr_t)p] = bytes ? bytes : 16;
  return p;
}

void om_mi355x_free(void *p) {
  if (!p)
    return;
  if (t_ctx.ready)
    (void)hipStreamSynchronize(t_ctx.stream);
  {
    std::lock_guard<std::mutex> lk(g_mem_mutex);
    g_user_allocs.erase((uintptr_t)p);
    g_constants.erase(p);
    g_const_zero.erase(p);
    auto it = g_packed.find(p);
    if (it != g_packed.end()) {
      (void)hipFree(it->second.bp);
      (void)hipFree(it->second.colsum);
      g_packed.erase(it);
    }
  }
  (void)hipFree(p);
}

int om_mi355x_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  if (!t_ctx.init())
    return -1;
  hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
      t_ctx.stream);
  if (e == hipSuccess)
    e = hipStreamSynchronize(t_ctx.stream);
  if (e != hipSuccess) {
    fail(EIO, "host-to-device copy failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

int om_mi355x_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  if (!t_ctx.init())
    return -1;
  hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
      t_ctx.stream);
  if (e == hipSuccess)
    e = hipStreamSynchronize(t_ctx.stream);
  if (e != hipSuccess) {
    fail(EIO, "device-to-host copy failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

int om_mi355x_synchronize(void) {
  if (!t_ctx.init())
    return -1;
  // A stream with nothing left to do is found idle by a query; waiting on it
  // would still cost a round trip to the GPU (about 30 us).
  hipError_t e = hipStreamQuery(t_ctx.stream);
  if (e == hipErrorNotReady)
    e = hipStreamSynchronize(t_ctx.stream);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    fail(EIO, "stream synchronisation failed: %s", hipGetErrorString(e));
    return -1;
  }
  const bool mine_ok = t_ctx.dql_barrier_ok();
  return (noalloc_barrier_ok() && mine_ok) ? 0 : -1;
}

void om_mi355x_Synchronize(OMTensor *anchor) {
  (void)anchor;
  (void)om_mi355x_synchronize();
}

int om_mi355x_timer_start(void) {
  if (!t_ctx.init())
    return -1;
  hipError_t e = hipEventRecord(t_ctx.ev0, t_ctx.stream);
  if (e != hipSuccess) {
    fail(EIO, "hipEventRecord failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

float om_mi355x_timer_stop(void) {
  if (!t_ctx.init())
    return -1.0f;
  hipError_t e = hipEventRecord(t_ctx.ev1, t_ctx.stream);
  if (e == hipSuccess)
    e = hipEventSynchronize(t_ctx.ev1);
  float ms = -1.0f;
  if (e == hipSuccess)
    e = hipEventElapsedTime(&ms, t_ctx.ev0, t_ctx.ev1);
  if (e != hipSuccess) {
    fail(EIO, "event timing failed: %s", hipGetErrorString(e));
    return -1.0f;
  }
  return ms;
}

const char *om_mi355x_last_error(void) {
  t_last_error_returned.swap(t_last_error);
  t_last_error.clear();
  return t_last_error_returned.c_str();
}

const char *om_mi355x_last_gemm_kernel(void) { return last_gemm_kernel(); }

int om_mi355x_device_info(char *buf, size_t len) {
  if (!t_ctx.init())
    return -1;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  snprintf(buf, len, "%s|%s|%d|%d|%.1f", prop.name, prop.gcnArchName,
      prop.multiProcessorCount, prop.clockRate / 1000,
      (double)prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
  return 0;
}

} // extern "C"
