// Host execution of the library's kernels: one fiber per lane, workgroups spread over a pool of OS threads.
// TEST INFRASTRUCTURE ONLY (see include/hip/hip_runtime.h in this directory for what it checks and what it does not).
#include <sys/mman.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "hip/hip_runtime.h"

#if defined(KSQ_EMU_ASAN)
extern "C" {
void __sanitizer_start_switch_fiber(void** fake_stack_save, const void* bottom, size_t size);
void __sanitizer_finish_switch_fiber(void* fake_stack_save, const void** bottom_old, size_t* size_old);
void __asan_unpoison_memory_region(void const volatile* addr, size_t size);
}
#endif

// ---- context switch (x86-64 System V: callee-saved registers and the stack pointer) ------------------------------------
extern "C" void emu_switch(void** save_sp, void* load_sp);
asm(R"(
.text
.globl emu_switch
.type emu_switch,@function
emu_switch:
  pushq %rbp
  pushq %rbx
  pushq %r12
  pushq %r13
  pushq %r14
  pushq %r15
  movq %rsp, (%rdi)
  movq %rsi, %rsp
  popq %r15
  popq %r14
  popq %r13
  popq %r12
  popq %rbx
  popq %rbp
  ret
.size emu_switch,.-emu_switch
)");

namespace emu {

thread_local LaneState* cur = nullptr;

namespace {

// ---- configuration and error log ----------------------------------------------------------------------------------------
std::mutex g_log_mutex;
std::vector<std::string> g_errors;
std::atomic<long> g_error_count{0};
std::atomic<long> g_partial_rendezvous{0};
std::atomic<int> g_sample_blocks{0};  // 0: every workgroup; n: about n column positions of a grid (all of grid.y each)
int g_threads = 0;
constexpr size_t kMaxLoggedErrors = 64;

void log_error(const std::string& s) {
  g_error_count++;
  std::lock_guard<std::mutex> lock(g_log_mutex);
  if (g_errors.size() < kMaxLoggedErrors) g_errors.push_back(s);
}

// ---- allocation registry --------------------------------------------------------------------------------------------------
struct Alloc {
  uintptr_t lo, hi;
  std::string tag;
};
std::mutex g_alloc_mutex;
std::vector<Alloc> g_allocs;           // sorted by lo, disjoint
std::atomic<unsigned> g_alloc_version{0};

void register_range(uintptr_t lo, size_t bytes, const char* tag) {
  if (bytes == 0) return;
  std::lock_guard<std::mutex> lock(g_alloc_mutex);
  const uintptr_t hi = lo + bytes;
  // a new tensor replaces whatever stale entries it overlaps
  g_allocs.erase(std::remove_if(g_allocs.begin(), g_allocs.end(), [&](const Alloc& a) { return a.lo < hi && lo < a.hi; }),
                 g_allocs.end());
  Alloc a{lo, hi, tag ? tag : ""};
  g_allocs.insert(std::upper_bound(g_allocs.begin(), g_allocs.end(), a, [](const Alloc& x, const Alloc& y) { return x.lo < y.lo; }), a);
  g_alloc_version++;
}
void unregister_range(uintptr_t lo) {
  std::lock_guard<std::mutex> lock(g_alloc_mutex);
  g_allocs.erase(std::remove_if(g_allocs.begin(), g_allocs.end(), [&](const Alloc& a) { return a.lo == lo; }), g_allocs.end());
  g_alloc_version++;
}

// a launch works on a snapshot: the registry does not change while kernels run
struct Snapshot {
  unsigned version = ~0u;
  std::vector<Alloc> allocs;
};
Snapshot g_snapshot;
void refresh_snapshot() {
  std::lock_guard<std::mutex> lock(g_alloc_mutex);
  if (g_snapshot.version != g_alloc_version.load()) {
    g_snapshot.allocs = g_allocs;
    g_snapshot.version = g_alloc_version.load();
  }
}
const Alloc* find_alloc(uintptr_t p) {
  const auto& v = g_snapshot.allocs;
  size_t lo = 0, hi = v.size();
  while (lo < hi) {
    const size_t mid = (lo + hi) / 2;
    if (v[mid].hi <= p) lo = mid + 1;
    else hi = mid;
  }
  return (lo < v.size() && v[lo].lo <= p) ? &v[lo] : nullptr;
}

// ---- fibers ---------------------------------------------------------------------------------------------------------------
#if defined(KSQ_EMU_ASAN)
constexpr size_t kStackBytes = 1 << 20;
#else
constexpr size_t kStackBytes = 256 << 10;
#endif
constexpr size_t kGuardBytes = 4096;

enum class Wait { kNone, kWave, kBlock };

struct Fiber {
  LaneState ls;
  void* sp = nullptr;
  char* stack = nullptr;  // lowest address of the mapping (guard page first)
  bool done = false;
  Wait wait = Wait::kNone;
  unsigned wait_gen = 0;
};

struct BlockState {
  unsigned gen = 0;
  int arrived = 0, alive = 0;
};

struct Worker {
  std::vector<Fiber> fibers;
  std::vector<WaveState> waves;
  BlockState block;
  void* sched_sp = nullptr;
  Fiber* running = nullptr;
  void (*tramp)(void*) = nullptr;
  void* closure = nullptr;
  const char* kernel = "";
#if defined(KSQ_EMU_ASAN)
  const void* sched_stack_bottom = nullptr;
  size_t sched_stack_size = 0;
#endif
};
thread_local Worker* tl_worker = nullptr;

void to_scheduler(Worker* w, Fiber* f) {
#if defined(KSQ_EMU_ASAN)
  void* fake = nullptr;
  __sanitizer_start_switch_fiber(f->done ? nullptr : &fake, w->sched_stack_bottom, w->sched_stack_size);
  emu_switch(&f->sp, w->sched_sp);
  __sanitizer_finish_switch_fiber(fake, nullptr, nullptr);
#else
  emu_switch(&f->sp, w->sched_sp);
#endif
}

void to_fiber(Worker* w, Fiber* f) {
  w->running = f;
  cur = &f->ls;
#if defined(KSQ_EMU_ASAN)
  void* fake = nullptr;
  __sanitizer_start_switch_fiber(&fake, f->stack + kGuardBytes, kStackBytes - kGuardBytes);
  emu_switch(&w->sched_sp, f->sp);
  __sanitizer_finish_switch_fiber(fake, &w->sched_stack_bottom, &w->sched_stack_size);
#else
  emu_switch(&w->sched_sp, f->sp);
#endif
  w->running = nullptr;
}

extern "C" void emu_fiber_entry() {
  Worker* w = tl_worker;
  Fiber* f = w->running;
#if defined(KSQ_EMU_ASAN)
  __sanitizer_finish_switch_fiber(nullptr, &w->sched_stack_bottom, &w->sched_stack_size);
#endif
  w->tramp(w->closure);
  f->done = true;
  to_scheduler(w, f);
  std::abort();  // a finished fiber is never resumed
}

void prepare_fiber(Fiber* f) {
  if (!f->stack) {
    void* m = mmap(nullptr, kStackBytes, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (m == MAP_FAILED) {
      std::perror("emu: mmap of a lane stack");
      std::abort();
    }
    f->stack = static_cast<char*>(m);
    mprotect(f->stack, kGuardBytes, PROT_NONE);
  }
#if defined(KSQ_EMU_ASAN)
  // the frames of the lane that used this stack before never returned (a finished fiber is switched away from):
  // their red zones are still poisoned
  __asan_unpoison_memory_region(f->stack + kGuardBytes, kStackBytes - kGuardBytes);
#endif
  // top of stack: [fake return slot][entry][rbp rbx r12 r13 r14 r15]; after the pops and `ret` the stack pointer is
  // 8 below a 16-byte boundary, as at the entry of any called function
  uintptr_t top = reinterpret_cast<uintptr_t>(f->stack + kStackBytes) & ~(uintptr_t)15;
  void** sp = reinterpret_cast<void**>(top);
  *--sp = nullptr;
  *--sp = reinterpret_cast<void*>(&emu_fiber_entry);
  for (int i = 0; i < 6; ++i) *--sp = nullptr;
  f->sp = sp;
  f->done = false;
  f->wait = Wait::kNone;
}

void complete_wave(WaveState* ws) {
  const int slot = (int)(ws->gen & 1u);
  ws->first[slot] = ws->alive_mask ? __builtin_ctzll(ws->alive_mask) : 0;
  if (ws->fn) ws->fn(ws, slot, ws->fn_kind);
  ws->fn = nullptr;
  ws->arrived = 0;
  ws->gen++;
}

std::string where(const Worker* w, const LaneState& ls) {
  char buf[256];
  std::snprintf(buf, sizeof(buf), "%s block (%u,%u,%u) thread %u", w->kernel, ls.bid.x, ls.bid.y, ls.bid.z, ls.tid.x);
  return buf;
}

// one workgroup, start to finish
void run_block(Worker* w, dim3 grid, dim3 block, dim3 bid) {
  const int n = (int)(block.x * block.y * block.z), nwaves = (n + 63) / 64;
  if ((int)w->fibers.size() < n) w->fibers.resize(n);
  if ((int)w->waves.size() < nwaves) w->waves.resize(nwaves);
  w->block = BlockState{};
  w->block.alive = n;
  for (int v = 0; v < nwaves; ++v) {
    WaveState& ws = w->waves[v];
    ws.gen = 0;
    ws.arrived = 0;
    ws.alive = std::min(64, n - 64 * v);
    ws.alive_mask = ws.alive == 64 ? ~0ull : ((1ull << ws.alive) - 1);
    ws.fn = nullptr;
    ws.site = 0;
  }
  for (int i = 0; i < n; ++i) {
    Fiber& f = w->fibers[i];
    prepare_fiber(&f);
    f.ls.tid = dim3((unsigned)i % block.x, ((unsigned)i / block.x) % block.y, (unsigned)i / (block.x * block.y));
    f.ls.bid = bid;
    f.ls.bdim = block;
    f.ls.gdim = grid;
    f.ls.lane = i & 63;
    f.ls.wave = &w->waves[i >> 6];
  }
  int alive = n;
  while (alive > 0) {
    bool progress = false;
    for (int i = 0; i < n; ++i) {
      Fiber& f = w->fibers[i];
      if (f.done) continue;
      if (f.wait == Wait::kWave && f.ls.wave->gen == f.wait_gen) continue;
      if (f.wait == Wait::kBlock && w->block.gen == f.wait_gen) continue;
      f.wait = Wait::kNone;
      to_fiber(w, &f);
      progress = true;
      if (f.done) {
        --alive;
        WaveState* ws = f.ls.wave;
        ws->alive--;
        ws->alive_mask &= ~(1ull << f.ls.lane);
        if (ws->arrived > 0 && ws->arrived == ws->alive) complete_wave(ws);
        w->block.alive--;
        if (w->block.arrived > 0 && w->block.arrived == w->block.alive) {
          w->block.arrived = 0;
          w->block.gen++;
        }
      }
    }
    if (progress) continue;
    // Nothing can run.  The one legitimate case: a cross-lane operation inside a branch that only some lanes of the
    // wave took (the hardware runs it with a partial execution mask while the others wait at the join).  Such a wave
    // has lanes at a rendezvous and all its other lanes at the workgroup barrier; let the rendezvous go.
    bool released = false;
    for (int v = 0; v < nwaves && !released; ++v) {
      WaveState* ws = &w->waves[v];
      if (ws->arrived > 0 && ws->arrived < ws->alive) {
        complete_wave(ws);
        g_partial_rendezvous++;
        released = true;
      }
    }
    if (!released) {
      std::string msg = std::string("deadlock in ") + w->kernel + ": ";
      for (int i = 0; i < n && msg.size() < 400; ++i) {
        Fiber& f = w->fibers[i];
        if (f.done) continue;
        msg += "thread " + std::to_string(i) + (f.wait == Wait::kBlock ? " at barrier; " : " at rendezvous; ");
        i |= 63;  // one lane per wave is enough
      }
      log_error(msg);
      std::fprintf(stderr, "emu: %s\n", msg.c_str());
      std::abort();
    }
  }
}

// ---- worker pool ------------------------------------------------------------------------------------------------------------
struct Job {
  const char* name;
  dim3 grid, block;
  void (*tramp)(void*);
  void* closure;
  std::vector<dim3> blocks;
  std::atomic<size_t> next{0};
};

class Pool {
 public:
  static Pool& get() {
    static Pool* p = new Pool();  // never destroyed: the workers outlive static destruction
    return *p;
  }
  void run(Job* job) {
    if (threads_.empty()) {  // single-threaded configuration: the caller is the worker
      static thread_local Worker* w = new Worker();
      work(w, job);
      return;
    }
    std::unique_lock<std::mutex> lock(m_);
    job_ = job;
    pending_ = (int)threads_.size();
    ++epoch_;
    cv_.notify_all();
    done_cv_.wait(lock, [&] { return pending_ == 0; });
    job_ = nullptr;
  }

 private:
  Pool() {
    int n = g_threads;
    if (n <= 0) {
      const char* e = std::getenv("KSQ_EMU_THREADS");
      n = e ? std::atoi(e) : (int)std::min(8u, std::max(1u, std::thread::hardware_concurrency()));
    }
#if defined(KSQ_EMU_ASAN)
    n = 1;  // LDS is one plain static per kernel in that build
#endif
    if (n <= 1) return;
    for (int i = 0; i < n; ++i) threads_.emplace_back([this] { loop(); });
    for (auto& t : threads_) t.detach();
  }
  static void work(Worker* w, Job* job) {
    tl_worker = w;
    w->tramp = job->tramp;
    w->closure = job->closure;
    w->kernel = job->name;
    for (;;) {
      const size_t i = job->next.fetch_add(1);
      if (i >= job->blocks.size()) break;
      run_block(w, job->grid, job->block, job->blocks[i]);
    }
  }
  void loop() {
    Worker* w = new Worker();
    unsigned seen = 0;
    for (;;) {
      Job* job;
      {
        std::unique_lock<std::mutex> lock(m_);
        cv_.wait(lock, [&] { return epoch_ != seen; });
        seen = epoch_;
        job = job_;
      }
      work(w, job);
      {
        std::lock_guard<std::mutex> lock(m_);
        if (--pending_ == 0) done_cv_.notify_all();
      }
    }
  }
  std::mutex m_;
  std::condition_variable cv_, done_cv_;
  std::vector<std::thread> threads_;
  Job* job_ = nullptr;
  unsigned epoch_ = 0;
  int pending_ = 0;
};

}  // namespace

// ---- what the inline builtins call --------------------------------------------------------------------------------------------
int wave_rendezvous(int site, void (*fn)(WaveState*, int, int), int kind) {
  Worker* w = tl_worker;
  Fiber* f = w->running;
  WaveState* ws = f->ls.wave;
  const int slot = (int)(ws->gen & 1u);
  if (ws->arrived == 0) {
    ws->site = site;
    ws->fn = fn;
    ws->fn_kind = kind;
  } else if (ws->site != site) {
    const std::string msg = where(w, f->ls) + ": lanes of one wave meet at different cross-lane operations (lines " +
                            std::to_string(ws->site) + " and " + std::to_string(site) + ")";
    log_error(msg);
    std::fprintf(stderr, "emu: %s\n", msg.c_str());
    std::abort();
  }
  if (++ws->arrived == ws->alive) {
    complete_wave(ws);
    return slot;
  }
  f->wait = Wait::kWave;
  f->wait_gen = ws->gen;
  to_scheduler(w, f);
  return slot;
}

void block_barrier() {
  Worker* w = tl_worker;
  Fiber* f = w->running;
  if (++w->block.arrived == w->block.alive) {
    w->block.arrived = 0;
    w->block.gen++;
    return;
  }
  f->wait = Wait::kBlock;
  f->wait_gen = w->block.gen;
  to_scheduler(w, f);
}

Rsrc make_rsrc(const void* base, uint32_t num_records) {
  Rsrc r{static_cast<const char*>(base), num_records, 0, 0};
  if (num_records != 0) {
    if (const Alloc* a = find_alloc(reinterpret_cast<uintptr_t>(base))) {
      r.lo = a->lo;
      r.hi = a->hi;
    }
  }
  return r;
}

void report_oob(const char* what, const Rsrc& r, uint32_t voff, uint32_t soff, uint32_t bytes) {
  Worker* w = tl_worker;
  char buf[512];
  const uintptr_t a = reinterpret_cast<uintptr_t>(r.base) + voff + soff;
  if (r.lo == r.hi)
    std::snprintf(buf, sizeof(buf), "%s: %s of %u bytes passes the range check (voffset %u < num_records %u) but the "
                  "resource base %p is in no registered allocation (soffset %u)",
                  where(w, w->running->ls).c_str(), what, bytes, voff, r.num_records, (const void*)r.base, soff);
  else
    std::snprintf(buf, sizeof(buf), "%s: %s of %u bytes passes the range check (voffset %u, num_records %u, soffset %u) "
                  "but reads [%+ld, %+ld) relative to the end of its %zu-byte allocation",
                  where(w, w->running->ls).c_str(), what, bytes, voff, r.num_records, soff, (long)(a - r.hi),
                  (long)(a + bytes - r.hi), (size_t)(r.hi - r.lo));
  log_error(buf);
}

const void* symbol(const void* p, size_t bytes, const char* name) {
  register_range(reinterpret_cast<uintptr_t>(p), bytes, name);
  return p;
}

void launch_impl(const char* name, dim3 grid, dim3 block, void (*tramp)(void*), void* closure) {
  refresh_snapshot();
  static const bool trace = std::getenv("KSQ_EMU_TRACE") != nullptr;
  if (trace)
    std::fprintf(stderr, "emu: launch %s grid (%u,%u,%u) block %u\n", name, grid.x, grid.y, grid.z, block.x * block.y * block.z);
  Job job;
  job.name = name;
  job.grid = grid;
  job.block = block;
  job.tramp = tramp;
  job.closure = closure;
  // sampling keeps whole columns of grid.y (the split-K dimension of the kernels that hand tiles over between
  // workgroups: their arrival counters return to zero only when every split has run)
  const size_t positions = (size_t)grid.x * grid.z;
  const int sample = g_sample_blocks.load();
  std::vector<size_t> pick;
  if (sample <= 0 || positions <= (size_t)sample) {
    for (size_t i = 0; i < positions; ++i) pick.push_back(i);
  } else {
    for (int i = 0; i < sample; ++i) pick.push_back((size_t)((double)i * (double)(positions - 1) / (double)(sample - 1) + 0.5));
    pick.erase(std::unique(pick.begin(), pick.end()), pick.end());
  }
  for (size_t pos : pick)
    for (unsigned y = 0; y < grid.y; ++y) job.blocks.push_back(dim3((unsigned)(pos % grid.x), y, (unsigned)(pos / grid.x)));
  Pool::get().run(&job);
}

// ---- e4m3 (OCP "fn": bias 7, largest finite 448, no infinity, NaN = S.1111.111) ---------------------------------------------------
static float decode_e4m3(unsigned c) {
  const unsigned e = (c >> 3) & 15u, m = c & 7u;
  float v;
  if (e == 15 && m == 7) v = NAN;
  else if (e == 0) v = std::ldexp((float)m, -9);
  else v = std::ldexp(1.0f + (float)m / 8.0f, (int)e - 7);
  return (c & 0x80u) ? -v : v;
}
float e4m3_table[256];
namespace {
struct FillTable {
  FillTable() {
    for (unsigned c = 0; c < 256; ++c) e4m3_table[c] = decode_e4m3(c);
  }
} g_fill_table;
}  // namespace

// round to nearest even, saturating at +-448 (the callers clamp first; NaN stays NaN)
uint8_t f32_to_e4m3(float v) {
  uint32_t bits;
  std::memcpy(&bits, &v, 4);
  const uint8_t sign = (uint8_t)((bits >> 24) & 0x80u);
  const float a = std::fabs(v);
  if (std::isnan(v)) return (uint8_t)(sign | 0x7Fu);
  if (a >= 464.0f) return (uint8_t)(sign | 0x7Eu);  // at or above the midpoint between 448 and the next step
  if (a < 0.015625f) {                             // below the smallest normal 2^-6: steps of 2^-9
    const float q = std::nearbyint(a * 512.0f);   // default rounding mode: ties to even
    return (uint8_t)(sign | (uint8_t)q);           // q = 8 is the smallest normal's code
  }
  uint32_t ab = bits & 0x7FFFFFFFu;
  ab += 0x7FFFFu + ((ab >> 20) & 1u);  // round the 23-bit fraction to 3 bits, ties to even
  const int e = (int)(ab >> 23) - 127 + 7;
  const uint32_t m = (ab >> 20) & 7u;
  if (e > 15 || (e == 15 && m == 7)) return (uint8_t)(sign | 0x7Eu);
  return (uint8_t)(sign | (uint8_t)(e << 3) | (uint8_t)m);
}

// ---- matrix instructions: D = A x B for the whole wave, computed once by the lane that completes the rendezvous -----------
// Lane l = 16 j + c holds row c of A and column c of B for the k elements of its quarter j, and receives
// D[4 j + e][c], e = 0..3.  Both operands use the same lane -> k mapping, so only rows and columns matter here.
void mfma_collective(WaveState* w, int slot, int kind) {
  int per_lane;  // k elements per lane
  switch (kind) {
    case kMfmaF16:
    case kMfmaBf16:
    case kMfmaFp8x32: per_lane = 8; break;
    default: per_lane = 32; break;
  }
  static thread_local float A[16][128], B[16][128];
  const int K = 4 * per_lane;
  for (int l = 0; l < 64; ++l) {
    const int j = l >> 4, c = l & 15;
    const uint32_t* a = &w->x[slot][l][0];
    const uint32_t* b = &w->x[slot][l][8];
    for (int e = 0; e < per_lane; ++e) {
      float av, bv;
      if (kind == kMfmaF16) {
        const uint16_t ab = (uint16_t)(a[e >> 1] >> (16 * (e & 1))), bb = (uint16_t)(b[e >> 1] >> (16 * (e & 1)));
        _Float16 ah, bh;
        std::memcpy(&ah, &ab, 2);
        std::memcpy(&bh, &bb, 2);
        av = (float)ah;
        bv = (float)bh;
      } else if (kind == kMfmaBf16) {
        const uint32_t ab = (a[e >> 1] >> (16 * (e & 1))) << 16, bb = (b[e >> 1] >> (16 * (e & 1))) << 16;
        std::memcpy(&av, &ab, 4);
        std::memcpy(&bv, &bb, 4);
      } else {
        av = e4m3_table[(a[e >> 2] >> (8 * (e & 3))) & 0xFFu];
        bv = e4m3_table[(b[e >> 2] >> (8 * (e & 3))) & 0xFFu];
      }
      A[c][j * per_lane + e] = av;
      B[c][j * per_lane + e] = bv;
    }
  }
  for (int l = 0; l < 64; ++l) {
    if (!((w->alive_mask >> l) & 1)) continue;
    const int j = l >> 4, c = l & 15;
    for (int e = 0; e < 4; ++e) {
      const float* ar = A[4 * j + e];
      const float* bc = B[c];
      double s = 0.0;
      for (int k = 0; k < K; ++k) s += (double)ar[k] * (double)bc[k];
      const float f = (float)s;
      std::memcpy(&w->x[slot][l][e], &f, 4);
    }
  }
}

}  // namespace emu

// ---- host API ---------------------------------------------------------------------------------------------------------------------
extern "C" {

hipError_t hipGetDevice(int* dev) {
  *dev = 0;
  return hipSuccess;
}
hipError_t hipGetDeviceProperties(hipDeviceProp_t* prop, int) {
  const char* e = std::getenv("KSQ_EMU_CUS");
  prop->multiProcessorCount = e ? std::atoi(e) : 256;
  std::snprintf(prop->name, sizeof(prop->name), "emulated gfx950");
  return hipSuccess;
}
hipError_t hipGetLastError(void) { return hipSuccess; }
const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated error"; }
hipError_t hipMalloc(void** p, size_t bytes) {
  // 256-byte aligned like device allocations; the registered size is the exact one asked for
  if (posix_memalign(p, 256, bytes ? bytes : 1) != 0) return hipErrorInvalidValue;
  emu::register_range(reinterpret_cast<uintptr_t>(*p), bytes, "hipMalloc");
  return hipSuccess;
}
hipError_t hipFree(void* p) {
  if (p) emu::unregister_range(reinterpret_cast<uintptr_t>(p));
  std::free(p);
  return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t bytes, unsigned) {
  *p = std::malloc(bytes ? bytes : 1);
  return *p ? hipSuccess : hipErrorInvalidValue;
}
hipError_t hipHostFree(void* p) {
  std::free(p);
  return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, int) {
  std::memmove(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, int, hipStream_t) {
  std::memmove(dst, src, bytes);
  return hipSuccess;
}
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t) {
  std::memset(dst, value, bytes);
  return hipSuccess;
}

// ---- control surface for the tests ------------------------------------------------------------------------------------------------
// Tensors that kernels may touch through buffer resources are announced here (address, size); a later registration
// replaces whatever it overlaps.
void ksq_emu_register(const void* p, size_t bytes) { emu::register_range(reinterpret_cast<uintptr_t>(p), bytes, "tensor"); }
void ksq_emu_unregister(const void* p) { emu::unregister_range(reinterpret_cast<uintptr_t>(p)); }
void ksq_emu_clear_registry(void) {
  std::lock_guard<std::mutex> lock(emu::g_alloc_mutex);
  emu::g_allocs.erase(std::remove_if(emu::g_allocs.begin(), emu::g_allocs.end(),
                                     [](const emu::Alloc& a) { return a.tag == "tensor"; }),
                      emu::g_allocs.end());
  emu::g_alloc_version++;
}
// 0: run every workgroup; n > 0: run about n positions of grid.x * grid.z (first and last included), all of grid.y
void ksq_emu_set_block_sample(int n) { emu::g_sample_blocks = n; }
long ksq_emu_error_count(void) { return emu::g_error_count.load(); }
long ksq_emu_partial_rendezvous_count(void) { return emu::g_partial_rendezvous.load(); }
// i-th logged error (at most 64 are kept), or "" past the end
const char* ksq_emu_error_string(int i) {
  static thread_local std::string s;
  std::lock_guard<std::mutex> lock(emu::g_log_mutex);
  s = (i >= 0 && (size_t)i < emu::g_errors.size()) ? emu::g_errors[(size_t)i] : "";
  return s.c_str();
}
void ksq_emu_clear_errors(void) {
  std::lock_guard<std::mutex> lock(emu::g_log_mutex);
  emu::g_errors.clear();
  emu::g_error_count = 0;
}

}  // extern "C"

// A standalone test program that links the emulated library has no caller to ask for the error log: with
// KSQ_EMU_EXIT_CODE_ON_ERROR=<code> in the environment the process prints the log and ends with that code if anything
// was reported.
namespace {
struct ExitReport {
  ~ExitReport() {
    const char* e = std::getenv("KSQ_EMU_EXIT_CODE_ON_ERROR");
    if (!e || emu::g_error_count.load() == 0) return;
    std::fprintf(stderr, "emu: %ld out-of-bounds accesses reported\n", emu::g_error_count.load());
    for (const std::string& m : emu::g_errors) std::fprintf(stderr, "emu: %s\n", m.c_str());
    std::fflush(nullptr);
    _Exit(std::atoi(e));
  }
} g_exit_report;
}  // namespace
