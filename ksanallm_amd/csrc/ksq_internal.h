// Internal declarations shared by the HIP translation units of libksq.so (not installed).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "ksq.h"

namespace ksq {

// ---- error plumbing (thread-local message behind ksq_last_error_string) -------------------------------------
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define KSQ_HIP_TRY(expr)                                                                      \
  do {                                                                                         \
    hipError_t e__ = (expr);                                                                   \
    if (e__ != hipSuccess) return ::ksq::fail(KSQ_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e__)); \
  } while (0)

#define KSQ_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) return ::ksq::fail((code), __VA_ARGS__); \
  } while (0)

// ---- launch log ----------------------------------------------------------------------------------------------------
// What the last GEMM entry point on this thread launched (kernel, template arguments, grid), for ksq_last_launch_string;
// a no-op unless ksq_set_launch_log(1) was called, so the launch path of a serving process formats nothing.
void note_launch(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void reset_launch_note();  // at the top of every GEMM entry point

// ---- tuning / test overrides -------------------------------------------------------------------------------
// The launch planners can be overridden through KSQ_* environment variables.  They are looked up only in a process
// that had KSQ_TUNING=1 in its environment when the library was first used: otherwise this returns nullptr without
// touching the environment, so the launch path of a serving process makes no getenv calls.
const char* tuning_env(const char* name);

// ---- fragment-order geometry -------------------------------------------------------------------------------
constexpr int kTileN = 16;        // columns per weight tile
constexpr int kTileK = 128;       // k per weight tile
constexpr int kTileWords = 256;   // 32-bit words per tile (64 lanes x 4)

// Position of logical element (k, n) in the fragment-order weight buffer: index of the 32-bit word and the
// nibble inside it.  Tiles are [N/16][K/128]; see include/ksq.h for the definition this implements.
__host__ __device__ inline void frag_position(size_t k, size_t n, size_t K, size_t* word, int* nibble) {
  size_t nt = n / kTileN, kt = k / kTileK;
  int c = (int)(n % kTileN);
  int kk = (int)(k % kTileK);
  int d = kk >> 5;        // which of the four MFMAs of the tile
  int j = (kk >> 3) & 3;  // k sub-group = lane / 16
  int e = kk & 7;
  int lane = 16 * j + c;
  *word = ((nt * (K / kTileK) + kt) * 64 + (size_t)lane) * 4 + (size_t)d;
  *nibble = (e & 1) ? 4 + (e >> 1) : (e >> 1);
}

// Inverse for one output word: which (k0, n) the word's eight elements start at.
__host__ __device__ inline void frag_word_origin(size_t word, size_t K, size_t* k0, size_t* n) {
  size_t d = word & 3;
  size_t lane = (word >> 2) & 63;
  size_t tile = word >> 8;
  size_t KT = K / kTileK;
  size_t nt = tile / KT, kt = tile % KT;
  *n = nt * kTileN + (lane & 15);
  *k0 = kt * kTileK + 32 * d + 8 * (lane >> 4);
}

// element e (0..7) of a fragment word lives in this nibble
__host__ __device__ inline int frag_nibble_of(int e) { return (e & 1) ? 4 + (e >> 1) : (e >> 1); }

// ---- split-K bookkeeping -----------------------------------------------------------------------------------
// Arrival counters of the split-K fix-up.  They live in library-owned device memory (zero at load, returned
// to zero by the last-arriving wave of every tile), so no launch has to clear anything.  Every stream that launches
// a split-K kernel owns one of kCounterSlots regions for good: launches on one stream run one after the other, so
// they never share counters with a launch still in flight.  A device's first kCounterSlots streams get a region;
// for any later stream this returns nullptr and the caller plans without a split across workgroups.
constexpr int kCounterSlots = 64;
constexpr int kCountersPerSlot = 16384;
unsigned* counter_slot_device_ptr(hipStream_t stream);  // the stream's region (device address) or nullptr
bool counter_slot_available(hipStream_t stream);        // the same answer without claiming a region
static_assert(kCountersPerSlot * 4 == KSQ_SPLITK_COUNTER_BYTES, "ksq.h states the size of a counter region");

// ---- the few places where the kernels speak to the compiler or the machine in assembly ----------------------------------
// A host build of the kernels (the CPU emulation that the tests use to walk every kernel's addressing, KSQ_EMU) has
// neither register classes nor wait counters; everything else in the kernels is plain C++ plus builtins.
#if defined(KSQ_EMU)
#define KSQ_PIN_SGPR(x) ((void)(x))
#define KSQ_PIN_VGPR(x) ((void)(x))
#define KSQ_WAIT_ALL_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)  // where the emulated lanes of a wave meet
#else
// keeps a constant in a scalar / vector register instead of rematerialising it as a literal at every use
#define KSQ_PIN_SGPR(x) asm volatile("" : "+s"(x))
#define KSQ_PIN_VGPR(x) asm volatile("" : "+v"(x))
#define KSQ_WAIT_ALL_VMEM() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#endif

#if defined(__HIPCC__)
// Split-K partial tiles cross workgroups (and XCDs, each with its own L2) through agent-scope relaxed atomics: the
// stores write through and the loads miss the non-coherent caches, so no whole-cache write-back or invalidate is
// needed around the arrival counter (splitk_arrive_last below).
typedef float ksq_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long ksq_u64x2 __attribute__((ext_vector_type(2)));

__device__ inline void store_agent(ksq_f32x4* p, ksq_f32x4 v) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(p);
  ksq_u64x2 w = __builtin_bit_cast(ksq_u64x2, v);
  __hip_atomic_store(q, w[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(q + 1, w[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ inline ksq_f32x4 load_agent(const ksq_f32x4* p) {
  unsigned long long* q = reinterpret_cast<unsigned long long*>(const_cast<ksq_f32x4*>(p));
  ksq_u64x2 w;
  w[0] = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  w[1] = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __builtin_bit_cast(ksq_f32x4, w);
}

// Units [begin, end) of split `split` of `ksplit` over `total` k units: floor(total * split / ksplit) and the same for
// split + 1.  One split, the common case, costs nothing.  Otherwise 32-bit divisions; a 64-bit one is some 150 scalar
// instructions, and two of them in front of a wave's first load show in a kernel that lasts a few microseconds.  The
// quotients come from the vector unit and are uniform: readfirstlane says so (a value that crosses a basic block in a
// vector register otherwise counts as divergent, and loads whose scalar offset derives from it get wrapped in loops).
__device__ inline void split_range(int total, int split, int ksplit, int* begin, int* end) {
  if (ksplit <= 1) {
    *begin = 0;
    *end = total;
  } else if (total < (1 << 26)) {  // ksplit <= 32: the products fit
    *begin = __builtin_amdgcn_readfirstlane((int)((unsigned)(total * split) / (unsigned)ksplit));
    *end = __builtin_amdgcn_readfirstlane((int)((unsigned)(total * (split + 1)) / (unsigned)ksplit));
  } else {
    *begin = __builtin_amdgcn_readfirstlane((int)(((long)total * split) / ksplit));
    *end = __builtin_amdgcn_readfirstlane((int)(((long)total * (split + 1)) / ksplit));
  }
}

// A wave that has parked its partial tile (store_agent) arrives at the tile's counter; every lane makes the call.
// Returns true, in every lane, in the wave that finds the count complete: that wave then reads all splits' tiles
// (load_agent).  Ordering: the tile's stores are agent-scope atomics, performed beyond the XCD's L2, and
// `s_waitcnt vmcnt(0)` holds the wave until every one of them is acknowledged, so the increment is issued after they
// are visible device-wide; the reader's loads are agent-scope atomics too and are issued after its own increment has
// returned.  The portable form -- a release fence before the increment and an acquire fence after it, agent scope
// -- was built and measured: on this device it writes back and invalidates the XCD's whole L2 around every tile
// (Llama-2-7B o at M = 64 10.6 -> 31.7 us, down at M = 16 11.0 -> 15.2 us, Qwen-72B FP8 gate_up at M = 64 137 ->
// 1432 us), so the hand-over stays with the atomics and the wait.
__device__ inline bool splitk_arrive_last(unsigned* counter, int lane, int ksplit) {
  KSQ_WAIT_ALL_VMEM();
  unsigned arrived = 0;
  if (lane == 0) arrived = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  arrived = __builtin_amdgcn_readfirstlane(arrived);
  asm volatile("" ::: "memory");
  return arrived == (unsigned)(ksplit - 1);
}
#endif

// ---- workgroup id -> output tile, for the kernels that tile the whole [M, N] output ------------------------------
// A grid of mblocks x nblocks tiles is launched as exactly that many workgroups, rounded up to a multiple of eight:
// no workgroup is launched only to find that it has no tile (a regular pattern of such workgroups -- seven of eight
// with one row block padded to a band of eight -- was measured to leave seven of eight compute units without work,
// because consecutive workgroups go to consecutive compute units).  Hardware hands consecutive workgroup ids to the
// 8 XCDs in turn; every XCD (own L2) gets a contiguous run of logical ids.  Logical ids walk bands of eight row
// blocks, column block by column block and down the band's row blocks first (the last band is as high as what is
// left), so the workgroups resident on an XCD at one time share at most eight activation row blocks and a few
// neighbouring column blocks of the weights.
inline unsigned tile_grid(size_t mblocks, size_t nblocks) { return (unsigned)((mblocks * nblocks + 7) / 8 * 8); }
#if defined(__HIPCC__)
__device__ inline int tile_logical_id(int block, int grid) { return (block & 7) * (grid >> 3) + (block >> 3); }
#endif
__host__ __device__ inline bool tile_of(int lid, int mblocks, int nblocks, int* mb, int* nb) {
  if (lid >= mblocks * nblocks) return false;
  const int band = lid / (8 * nblocks);
  const int left = mblocks - 8 * band, h = left < 8 ? left : 8;
  const int idx = lid - band * 8 * nblocks;
  *nb = idx / h;
  *mb = 8 * band + (idx - *nb * h);
  return true;
}

// out [m][k_out] = in [m][k_in] followed by zeros, 16-bit elements, k_in and k_out multiples of 8 (ksq_repack.hip)
int pad_rows(void* out, const void* in, size_t m, size_t k_in, size_t k_out, hipStream_t s);

struct DeviceInfo {
  int cus;
};
const DeviceInfo* device_info();  // of the current device; nullptr on failure

// What a GEMM does with its fp32 result on the way out (ksq_epilogue in include/ksq.h).
struct Epilogue {
  int kind = KSQ_EPILOGUE_NONE;
  const void* bias = nullptr;  // T [n], 16-byte aligned
  float* row_absmax = nullptr;  // [m]: largest |stored value| per row, merged in by atomic maximum (or none)
};

// ---- launch plans ------------------------------------------------------------------------------------------
struct W4Plan {
  int MT;       // 16-row tiles per wave (1..4)
  int NT;       // 16-column tiles per wave
  int mblocks;  // grid.z
  int ksplit;   // grid.y
  int slices;   // k slices inside one workgroup (4 waves each)
  size_t partial_bytes;  // workspace the plan needs (0 when ksplit == 1)
  bool prefill;  // true: LDS-tiled MFMA kernel, false: streaming kernel
};
W4Plan w4a16_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes);
W4Plan w4a16_plan_with(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, int nt, int ks);

int w4a16_launch_stream(int dtype, const W4Plan& plan, void* out, const void* act, const void* weight,
                        const void* sz, size_t m, size_t n, size_t k, size_t g, void* workspace, hipStream_t s,
                        const Epilogue& epi = Epilogue());
struct PrefillPlan {
  int rows;    // rows per workgroup tile: 64 or 128
  int knt;     // 64-row kernel: column tiles per wave (1, 2 or 4)
  int nw;      // 128-row kernel: waves side by side (4 or 8)
  int kg;      // 128-row kernel with four waves side by side: k groups of such waves (1 or 2)
  int ct;      // 128-row kernel: column tiles per wave (1 to 4: 16 to 64 columns)
  int ksplit;  // grid.y: K split over workgroups
  size_t partial_bytes;
};
PrefillPlan w4a16_prefill_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes);
int w4a16_launch_prefill(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m,
                         size_t n, size_t k, size_t g, void* workspace, size_t workspace_bytes, hipStream_t s,
                         const Epilogue& epi = Epilogue());
size_t w4a16_prefill_workspace_bytes(int dtype, size_t m, size_t k);
bool w4a16_prefill_supported(int dtype, size_t m, size_t n, size_t k, size_t g, int cus);
int w4a16_stream_max_slices(int mt, int nt);

struct KstatPlan {
  bool ok;       // the k-stationary decode kernel takes this shape (m <= 64)
  int mt;        // 16-row tiles (1, 2 or 4)
  int nw;        // waves per workgroup (16 or 8)
  int tpw;       // k tiles per wave
  int ksplit;    // grid.y
  int nt_per_wg; // column tiles per workgroup
  int grid_x;
  int nb;        // column tiles per batch (= ring depth / tpw)
  bool phases;   // K walked in phases inside the workgroup (w4a16_kphase_kernel) instead of split over grid.y
  size_t partial_bytes;
};
// g = the group size where the caller knows it (it picks the batch size only; the workspace a plan needs does not
// depend on it)
KstatPlan w4a16_kstat_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, size_t g = 0);
int w4a16_launch_kstat(int dtype, const KstatPlan& plan, void* out, const void* act, const void* weight,
                       const void* sz, size_t m, size_t n, size_t k, size_t g, void* workspace, hipStream_t s,
                        const Epilogue& epi = Epilogue());

// accumulator-stationary decode kernel for 17 <= m <= 64
struct AstreamPlan {
  int mt;      // 16-row tiles (2 or 4)
  int ksplit;  // grid.y
  size_t partial_bytes;
};
bool w4a16_astream_supported(size_t m, size_t n, size_t k);
AstreamPlan w4a16_astream_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes);
int w4a16_launch_astream(int dtype, const AstreamPlan& plan, void* out, const void* act, const void* weight,
                         const void* sz, size_t m, size_t n, size_t k, size_t g, int cus, void* workspace,
                         hipStream_t s, const Epilogue& epi = Epilogue());

struct Fp8KstatPlan {
  bool ok;        // the k-stationary kernel takes this shape (m <= 64)
  int mt;         // 16-row tiles (1, 2 or 4)
  int tpw;        // 128-byte k stages per wave (16 waves per workgroup)
  int ksplit;     // grid.y
  int nt_per_wg;  // column tiles per workgroup
  int grid_x;
  int nb;         // column tiles per batch
  bool phases;    // K walked in phases inside the workgroup (fp8_kphase_kernel) instead of split over grid.y
  size_t partial_bytes;
};
// `fused`: plan for the kernel that quantises its own activations (m <= 8)
Fp8KstatPlan fp8_kstat_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, bool fused = false);
// act_src != nullptr: the activations as 16-bit elements of the output type, quantised per token inside the kernel
// (act_q / act_scale unused); needs a plan made with `fused`
int fp8_launch_kstat(int out_dtype, const Fp8KstatPlan& plan, void* out, const void* act_q, const float* act_scale,
                     size_t act_scale_count, const void* w_q, const float* w_scale, size_t w_scale_count, size_t m,
                     size_t n, size_t k, void* workspace, hipStream_t s, const Epilogue& epi = Epilogue(),
                     const void* act_src = nullptr);

struct Fp8Plan {
  int MT;
  int mblocks;
  int ksplit;
  size_t partial_bytes;
  bool prefill;
};
Fp8Plan fp8_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes);
bool fp8_prefill_supported(size_t m, size_t n, size_t k, int cus);
size_t fp8_prefill_workspace_bytes(size_t m, size_t n, size_t k, int cus);  // partial tiles of a split last round
int fp8_launch_prefill(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                       const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                       void* workspace, size_t workspace_bytes, hipStream_t s, const Epilogue& epi = Epilogue());

}  // namespace ksq
