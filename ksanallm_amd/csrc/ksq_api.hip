// C-ABI entry points of libksq.so: argument validation, launch planning, error plumbing.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "ksq_internal.h"

namespace ksq {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

static std::atomic<int> g_launch_log{0};
static thread_local char g_launch[384] = "";

void note_launch(const char* fmt, ...) {
  if (!g_launch_log.load(std::memory_order_relaxed)) return;
  const size_t used = strlen(g_launch);
  if (used + 2 >= sizeof(g_launch)) return;
  if (used) {  // several launches behind one entry point: "a + b"
    memcpy(g_launch + used, " + ", 4);
  }
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_launch + strlen(g_launch), sizeof(g_launch) - strlen(g_launch), fmt, ap);
  va_end(ap);
}
void reset_launch_note() { g_launch[0] = 0; }

// ---- per-device state -----------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned g_splitk_counters[kCounterSlots * kCountersPerSlot];
// Scratch of ksq_w4a16_gemm_static_scratch: stands in for the caller's workspace.  In host code this name is only a
// handle for hipGetSymbolAddress; the address kept per device below is what kernels and copies get.
static __device__ __align__(256) unsigned char g_static_scratch[KSQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 16;
constexpr int kMaxBoundStreams = 256;
struct PerDevice {
  std::once_flag once;
  bool ok = false;
  DeviceInfo info{};
  unsigned* counters = nullptr;
  unsigned char* static_scratch = nullptr;
  std::mutex slot_mutex;
  int slots_used = 0;
  hipStream_t slot_owner[kCounterSlots] = {};
  int bound_used = 0;  // caller-owned counters, by stream (ksq_bind_splitk_counters)
  hipStream_t bound_stream[kMaxBoundStreams] = {};
  unsigned* bound_ptr[kMaxBoundStreams] = {};
};
PerDevice g_dev[kMaxDevices];

PerDevice* current_device_state() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(KSQ_ERR_HIP, "hipGetDevice failed or device index out of range");
    return nullptr;
  }
  PerDevice* pd = &g_dev[dev];
  std::call_once(pd->once, [pd, dev]() {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return;
    pd->info.cus = prop.multiProcessorCount;
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_splitk_counters)) != hipSuccess || p == nullptr) return;
    pd->counters = static_cast<unsigned*>(p);
    void* q = nullptr;
    if (hipGetSymbolAddress(&q, HIP_SYMBOL(g_static_scratch)) != hipSuccess || q == nullptr) return;
    pd->static_scratch = static_cast<unsigned char*>(q);
    pd->ok = true;
  });
  if (!pd->ok) {
    fail(KSQ_ERR_HIP, "device %d: could not query properties or resolve the library's device arrays", dev);
    return nullptr;
  }
  return pd;
}
}  // namespace

const DeviceInfo* device_info() {
  PerDevice* pd = current_device_state();
  return pd ? &pd->info : nullptr;
}

// A stream's counters: the caller's own (ksq_bind_splitk_counters) if it bound any, else the stream's region of the
// library's array, claimed on first use.
unsigned* counter_slot_device_ptr(hipStream_t stream) {
  PerDevice* pd = current_device_state();
  if (!pd) return nullptr;
  std::lock_guard<std::mutex> lock(pd->slot_mutex);
  for (int i = 0; i < pd->bound_used; ++i)
    if (pd->bound_stream[i] == stream && pd->bound_ptr[i]) return pd->bound_ptr[i];
  int slot = 0;
  while (slot < pd->slots_used && pd->slot_owner[slot] != stream) ++slot;
  if (slot == pd->slots_used) {
    if (slot == kCounterSlots) return nullptr;  // every region has an owner: this stream runs without split-K
    pd->slot_owner[pd->slots_used++] = stream;
  }
  return pd->counters + (size_t)slot * kCountersPerSlot;
}

// Whether counter_slot_device_ptr would succeed, without claiming a region: the planners ask before they plan a split,
// the launchers claim when a split is in the plan, so a stream that never splits never owns a region.
bool counter_slot_available(hipStream_t stream) {
  PerDevice* pd = current_device_state();
  if (!pd) return false;
  std::lock_guard<std::mutex> lock(pd->slot_mutex);
  for (int i = 0; i < pd->bound_used; ++i)
    if (pd->bound_stream[i] == stream && pd->bound_ptr[i]) return true;
  for (int slot = 0; slot < pd->slots_used; ++slot)
    if (pd->slot_owner[slot] == stream) return true;
  return pd->slots_used < kCounterSlots;
}

static int bind_counters(hipStream_t stream, unsigned* counters) {
  PerDevice* pd = current_device_state();
  if (!pd) return KSQ_ERR_HIP;
  std::lock_guard<std::mutex> lock(pd->slot_mutex);
  int i = 0;
  while (i < pd->bound_used && pd->bound_stream[i] != stream) ++i;
  if (i == pd->bound_used) {
    if (counters == nullptr) return KSQ_OK;  // nothing bound: nothing to undo
    int free_i = 0;
    while (free_i < pd->bound_used && pd->bound_ptr[free_i]) ++free_i;  // reuse an unbound entry
    i = free_i;
    if (i == kMaxBoundStreams) return fail(KSQ_ERR_UNSUPPORTED, "%d streams already have counters bound", kMaxBoundStreams);
    if (i == pd->bound_used) ++pd->bound_used;
    pd->bound_stream[i] = stream;
  }
  pd->bound_ptr[i] = counters;
  return KSQ_OK;
}

static unsigned char* static_scratch_device_ptr() {
  PerDevice* pd = current_device_state();
  return pd ? pd->static_scratch : nullptr;
}

const char* tuning_env(const char* name) {
  static const bool enabled = [] {
    const char* e = getenv("KSQ_TUNING");
    return e && atoi(e) != 0;
  }();
  return enabled ? getenv(name) : nullptr;
}

static int env_int(const char* name, int dflt) {
  const char* v = tuning_env(name);
  if (!v || !*v) return dflt;
  return atoi(v);
}

// ---- launch planning ------------------------------------------------------------------------------------------
// The streaming kernel gives every wave NT column tiles x a contiguous range of k tiles and keeps D tiles per
// column tile in flight.  What bounds it on narrow N is the number of bytes in flight, i.e. the number of waves:
// about one wave per SIMD (4 per CU) is needed before HBM latency is covered.  Splitting k across workgroups
// (grid.y) buys those waves at the price of fp32 partial tiles written and read once each plus three dependent
// trips to device memory (~3 us measured), so it is used only when the column tiles alone give fewer than one wave
// per SIMD, and it is bounded by the workspace and by a traffic budget relative to the weight bytes.  k can also
// be sliced inside a workgroup (reduced through LDS); measured slower than one slice on MI355X for the decode
// shapes, so it is off by default (KSQ_W4_SLICES selects it).
W4Plan w4a16_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes) {
  return w4a16_plan_with(m, n, k, cus, workspace_bytes, 0, 0);
}

// nt / ks: column tiles per wave and K splits asked for (0 = the planner's own choice); the split still shrinks to
// what the workspace holds
W4Plan w4a16_plan_with(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, int nt, int ks) {
  W4Plan p{};
  const size_t ntiles = n / kTileN, ktiles = k / kTileK;
  const size_t simds = (size_t)cus * 4;
  p.prefill = false;
  if (m <= 64) {
    p.MT = (int)((m + 15) / 16);
    p.mblocks = 1;
    p.NT = (p.MT >= 2 || ntiles >= simds) ? 2 : 1;
  } else {
    p.MT = 4;
    p.mblocks = (int)((m + 63) / 64);
    p.NT = 2;
  }
  if (nt == 1 || nt == 2 || nt == 4) p.NT = nt;
  int nt_env = env_int("KSQ_W4_NT", 0);
  if (nt_env == 1 || nt_env == 2 || nt_env == 4) p.NT = nt_env;
  p.slices = 1;
  int sl_env = env_int("KSQ_W4_SLICES", 0);
  const int max_slices = m <= 64 ? w4a16_stream_max_slices(p.MT, p.NT) : 1;
  if (sl_env == 1 || (sl_env == 2 && max_slices >= 2) || (sl_env == 4 && max_slices >= 4)) p.slices = sl_env;
  const size_t ngroups = (ntiles + p.NT - 1) / p.NT;
  size_t ksplit = 1;
  if (m <= 64) {
    size_t wanted = simds / ngroups;  // waves per split = ngroups
    const size_t mpad = (size_t)p.MT * 16;
    size_t cap = k / (32 * mpad);  // partial write + read <= 50% of the weight bytes
    if (cap > ktiles / 4) cap = ktiles / 4;  // at least four k tiles per wave
    if (wanted > cap) wanted = cap;
    if (wanted < 1) wanted = 1;
    ksplit = wanted;
    if (ks >= 1 && (size_t)ks <= ktiles) ksplit = (size_t)ks;
    int ks_env = env_int("KSQ_W4_KSPLIT", 0);
    if (ks_env >= 1 && (size_t)ks_env <= ktiles) ksplit = (size_t)ks_env;
    if (ngroups * (size_t)p.mblocks > (size_t)kCountersPerSlot) ksplit = 1;
  }
  auto need = [&](size_t ks) { return ks <= 1 ? (size_t)0 : ks * (size_t)p.mblocks * ntiles * p.MT * 64 * 16; };
  while (ksplit > 1 && need(ksplit) > workspace_bytes) --ksplit;
  p.ksplit = (int)ksplit;
  p.partial_bytes = need(ksplit);
  return p;
}

Fp8Plan fp8_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes) {
  Fp8Plan p{};
  const size_t ntiles = (n + 15) / 16, kblocks = k / 64;
  p.prefill = false;
  if (m <= 64) {
    p.MT = (int)((m + 15) / 16);
    p.mblocks = 1;
  } else {
    p.MT = 4;
    p.mblocks = (int)((m + 63) / 64);
  }
  const size_t wgs = ((ntiles + 3) / 4) * (size_t)p.mblocks;
  size_t ksplit = 1;
  if (m <= 64) {
    const size_t target = (size_t)cus * 4;
    ksplit = (target + wgs / 2) / wgs;
    const size_t mpad = (size_t)p.MT * 16;
    size_t traffic_cap = k / (32 * mpad);  // partial write+read <= 25% of the weight bytes
    if (ksplit > traffic_cap) ksplit = traffic_cap;
    if (ksplit > kblocks / 4) ksplit = kblocks / 4;
    if (ksplit > 16) ksplit = 16;
    if (ksplit < 1) ksplit = 1;
    int ks_env = env_int("KSQ_FP8_KSPLIT", 0);
    if (ks_env >= 1 && (size_t)ks_env <= kblocks) ksplit = (size_t)ks_env;
    if (ntiles * (size_t)p.mblocks > (size_t)kCountersPerSlot) ksplit = 1;
  }
  auto need = [&](size_t ks) { return ks <= 1 ? (size_t)0 : ks * (size_t)p.mblocks * ntiles * p.MT * 64 * 16; };
  while (ksplit > 1 && need(ksplit) > workspace_bytes) --ksplit;
  p.ksplit = (int)ksplit;
  p.partial_bytes = need(ksplit);
  return p;
}

}  // namespace ksq

using namespace ksq;

extern "C" {

int ksq_version(void) { return 100; }

const char* ksq_last_error_string(void) { return g_error; }

void ksq_set_launch_log(int enabled) { g_launch_log.store(enabled ? 1 : 0); }

const char* ksq_last_launch_string(void) { return g_launch; }

int ksq_bind_splitk_counters(void* stream, void* counters, size_t bytes) {
  KSQ_REQUIRE(counters == nullptr || bytes >= (size_t)KSQ_SPLITK_COUNTER_BYTES, KSQ_ERR_INVALID_ARGUMENT,
              "%zu bytes of counters; %zu are needed", bytes, (size_t)KSQ_SPLITK_COUNTER_BYTES);
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(counters) & 255) == 0, KSQ_ERR_INVALID_ARGUMENT,
              "counters must be 256-byte aligned");
  return bind_counters(static_cast<hipStream_t>(stream), static_cast<unsigned*>(counters));
}

int ksq_device_compute_units(void) {
  const DeviceInfo* di = device_info();
  return di ? di->cus : 0;
}

static int check_w4_shape(size_t k, size_t n, size_t g) {
  KSQ_REQUIRE(k > 0 && n > 0, KSQ_ERR_INVALID_ARGUMENT, "k and n must be positive (k=%zu n=%zu)", k, n);
  // the reference kernels accept group sizes 64 and 128 only (LK/asymmetric_gemm/fpA_intB_gemm/
  // fpA_intB_gemm_template.h:130) and k % 64 == 0 (:168-171); the fragment order needs whole 128 x 16 tiles
  KSQ_REQUIRE(g == 64 || g == 128, KSQ_ERR_UNSUPPORTED, "group size %zu not supported (64 or 128)", g);
  KSQ_REQUIRE(k % g == 0, KSQ_ERR_UNSUPPORTED, "k=%zu must be a multiple of the group size %zu", k, g);
  KSQ_REQUIRE(n % kTileN == 0, KSQ_ERR_UNSUPPORTED, "n=%zu must be a multiple of %d", n, kTileN);
  KSQ_REQUIRE(k < (1u << 30) && n < (1u << 30), KSQ_ERR_UNSUPPORTED, "k or n too large");
  return KSQ_OK;
}

int ksq_w4a16_repack_sizes(size_t k, size_t n, size_t g, size_t* weight_bytes, size_t* sz_bytes) {
  int rc = check_w4_shape(k, n, g);
  if (rc != KSQ_OK) return rc;
  KSQ_REQUIRE(weight_bytes && sz_bytes, KSQ_ERR_INVALID_ARGUMENT, "null output pointer");
  const size_t kp = (k + kTileK - 1) / kTileK * kTileK;  // an odd multiple of 64 (g = 64) is padded to whole k tiles
  *weight_bytes = kp * n / 2;
  *sz_bytes = (kp / g) * n * 4;
  return KSQ_OK;
}

// the copy of the activations with rows padded to whole k tiles, in front of the workspace, when k % 128 == 64
static size_t padded_act_bytes(size_t m, size_t k) {
  return k % kTileK == 0 ? 0 : (m * (k + 64) * 2 + 255) / 256 * 256;
}

int ksq_w4a16_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes) {
  KSQ_REQUIRE(bytes, KSQ_ERR_INVALID_ARGUMENT, "null output pointer");
  KSQ_REQUIRE(max_m > 0, KSQ_ERR_INVALID_ARGUMENT, "max_m must be positive");
  if (k % kTileK == 64) {  // group size 64: planned on the padded K, plus the padded copy of the activations
    int rcp = ksq_w4a16_workspace_bytes(max_m, n, k + 64, bytes);
    if (rcp == KSQ_OK) *bytes += padded_act_bytes(max_m, k);
    return rcp;
  }
  int rc = check_w4_shape(k, n, 128);
  if (rc != KSQ_OK) return rc;
  const DeviceInfo* di = device_info();
  const int cus = di ? di->cus : 256;  // sizing only; without a device assume a full MI355X
  size_t best = 0;
  const size_t ms[4] = {16, 32, 48, 64};
  for (size_t mm : ms) {
    if (mm - 15 > max_m) break;
    W4Plan p = w4a16_plan(mm, n, k, cus, (size_t)-1);
    if (p.partial_bytes > best) best = p.partial_bytes;
    if (mm == 16) {  // the four-way split of the streaming kernel that a very long K is routed to at 9 .. 16 rows
      const W4Plan lp = w4a16_plan_with(mm, n, k, cus, (size_t)-1, 2, 4);
      if (lp.partial_bytes > best) best = lp.partial_bytes;
    }
    KstatPlan kp = w4a16_kstat_plan(mm < max_m ? mm : max_m, n, k, cus, (size_t)-1);
    if (kp.ok && kp.partial_bytes > best) best = kp.partial_bytes;
    const size_t am = mm < max_m ? mm : max_m;
    if (w4a16_astream_supported(am, n, k)) {
      const AstreamPlan ap = w4a16_astream_plan(am, n, k, cus, (size_t)-1);
      if (ap.partial_bytes > best) best = ap.partial_bytes;
    }
  }
  if (max_m >= 33) {  // the large-M kernels serve 33 rows and more where the shape suits them
    // the element type is not known here: size for the bf16 route of the prefill kernel, plus the largest set of
    // split-K partial tiles any m up to max_m asks for
    size_t partial = 0;
    // (the forms are chosen by an estimate in which the partial tiles count by their rows, so the plan can differ
    // between the first and the last row count of a block: both are asked)
    for (size_t mb = 1; mb <= (max_m + 63) / 64 && mb <= 2 * (size_t)cus; ++mb) {
      for (size_t mm : {(mb - 1) * 64 + 1, mb * 64 < max_m ? mb * 64 : max_m}) {
        const PrefillPlan pp = w4a16_prefill_plan(mm, n, k, cus, (size_t)-1);
        if (pp.partial_bytes > partial) partial = pp.partial_bytes;
      }
    }
    const size_t pf = w4a16_prefill_workspace_bytes(KSQ_BF16, max_m, k) + partial;
    if (pf > best) best = pf;
  }
  *bytes = best;
  return KSQ_OK;
}

int ksq_w4a16_workspace_bytes_ex(size_t max_m, size_t n, size_t k, int act_order, size_t* bytes) {
  int rc = ksq_w4a16_workspace_bytes(max_m, n, k, bytes);
  if (rc != KSQ_OK) return rc;
  if (act_order) *bytes += (max_m * k * 2 + 255) / 256 * 256;  // the permuted copy of the activations, in front
  return KSQ_OK;
}

static int w4a16_gemm_impl(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                           size_t k, size_t g, const int32_t* act_perm, int epilogue, const void* bias,
                           float* row_absmax, void* workspace, size_t workspace_bytes, void* stream) {
  reset_launch_note();
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(out && act && weight && sz, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(epilogue >= KSQ_EPILOGUE_NONE && epilogue <= KSQ_EPILOGUE_SILU_MUL, KSQ_ERR_INVALID_ARGUMENT,
              "bad epilogue %d", epilogue);
  KSQ_REQUIRE(epilogue != KSQ_EPILOGUE_BIAS || (bias && (reinterpret_cast<uintptr_t>(bias) & 15) == 0),
              KSQ_ERR_INVALID_ARGUMENT, "the bias epilogue needs a 16-byte aligned bias");
  int rc = check_w4_shape(k, n, g);
  if (rc != KSQ_OK) return rc;
  if (m == 0) return KSQ_OK;
  KSQ_REQUIRE(m < (1u << 24), KSQ_ERR_UNSUPPORTED, "m=%zu too large", m);
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(act) & 15) == 0 && (reinterpret_cast<uintptr_t>(weight) & 15) == 0 &&
                  (reinterpret_cast<uintptr_t>(sz) & 3) == 0 &&
                  (reinterpret_cast<uintptr_t>(out) & (epilogue == KSQ_EPILOGUE_SILU_MUL ? 7 : 1)) == 0,
              KSQ_ERR_INVALID_ARGUMENT, "act and weight must be 16-byte aligned");
  const DeviceInfo* di = device_info();
  if (!di) return KSQ_ERR_HIP;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) workspace = nullptr;
  if (!workspace) workspace_bytes = 0;
  if (k % kTileK != 0) {
    // K an odd multiple of 64 (group size 64): the repacked weight has a last k tile whose upper half is padding; the
    // activations get rows of k + 64 elements with zeros behind the data, in front of the workspace
    KSQ_REQUIRE(act_perm == nullptr, KSQ_ERR_UNSUPPORTED, "act_perm needs k %% 128 == 0 (got %zu)", k);
    const size_t need = padded_act_bytes(m, k);
    KSQ_REQUIRE(workspace_bytes >= need, KSQ_ERR_WORKSPACE,
                "k=%zu is not a multiple of 128: %zu bytes of 256-byte aligned workspace are needed for the padded "
                "activations", k, need);
    rc = pad_rows(workspace, act, m, k, k + 64, s);
    if (rc != KSQ_OK) return rc;
    act = workspace;
    workspace = static_cast<char*>(workspace) + need;
    workspace_bytes -= need;
    if (workspace_bytes == 0) workspace = nullptr;
    k += 64;
  }
  if (act_perm) {
    const size_t need = (m * k * 2 + 255) / 256 * 256;
    KSQ_REQUIRE(workspace_bytes >= need, KSQ_ERR_WORKSPACE,
                "act_perm needs %zu bytes of 256-byte aligned workspace for the permuted activations", need);
    rc = ksq_permute_columns(workspace, act, act_perm, m, k, stream);
    if (rc != KSQ_OK) return rc;
    act = workspace;
    workspace = static_cast<char*>(workspace) + need;
    workspace_bytes -= need;
    if (workspace_bytes == 0) workspace = nullptr;
  }
  Epilogue epi;
  epi.kind = epilogue;
  epi.bias = bias;
  epi.row_absmax = row_absmax;
  if (env_int("KSQ_W4_FORCE_STREAM", 0) == 0 && w4a16_prefill_supported(dtype, m, n, k, g, di->cus) &&
      workspace_bytes >= w4a16_prefill_workspace_bytes(dtype, m, k))
    return w4a16_launch_prefill(dtype, out, act, weight, sz, m, n, k, g, workspace, workspace_bytes, s, epi);
  // The kernels below split K across workgroups through arrival counters owned per stream; a stream that got none
  // (more streams than counter regions) is planned as if it had no workspace: same results, no split.
  if (workspace_bytes && !counter_slot_available(s)) workspace_bytes = 0;
  if (w4a16_astream_supported(m, n, k)) {
    // Measured on Llama-2 7B and 70B shapes: with three or four row tiles the accumulator-stationary kernel is
    // never slower than the k-stationary one.  With two it wins while every workgroup gets one to four column
    // tiles and loses beyond that, where its last round of workgroups is mostly empty or, with very wide weights,
    // it depends on the clock the device happens to hold.
    const size_t ntiles = n / kTileN, cus = (size_t)di->cus;
    const bool dflt = m > 32 || (ntiles >= cus && ntiles <= 4 * cus);
    if (env_int("KSQ_W4_ASTREAM", dflt ? 1 : 0) != 0) {
      const AstreamPlan ap = w4a16_astream_plan(m, n, k, di->cus, workspace_bytes);
      return w4a16_launch_astream(dtype, ap, out, act, weight, sz, m, n, k, g, di->cus, workspace, s, epi);
    }
  }
  if (m <= (size_t)env_int("KSQ_W4_KSTAT_MAX_M", 64) && env_int("KSQ_W4_KSTAT", 1) != 0) {
    KstatPlan kp = w4a16_kstat_plan(m, n, k, di->cus, workspace_bytes, g);
    // A K that the k-stationary kernel would split four ways or more across workgroups (nine to sixteen rows; fewer
    // rows walk K in phases instead): every workgroup then covers a quarter of K or less for many column tiles and
    // ends every batch in a hand-over.  The streaming kernel with two column tiles per wave and four splits is the
    // faster one there (Llama-3-70B down, K = 28672, sixteen rows: 38.4 -> 31.5 us).
    const bool long_k = kp.ok && !kp.phases && kp.mt == 1 && kp.ksplit >= 4 && env_int("KSQ_W4_LONG_K_STREAM", 1) != 0;
    if (long_k) {
      W4Plan lp = w4a16_plan(m, n, k, di->cus, workspace_bytes);
      if (lp.ksplit > 1) {  // the workspace holds its partial tiles
        lp = w4a16_plan_with(m, n, k, di->cus, workspace_bytes, 2, 4);
        if (lp.ksplit == 4) return w4a16_launch_stream(dtype, lp, out, act, weight, sz, m, n, k, g, workspace, s, epi);
      }
    }
    if (kp.ok) return w4a16_launch_kstat(dtype, kp, out, act, weight, sz, m, n, k, g, workspace, s, epi);
  }
  W4Plan plan = w4a16_plan(m, n, k, di->cus, workspace_bytes);
  return w4a16_launch_stream(dtype, plan, out, act, weight, sz, m, n, k, g, workspace, s, epi);
}

int ksq_w4a16_gemm_ex(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                      size_t k, size_t g, const int32_t* act_perm, int epilogue, const void* bias, void* workspace,
                      size_t workspace_bytes, void* stream) {
  return w4a16_gemm_impl(dtype, out, act, weight, sz, m, n, k, g, act_perm, epilogue, bias, nullptr, workspace,
                         workspace_bytes, stream);
}

int ksq_w4a16_gemm_rowmax(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                          size_t k, size_t g, int epilogue, const void* bias, float* row_absmax, void* workspace,
                          size_t workspace_bytes, void* stream) {
  KSQ_REQUIRE(row_absmax != nullptr && (reinterpret_cast<uintptr_t>(row_absmax) & 3) == 0, KSQ_ERR_INVALID_ARGUMENT,
              "row_absmax is null or misaligned");
  return w4a16_gemm_impl(dtype, out, act, weight, sz, m, n, k, g, nullptr, epilogue, bias, row_absmax, workspace,
                         workspace_bytes, stream);
}

int ksq_w4a16_gemm(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                   size_t k, size_t g, void* workspace, size_t workspace_bytes, void* stream) {
  return ksq_w4a16_gemm_ex(dtype, out, act, weight, sz, m, n, k, g, nullptr, KSQ_EPILOGUE_NONE, nullptr, workspace,
                           workspace_bytes, stream);
}

int ksq_w4a16_gemm_static_scratch(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m,
                                  size_t n, size_t k, size_t g, void* stream) {
  if (m == 0) return KSQ_OK;
  size_t need = 0;
  int rc = ksq_w4a16_workspace_bytes(m, n, k, &need);
  if (rc != KSQ_OK) return rc;
  KSQ_REQUIRE(need <= (size_t)KSQ_STATIC_SCRATCH_BYTES, KSQ_ERR_WORKSPACE,
              "m=%zu n=%zu k=%zu needs %zu bytes of scratch; the library's static scratch holds %zu: use "
              "ksq_w4a16_gemm with a workspace of the caller's",
              m, n, k, need, (size_t)KSQ_STATIC_SCRATCH_BYTES);
  unsigned char* scratch = static_scratch_device_ptr();  // this device's copy of the array
  if (!scratch) return KSQ_ERR_HIP;
  // Nothing in the scratch has to start at zero: split-K partial tiles and the re-encoded activations are written
  // in full before they are read, and the arrival counters live elsewhere and return to zero by themselves.
  return ksq_w4a16_gemm_ex(dtype, out, act, weight, sz, m, n, k, g, nullptr, KSQ_EPILOGUE_NONE, nullptr, scratch,
                           need, stream);
}

}  // extern "C"
