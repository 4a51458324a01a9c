// CPU stand-in for <hip/hip_runtime.h>: lets the library's HIP sources compile as plain C++ for x86 so that the very
// kernel code that runs on gfx950 can be executed on the host, one fiber per lane, by tests/emu/emu_runtime.cpp.
//
// TEST INFRASTRUCTURE ONLY.  Nothing under ksanallm_amd/ includes, links or loads this; the product library is built
// from the same sources by hipcc against the real header.  What the emulation is for:
//   * every range-checked buffer load is checked twice: against num_records as the hardware does, and against the
//     host allocation that the resource's base lies in -- an access that the hardware would let through but that
//     leaves the tensor is reported with kernel, workgroup and lane;
//   * raw pointer accesses are ordinary host accesses, so an AddressSanitizer build catches them;
//   * cross-lane operations (ds_bpermute, DPP, readfirstlane, MFMA, shuffles) and barriers are real rendezvous of the
//     participating lanes, so a lane-dependent branch around one of them deadlocks the emulation instead of passing;
//   * the C ABI of the emulated build is the library's own, so the parity tests run against the oracle on the CPU.
// What it does not model: timing, the asynchrony of memory operations (s_waitcnt is a no-op; a global -> LDS load
// lands at once), LDS bank conflicts, register pressure.
#pragma once

#define KSQ_EMU 1
#ifndef __HIPCC__
#define __HIPCC__ 1  // the sources guard their device-side helpers with it
#endif

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define KSQ_EMU_ASAN 1
#endif
#endif

// ---- language extensions --------------------------------------------------------------------------------------------
#define __global__
#define __device__
#define __host__
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define amdgpu_waves_per_eu(...)  // inside __attribute__(( )): leaves an empty attribute list
// LDS of the workgroup that the calling OS thread emulates.  AddressSanitizer puts red zones around plain statics only,
// so that build runs one workgroup at a time.
#if defined(KSQ_EMU_ASAN)
#define __shared__ static
#else
#define __shared__ static thread_local
#endif

struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

struct alignas(16) uint4 {
  unsigned x, y, z, w;
};

// ---- host API (the subset the library calls) -------------------------------------------------------------------------
typedef struct emu_stream_tag* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
constexpr hipError_t hipErrorInvalidValue = 1;
struct hipDeviceProp_t {
  int multiProcessorCount;
  char name[64];
};

extern "C" {
hipError_t hipGetDevice(int* dev);
hipError_t hipGetDeviceProperties(hipDeviceProp_t* prop, int dev);
hipError_t hipGetLastError(void);
const char* hipGetErrorString(hipError_t e);
hipError_t hipMalloc(void** p, size_t bytes);
hipError_t hipFree(void* p);
hipError_t hipHostMalloc(void** p, size_t bytes, unsigned flags = 0);
hipError_t hipHostFree(void* p);
hipError_t hipDeviceSynchronize(void);
hipError_t hipStreamSynchronize(hipStream_t s);
hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, int kind);
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes, int kind, hipStream_t s);
hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t s);
}
constexpr int hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3, hipMemcpyDefault = 4;

namespace emu {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x8_t __attribute__((ext_vector_type(8)));

// ---- per-lane state, visible to the inline builtins ------------------------------------------------------------------
struct WaveState {
  alignas(64) uint32_t x[2][64][16];  // exchange area of the cross-lane operations, two generations
  unsigned gen;                       // completed rendezvous of this wave
  int arrived, alive;
  uint64_t alive_mask;
  int first[2];                       // lowest live lane when the rendezvous of each generation parity completed
  int site;                           // source line at which the lanes of the pending rendezvous wait (all the same)
  void (*fn)(WaveState*, int slot, int kind);  // run once by whoever completes the rendezvous
  int fn_kind;
};
struct LaneState {
  dim3 tid, bid, bdim, gdim;
  int lane;  // 0..63 inside the wave
  WaveState* wave;
};
extern thread_local LaneState* cur;

// rendezvous of the live lanes of the calling lane's wave; returns the slot (generation parity) that was published to
int wave_rendezvous(int site, void (*fn)(WaveState*, int, int) = nullptr, int kind = 0);
inline int wave_slot() { return (int)(cur->wave->gen & 1u); }
void block_barrier();

// ---- memory registry: what a buffer resource may touch ----------------------------------------------------------------
struct Rsrc {
  const char* base;
  uint32_t num_records;
  uintptr_t lo, hi;  // the registered allocation that `base` lies in ([0,0): none)
};
Rsrc make_rsrc(const void* base, uint32_t num_records);
void report_oob(const char* what, const Rsrc& r, uint32_t voff, uint32_t soff, uint32_t bytes);
const void* symbol(const void* p, size_t bytes, const char* name);

inline bool in_range(const Rsrc& r, uint32_t voff, uint32_t bytes) {
  // raw buffer (stride 0): the vector offset alone is compared with num_records; the scalar offset is not
  return (uint64_t)voff + bytes <= (uint64_t)r.num_records;
}
inline const char* checked_address(const char* what, const Rsrc& r, uint32_t voff, uint32_t soff, uint32_t bytes) {
  const char* a = r.base + voff + soff;
  const uintptr_t u = reinterpret_cast<uintptr_t>(a);
  if (u < r.lo || u + bytes > r.hi) {
    report_oob(what, r, voff, soff, bytes);
    return nullptr;
  }
  return a;
}

// ---- launch -------------------------------------------------------------------------------------------------------------
void launch_impl(const char* name, dim3 grid, dim3 block, void (*tramp)(void*), void* closure);
template <class F>
inline void launch(const char* name, dim3 grid, dim3 block, F f) {
  launch_impl(name, grid, block, [](void* p) { (*static_cast<F*>(p))(); }, &f);
}

// ---- number formats -----------------------------------------------------------------------------------------------------
extern float e4m3_table[256];
uint8_t f32_to_e4m3(float v);

void mfma_collective(WaveState* w, int slot, int kind);  // kinds below
constexpr int kMfmaF16 = 0, kMfmaBf16 = 1, kMfmaFp8x32 = 2, kMfmaFp8x128 = 3;

template <int WORDS>
inline f32x4_t mfma(const void* a, const void* b, f32x4_t c, int kind, int site) {
  WaveState* w = cur->wave;
  const int slot = (int)(w->gen & 1u), l = cur->lane;
  std::memcpy(&w->x[slot][l][0], a, WORDS * 4);
  std::memcpy(&w->x[slot][l][8], b, WORDS * 4);
  wave_rendezvous(site, mfma_collective, kind);
  f32x4_t d;
  std::memcpy(&d, &w->x[slot][l][0], 16);
  return c + d;
}

}  // namespace emu

#define threadIdx (::emu::cur->tid)
#define blockIdx (::emu::cur->bid)
#define blockDim (::emu::cur->bdim)
#define gridDim (::emu::cur->gdim)

#define HIP_SYMBOL(x) ::emu::symbol(&(x), sizeof(x), #x)
inline hipError_t hipGetSymbolAddress(void** p, const void* sym) {
  *p = const_cast<void*>(sym);
  return hipSuccess;
}

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...) \
  ::emu::launch(#kernel, dim3(grid), dim3(block), [=]() { (kernel)(__VA_ARGS__); })

// ---- device builtins ----------------------------------------------------------------------------------------------------
#define __amdgpu_buffer_rsrc_t ::emu::Rsrc

inline emu::Rsrc __builtin_amdgcn_make_buffer_rsrc(const void* base, short /*stride*/, int num_records, int /*flags*/) {
  return emu::make_rsrc(base, (uint32_t)num_records);
}
inline emu::u32x4_t __builtin_amdgcn_raw_buffer_load_b128(const emu::Rsrc& r, unsigned voff, unsigned soff, int) {
  emu::u32x4_t v = {0u, 0u, 0u, 0u};
  if (!emu::in_range(r, voff, 16)) return v;
  if (const char* a = emu::checked_address("buffer_load_dwordx4", r, voff, soff, 16)) std::memcpy(&v, a, 16);
  return v;
}
inline unsigned __builtin_amdgcn_raw_buffer_load_b32(const emu::Rsrc& r, unsigned voff, unsigned soff, int) {
  unsigned v = 0;
  if (!emu::in_range(r, voff, 4)) return v;
  if (const char* a = emu::checked_address("buffer_load_dword", r, voff, soff, 4)) std::memcpy(&v, a, 4);
  return v;
}
// global -> LDS: lane l lands at lds + ioff + l * size (the LDS base is wave-uniform: M0)
inline void __builtin_amdgcn_raw_ptr_buffer_load_lds(const emu::Rsrc& r, __attribute__((address_space(3))) void* lds,
                                                     unsigned size, unsigned voff, unsigned soff, unsigned ioff, int) {
  char* dst = (char*)(void*)lds + ioff + (size_t)emu::cur->lane * size;
  if (!emu::in_range(r, voff + ioff, size)) {
    std::memset(dst, 0, size);
    return;
  }
  if (const char* a = emu::checked_address("buffer_load lds", r, voff + ioff, soff, size)) std::memcpy(dst, a, size);
}

inline void __builtin_amdgcn_sched_barrier(int) {}
inline void __builtin_amdgcn_sched_group_barrier(int, int, int) {}
// Lanes of a wave run in lockstep on the hardware and independently here.  Where a wave's lanes hand data to each
// other or to another workgroup through memory (an LDS transpose inside a wave, a partial tile followed by an arrival
// counter), the code has to wait for the wave's outstanding memory operations in between anyway; that wait is where the
// emulated lanes meet, so that "every lane's earlier accesses are complete" means here what it means there.
inline void __builtin_amdgcn_s_waitcnt(int, int site = __builtin_LINE()) { emu::wave_rendezvous(site); }
inline void __builtin_amdgcn_s_setprio(int) {}
inline void __builtin_amdgcn_s_sleep(int) {}
inline void __builtin_amdgcn_s_barrier() { emu::block_barrier(); }
inline void __syncthreads() { emu::block_barrier(); }

inline int __builtin_amdgcn_ds_bpermute(int addr, int val, int site = __builtin_LINE()) {
  emu::WaveState* w = emu::cur->wave;
  const int slot = emu::wave_slot();
  w->x[slot][emu::cur->lane][0] = (uint32_t)val;
  emu::wave_rendezvous(site);
  return (int)w->x[slot][(addr >> 2) & 63][0];
}
inline int __builtin_amdgcn_readfirstlane(int val, int site = __builtin_LINE()) {
  emu::WaveState* w = emu::cur->wave;
  const int slot = emu::wave_slot();
  w->x[slot][emu::cur->lane][0] = (uint32_t)val;
  emu::wave_rendezvous(site);
  return (int)w->x[slot][w->first[slot]][0];  // lanes may have left the kernel since: not alive_mask as it is now
}
// quad permutations only (dpp_ctrl < 0x100), all rows and banks enabled
inline int __builtin_amdgcn_update_dpp(int /*old*/, int src, int ctrl, int row_mask, int bank_mask, bool,
                                       int site = __builtin_LINE()) {
  if (ctrl >= 0x100 || row_mask != 0xF || bank_mask != 0xF) {
    std::fprintf(stderr, "emu: unsupported DPP control 0x%x\n", ctrl);
    std::abort();
  }
  emu::WaveState* w = emu::cur->wave;
  const int slot = emu::wave_slot(), l = emu::cur->lane;
  w->x[slot][l][0] = (uint32_t)src;
  emu::wave_rendezvous(site);
  return (int)w->x[slot][(l & ~3) | ((ctrl >> (2 * (l & 3))) & 3)][0];
}
template <typename V>
inline V emu_shfl_xor(V v, int mask, int site) {
  static_assert(sizeof(V) == 4, "32-bit shuffles only");
  emu::WaveState* w = emu::cur->wave;
  const int slot = emu::wave_slot(), l = emu::cur->lane;
  std::memcpy(&w->x[slot][l][0], &v, 4);
  emu::wave_rendezvous(site);
  V r;
  std::memcpy(&r, &w->x[slot][(l ^ mask) & 63][0], 4);
  return r;
}
inline float __shfl_xor(float v, int mask, int site = __builtin_LINE()) { return emu_shfl_xor(v, mask, site); }
inline int __shfl_xor(int v, int mask, int site = __builtin_LINE()) { return emu_shfl_xor(v, mask, site); }
inline unsigned __shfl_xor(unsigned v, int mask, int site = __builtin_LINE()) { return emu_shfl_xor(v, mask, site); }

typedef _Float16 emu_half8 __attribute__((ext_vector_type(8)));
typedef __bf16 emu_bf16x8 __attribute__((ext_vector_type(8)));
inline emu::f32x4_t __builtin_amdgcn_mfma_f32_16x16x32_f16(emu_half8 a, emu_half8 b, emu::f32x4_t c, int, int, int,
                                                          int site = __builtin_LINE()) {
  return emu::mfma<4>(&a, &b, c, emu::kMfmaF16, site);
}
inline emu::f32x4_t __builtin_amdgcn_mfma_f32_16x16x32_bf16(emu_bf16x8 a, emu_bf16x8 b, emu::f32x4_t c, int, int, int,
                                                           int site = __builtin_LINE()) {
  return emu::mfma<4>(&a, &b, c, emu::kMfmaBf16, site);
}
inline emu::f32x4_t __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(long a, long b, emu::f32x4_t c, int, int, int,
                                                              int site = __builtin_LINE()) {
  return emu::mfma<2>(&a, &b, c, emu::kMfmaFp8x32, site);
}
// e4m3 x e4m3 (cbsz = blgp = 0), unit block scales
inline emu::f32x4_t __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(emu::i32x8_t a, emu::i32x8_t b, emu::f32x4_t c,
                                                                     int cbsz, int blgp, int, int, int, int,
                                                                     int site = __builtin_LINE()) {
  if (cbsz != 0 || blgp != 0) {
    std::fprintf(stderr, "emu: f8f6f4 MFMA formats other than e4m3 are not modelled\n");
    std::abort();
  }
  return emu::mfma<8>(&a, &b, c, emu::kMfmaFp8x128, site);
}

inline int __builtin_amdgcn_cvt_pk_fp8_f32(float a, float b, int old, bool high) {
  const uint32_t pair = (uint32_t)emu::f32_to_e4m3(a) | ((uint32_t)emu::f32_to_e4m3(b) << 8);
  const uint32_t o = (uint32_t)old;
  return (int)(high ? ((o & 0x0000FFFFu) | (pair << 16)) : ((o & 0xFFFF0000u) | pair));
}
inline float __builtin_amdgcn_cvt_f32_fp8(int src, int byte_sel) {
  return emu::e4m3_table[((uint32_t)src >> (8 * byte_sel)) & 0xFFu];
}

inline float __expf(float x) { return std::exp(x); }

#ifndef __HIP_MEMORY_SCOPE_AGENT
#define __HIP_MEMORY_SCOPE_AGENT 4
#endif
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n((p), (v), __ATOMIC_SEQ_CST)
#define __hip_atomic_load(p, order, scope) __atomic_load_n((p), __ATOMIC_SEQ_CST)
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)
inline unsigned atomicMax(unsigned* p, unsigned v) {
  unsigned old = __atomic_load_n(p, __ATOMIC_SEQ_CST);
  while (old < v && !__atomic_compare_exchange_n(p, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_SEQ_CST)) {
  }
  return old;
}
