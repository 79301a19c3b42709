// Host-side stand-in for <hip/hip_runtime.h>, used ONLY by the CPU test build of the kernels
// (tests/emu/build_emu.py).  It lets the unmodified kernel sources compile with the host clang and
// runs every workgroup as a set of cooperatively scheduled fibers, one per lane, so that shared
// memory, barriers, wave shuffles and MFMA behave as on the device.  With guard pages around test
// buffers this turns out-of-bounds accesses into a host SIGSEGV instead of a GPU fault.
//
// It is test infrastructure: the shipped library is built by hipcc from the same sources and never
// includes this file.
#pragma once
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <ucontext.h>

#include <algorithm>
#include <atomic>
#include <functional>
#include <thread>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __restrict__
#define __launch_bounds__(...)
#define __shared__ thread_local
#define __align__(n) __attribute__((aligned(n)))
#define HIP_KERNEL_NAME(...) __VA_ARGS__

struct dim3 {
  unsigned x, y, z;
  dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint3 { unsigned x, y, z; };

typedef int hipError_t;
typedef void* hipStream_t;
enum { hipSuccess = 0, hipErrorInvalidValue = 1 };
enum hipFuncAttribute { hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
static inline hipError_t hipGetLastError() { return hipSuccess; }
static inline hipError_t hipPeekAtLastError() { return hipSuccess; }
static inline const char* hipGetErrorString(hipError_t) { return "emu"; }
template <class F> static inline hipError_t hipFuncSetAttribute(F, hipFuncAttribute, int) { return hipSuccess; }
static inline hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) { memset(p, v, n); return hipSuccess; }
static inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
// a __device__ array is a host array here, and its symbol is its address
#define HIP_SYMBOL(x) (&(x))
static inline hipError_t hipGetSymbolAddress(void** p, const void* sym) { *p = const_cast<void*>(sym); return hipSuccess; }
enum hipDeviceAttribute_t { hipDeviceAttributeMultiprocessorCount = 63 };
// a small "device" so that the test shapes exercise both the one-slab-per-workgroup and the shared-tile launches
static inline hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t, int) { *v = 8; return hipSuccess; }
typedef void* hipEvent_t;
static inline hipError_t hipEventCreate(hipEvent_t* e) { *e = nullptr; return hipSuccess; }
static inline hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
static inline hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
static inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { *ms = 0.f; return hipSuccess; }
static inline hipError_t hipEventDestroy(hipEvent_t) { return hipSuccess; }

namespace emu {

constexpr int kMaxThreads = 1024;
constexpr int kWave = 64;
constexpr size_t kStack = 256 * 1024;
constexpr size_t kLds = 160 * 1024;

struct WaveX {
  unsigned gen = 0;
  int count = 0;
  alignas(16) unsigned char slot[2][kWave][128];
};

struct Fiber {
  ucontext_t ctx;
  bool done = false;
};

struct Block {
  uint3 bidx, bdim, gdim;
  int nthreads = 0;
  int cur = 0;
  int alive = 0;
  int bar_count = 0;
  unsigned bar_gen = 0;
  ucontext_t sched;
  std::vector<Fiber> fibers;
  std::vector<WaveX> waves;
  std::vector<char> stacks;
  const std::function<void()>* body = nullptr;
};

extern thread_local Block* g_blk;

inline void yield() { swapcontext(&g_blk->fibers[g_blk->cur].ctx, &g_blk->sched); }
inline int tid() { return g_blk->cur; }
inline int lane() { return g_blk->cur % kWave; }
inline int wave_lanes(int w) { return std::min(kWave, g_blk->nthreads - w * kWave); }

inline void syncthreads() {
  Block* b = g_blk;
  unsigned gen = b->bar_gen;
  if (++b->bar_count == b->alive) {
    b->bar_count = 0;
    b->bar_gen++;
  } else {
    while (b->bar_gen == gen) yield();
  }
}

// Every lane of the wave deposits `bytes` bytes, waits for the others, and gets a view of all deposits.
inline const unsigned char (*wave_exchange(const void* mine, size_t bytes))[128] {
  Block* b = g_blk;
  int w = b->cur / kWave, l = b->cur % kWave;
  WaveX& x = b->waves[w];
  unsigned gen = x.gen;
  int p = gen & 1;
  if (bytes > 128) abort();
  memcpy(x.slot[p][l], mine, bytes);
  if (++x.count == wave_lanes(w)) {
    x.count = 0;
    x.gen++;
  } else {
    while (x.gen == gen) yield();
  }
  return x.slot[p];
}

template <class T> inline T shfl(T v, int src) {
  auto s = wave_exchange(&v, sizeof(T));
  T o;
  memcpy(&o, s[src & (kWave - 1)], sizeof(T));
  return o;
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane 4 a + b receives element b of the lanes 4 e + a, e = 0..3
typedef short s16x4_t __attribute__((ext_vector_type(4)));
inline s16x4_t ds_read_tr16(const void* p) {
  uint64_t mine;
  memcpy(&mine, p, 8);
  auto s = wave_exchange(&mine, 8);
  const int l = lane(), base = l & ~15, n = l & 15;
  s16x4_t out;
  for (int e = 0; e < 4; ++e) {
    uint16_t h;
    memcpy(&h, s[base + 4 * e + (n >> 2)] + 2 * (n & 3), 2);
    out[e] = (short)h;
  }
  return out;
}

// rendezvous of the lanes of one wave (lanes run as cooperative fibers: a wave-private LDS hand-over needs one)
inline void wave_sync() { char c = 0; (void)wave_exchange(&c, 1); }

void run_grid(dim3 grid, dim3 block, size_t smem, const std::function<void()>& body);

// ---- MFMA (layouts as on CDNA3/4: see gdn_common.h) ----
template <class V> inline void unpack_bf16(const unsigned char* p, float* out, int n) {
  for (int e = 0; e < n; ++e) {
    uint16_t h;
    memcpy(&h, p + 2 * e, 2);
    uint32_t u = (uint32_t)h << 16;
    memcpy(&out[e], &u, 4);
  }
}

template <class VA, class VC> inline VC mfma_32x32x16_bf16(VA a, VA b, VC c) {
  struct { VA a, b; } mine{a, b};
  auto s = wave_exchange(&mine, sizeof(mine));
  int l = lane(), half = l >> 5, col = l & 31;
  for (int r = 0; r < 16; ++r) {
    int i = 8 * (r >> 2) + 4 * half + (r & 3);
    float sum = 0.f;
    for (int k = 0; k < 16; ++k) {
      float av, bv;
      unpack_bf16<VA>(s[i + 32 * (k >> 3)] + 2 * (k & 7), &av, 1);
      unpack_bf16<VA>(s[col + 32 * (k >> 3)] + sizeof(VA) + 2 * (k & 7), &bv, 1);
      sum += av * bv;
    }
    c[r] += sum;
  }
  return c;
}

template <class VA, class VC> inline VC mfma_16x16x32_bf16(VA a, VA b, VC c) {
  struct { VA a, b; } mine{a, b};
  auto s = wave_exchange(&mine, sizeof(mine));
  int l = lane(), q = l >> 4, col = l & 15;
  for (int r = 0; r < 4; ++r) {
    int i = 4 * q + r;
    float sum = 0.f;
    for (int k = 0; k < 32; ++k) {
      float av, bv;
      unpack_bf16<VA>(s[i + 16 * (k >> 3)] + 2 * (k & 7), &av, 1);
      unpack_bf16<VA>(s[col + 16 * (k >> 3)] + sizeof(VA) + 2 * (k & 7), &bv, 1);
      sum += av * bv;
    }
    c[r] += sum;
  }
  return c;
}

template <class VC> inline VC mfma_32x32x2_f32(float a, float b, VC c) {
  struct { float a, b; } mine{a, b};
  auto s = wave_exchange(&mine, sizeof(mine));
  int l = lane(), half = l >> 5, col = l & 31;
  for (int r = 0; r < 16; ++r) {
    int i = 8 * (r >> 2) + 4 * half + (r & 3);
    for (int k = 0; k < 2; ++k) {
      float av, bv;
      memcpy(&av, s[i + 32 * k], 4);
      memcpy(&bv, s[col + 32 * k] + 4, 4);
      c[r] = fmaf(av, bv, c[r]);
    }
  }
  return c;
}

template <class VC> inline VC mfma_16x16x4_f32(float a, float b, VC c) {
  struct { float a, b; } mine{a, b};
  auto s = wave_exchange(&mine, sizeof(mine));
  int l = lane(), q = l >> 4, col = l & 15;
  for (int r = 0; r < 4; ++r) {
    int i = 4 * q + r;
    for (int k = 0; k < 4; ++k) {
      float av, bv;
      memcpy(&av, s[i + 16 * k], 4);
      memcpy(&bv, s[col + 16 * k] + 4, 4);
      c[r] = fmaf(av, bv, c[r]);
    }
  }
  return c;
}

struct TidProxy {
  struct X { operator unsigned() const { return g_blk->cur % g_blk->bdim.x; } } x;
  struct Y { operator unsigned() const { return (g_blk->cur / g_blk->bdim.x) % g_blk->bdim.y; } } y;
  struct Z { operator unsigned() const { return g_blk->cur / (g_blk->bdim.x * g_blk->bdim.y); } } z;
};
struct BidProxy {
  struct X { operator unsigned() const { return g_blk->bidx.x; } } x;
  struct Y { operator unsigned() const { return g_blk->bidx.y; } } y;
  struct Z { operator unsigned() const { return g_blk->bidx.z; } } z;
};
struct BdimProxy {
  struct X { operator unsigned() const { return g_blk->bdim.x; } } x;
  struct Y { operator unsigned() const { return g_blk->bdim.y; } } y;
  struct Z { operator unsigned() const { return g_blk->bdim.z; } } z;
};
struct GdimProxy {
  struct X { operator unsigned() const { return g_blk->gdim.x; } } x;
  struct Y { operator unsigned() const { return g_blk->gdim.y; } } y;
  struct Z { operator unsigned() const { return g_blk->gdim.z; } } z;
};

}  // namespace emu

static emu::TidProxy threadIdx;
static emu::BidProxy blockIdx;
static emu::BdimProxy blockDim;
static emu::GdimProxy gridDim;

#define __syncthreads() emu::syncthreads()
#define __builtin_amdgcn_s_barrier() emu::syncthreads()
#define __builtin_amdgcn_fence(...) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_rsqf(x) (1.0f / sqrtf(x))
#define __builtin_amdgcn_logf(x) log2f(x)
#define GDN_WAVES_PER_SIMD(n)
#define GDN_KEEP_HERE(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(m, n, s) ((void)0)
#define __builtin_amdgcn_wave_barrier() emu::wave_sync()
#define __builtin_amdgcn_s_sleep(x) emu::yield()
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu::ds_read_tr16((const void*)(uintptr_t)(p))
// direct global -> LDS load: lane l's `size` bytes land at dst + l*size (done at once: the emulator has no asynchrony)
#define __builtin_amdgcn_global_load_lds(src, dst, size, off, aux) \
  memcpy((unsigned char*)(uintptr_t)(dst) + (off) + emu::lane() * (size), (const void*)(uintptr_t)(src), (size))
// v_permlane32_swap: the upper 32 lanes of the first operand trade places with the lower 32 lanes of the second;
// returns (new first, new second)
struct emu_u32x2 { unsigned v[2]; unsigned operator[](int i) const { return v[i]; } };
inline emu_u32x2 __builtin_amdgcn_permlane32_swap(unsigned a, unsigned b, bool, bool) {
  const int l = emu::lane();
  const unsigned a_other = emu::shfl(a, l ^ 32), b_other = emu::shfl(b, l ^ 32);
  emu_u32x2 r;
  r.v[0] = l < 32 ? a : b_other;   // first: lower half keeps its own, upper half receives the second's lower half
  r.v[1] = l < 32 ? a_other : b;   // second: lower half receives the first's upper half, upper half keeps its own
  return r;
}
template <class T> inline T __shfl(T v, int src, int = 64) { return emu::shfl(v, src); }
template <class T> inline T __shfl_xor(T v, int m, int = 64) { return emu::shfl(v, emu::lane() ^ m); }
template <class T> inline T __shfl_up(T v, unsigned d, int = 64) {
  int l = emu::lane();
  return emu::shfl(v, l >= (int)d ? l - (int)d : l);
}
template <class T> inline T __shfl_down(T v, unsigned d, int = 64) {
  int l = emu::lane();
  return emu::shfl(v, l + (int)d < emu::kWave ? l + (int)d : l);
}

inline int emu_update_dpp(int /*old*/, int src, int ctrl) {
  const int l = emu::lane();
  int from = l;
  if (ctrl >= 0 && ctrl <= 0xFF) from = (l & ~3) | ((ctrl >> (2 * (l & 3))) & 3);          // quad_perm
  else if (ctrl == 0x141) from = (l & ~7) | (7 - (l & 7));                                  // row_half_mirror
  else if (ctrl == 0x140) from = (l & ~15) | (15 - (l & 15));                               // row_mirror
  else if (ctrl > 0x120 && ctrl <= 0x12F) from = (l & ~15) | ((l - (ctrl & 15)) & 15);      // row_ror:n
  else abort();
  return emu::shfl(src, from);
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) emu_update_dpp(old, src, ctrl)

#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) emu::mfma_32x32x16_bf16(a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu::mfma_16x16x32_bf16(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) emu::mfma_32x32x2_f32(a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, x, y, z) emu::mfma_16x16x4_f32(a, b, c)

#define __expf(x) expf(x)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __logf(x) logf(x)
static inline float __frsqrt_rn(float x) { return 1.0f / sqrtf(x); }
static inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
static inline float __fdividef(float a, float b) { return a / b; }
static inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }
static inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
static inline float atomicAdd(float* p, float v) { float o = *p; *p = o + v; return o; }
static inline int atomicAdd(int* p, int v) { int o = *p; *p = o + v; return o; }

#define hipLaunchKernelGGL(kernel, grid, block, smem, stream, ...) \
  emu::run_grid((grid), (block), (smem), [=]() { kernel(__VA_ARGS__); })
