// Device-side building blocks shared by the gated-delta-rule kernels (gfx950 / CDNA4).
//
// Conventions
//   * wavefront = 64 lanes; workgroups are 256 threads (4 waves) unless stated otherwise.
//   * chunk = 64 tokens.  A "tile" in LDS is [rows][ld] with ld = cols + 16 bytes of padding so that
//     16-byte fragment reads of consecutive rows fall into different banks.
//   * every matrix-core contraction accumulates one 32x32 fp32 tile per wave, C[i][j] += sum_k A[i][k] * B[k][j]:
//       bf16: v_mfma_f32_32x32x16_bf16   lane l holds A[l%32][8*(l/32)+0..7] and B[8*(l/32)+0..7][l%32]
//       fp32: v_mfma_f32_32x32x2_f32     lane l holds A[l%32][l/32]          and B[l/32][l%32]
//     accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32].
//     The k index inside one instruction may be permuted freely as long as A and B agree; the fp32
//     path uses that to read 4 consecutive k per lane with one 16-byte load.
//     Operands come from LDS tiles (mma32<>) or, mostly, as "fragments": the registers a lane feeds to the
//     instruction, kept together per 32x32 tile (AccB<>).  Tiles travel between kernels, and between waves through
//     LDS, in that fragment order, and change orientation by a pass through the matrix core (mfma_transpose).
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

// dynamic LDS, one array per workgroup
extern __shared__ __align__(16) unsigned char gdn_smem[];

namespace gdn {

constexpr int kChunk = 64;
constexpr int kThreads = 256;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// round to nearest even; one v_cvt_pk_bf16_f32 on gfx950
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  const f32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) { return (uint16_t)(f32x2_to_bf16x2(f, 0.f) & 0xffffu); }

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int kVec = 4;  // elements per 16 bytes
  static __device__ __forceinline__ float to_f(float x) { return x; }
  static __device__ __forceinline__ float from_f(float x) { return x; }
};
template <> struct Elem<bf16_t> {
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float to_f(bf16_t x) { return bf16_to_f32(x.bits); }
  static __device__ __forceinline__ bf16_t from_f(float x) { bf16_t r; r.bits = f32_to_bf16(x); return r; }
};
template <> struct Elem<f16_t> {
  static constexpr int kVec = 8;
  static __device__ __forceinline__ float to_f(f16_t x) { _Float16 h = __builtin_bit_cast(_Float16, x.bits); return (float)h; }
  static __device__ __forceinline__ f16_t from_f(float x) { _Float16 h = (_Float16)x; f16_t r; r.bits = __builtin_bit_cast(uint16_t, h); return r; }
};

// padded leading dimension (in elements) of an LDS tile with `cols` columns
template <typename T> __device__ __host__ constexpr int lds_ld(int cols) { return cols + 16 / (int)sizeof(T); }

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global load
// and store of the wave (vmcnt(0)), which would serialise a software pipeline whose whole point is to keep global
// loads in flight across the barrier; kernels that hand data between waves through LDS only use this one.
#define GDN_LDS_BARRIER()                                             \
  do {                                                                \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");   \
    __builtin_amdgcn_s_barrier();                                     \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");   \
  } while (0)
// Instruction-scheduling fence: nothing is moved across it.  Used to pin hand-made software pipelines (issue the
// LDS reads of the next group, then the matrix instructions of this group) that the scheduler would otherwise
// serialise into read -> wait -> multiply.
#define GDN_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
// Workgroups are dealt to the 8 XCDs (each with its own L2) round-robin by their linear index.  The recurrence kernels
// number their workgroups so that the value heads of one q/k group, which read the same K / Q^T tiles, share an XCD:
// with P = (sequences x q/k groups) a multiple of 8, workgroup b handles pair (b/8/grp) 8 + b % 8, head b/8 % grp of it.
// Returns the plain index n Hv + h.
__device__ __forceinline__ int xcd_grouped_head(int b, int total, int grp) {
  const int pairs = total / grp;
  if (grp == 1 || pairs % 8 != 0) return b;
  const int j = b & 7, m = b >> 3;
  return ((m / grp) * 8 + j) * grp + m % grp;
}
// Kernel attribute: register budget of 512 / n per lane (n waves per SIMD).  With more than 256 registers allowed the
// compiler keeps matrix accumulators in the accumulation registers, and every vector instruction that touches them
// (decay, packing) then costs an extra move in each direction; a budget that allows more workgroups per CU is what
// the memory-bound kernels gain most from.
#ifndef GDN_WAVES_PER_SIMD
#define GDN_WAVES_PER_SIMD(n) __attribute__((amdgpu_waves_per_eu(n, n)))
#endif
// Pins a register value to this point of the program: the compiler can neither compute what follows from it earlier
// nor sink what precedes it.  Used where a cheap operation on a loaded value would otherwise be moved up to right
// behind the load and make the wave wait for it there, before the loads that follow have been issued.
#ifndef GDN_KEEP_HERE
#define GDN_KEEP_HERE(x) asm volatile("" : "+v"(x))
#endif
// The workgroups of a launch start together and, doing equal work, stay in step: they all load at the same time and
// all compute at the same time, and the two workgroups that share a CU do not fill each other's waits.  Holding back
// the second workgroup of each CU once (workgroup ids are handed out breadth first, so with `cus` compute units these
// are ids cus .. 2 cus - 1) shifts it, and every workgroup that later takes over its place, for the rest of the launch.
// Worth 2 % on the chunk-local backward kernel, measured in alternation with the same build without the wait; nothing
// on kernels whose phases are shorter or that run one workgroup per CU.  The wait costs its own length once, at the
// end of the launch, so launches of fewer than `min_groups` workgroups skip it.
// UNITS: 64 clock cycles each (the argument of s_sleep is an immediate, at most 127).
template <int UNITS> __device__ __forceinline__ void stagger_second_resident(int times, int min_groups, int cus) {
  const int lin = blockIdx.x + gridDim.x * blockIdx.y;
  if ((int)(gridDim.x * gridDim.y) >= min_groups && lin >= cus && lin < 2 * cus) {
    for (int i = 0; i < times; ++i) __builtin_amdgcn_s_sleep(UNITS);
  }
}
// Asks the scheduler for the pattern (1 matrix instruction, nvalu vector instructions) x nmfma in the current
// scheduling region.
#define GDN_INTERLEAVE_MFMA_VALU(nmfma, nvalu)                        \
  do {                                                                \
    _Pragma("unroll") for (int gdn_i_ = 0; gdn_i_ < (nmfma); ++gdn_i_) { \
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              \
      __builtin_amdgcn_sched_group_barrier(0x002, (nvalu), 0);        \
    }                                                                 \
  } while (0)
// Orders the LDS traffic of one wave when its lanes hand data to each other through a wave-private LDS patch.  The
// hardware already executes a wave's LDS instructions in order; this only stops the compiler from reordering them.
#define GDN_WAVE_LDS_SYNC()                                           \
  do {                                                                \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");   \
    __builtin_amdgcn_wave_barrier();                                  \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");   \
  } while (0)
// Asynchronous copy global -> LDS that bypasses the registers: each of the 64 lanes of a wave moves 16 bytes from its
// own address `src`, and lane l's piece lands at lds_wave_base + 16 l (lds_wave_base must be wave-uniform).  A tile
// in fragment order ([k-group][lane][16 bytes]) is therefore copied verbatim by one such load per k-group.
// Completion is counted with the vector-memory loads: GDN_WAIT_VMEM() and then a barrier publish the data.
#define GDN_WAIT_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)   // vmcnt(0); expcnt and lgkmcnt left alone
template <typename T> __device__ __forceinline__ void load16_to_lds(const T* src, T* lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                   (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}
// beta (and its gradient) as the caller holds it: fp32, or, with `same` set, the 16-bit type T of q, k, v.  The value
// is fetched raw and converted later, so that a loader can issue the fetch without waiting for it.
template <typename T> __device__ __forceinline__ uint32_t gate_raw(const void* p, int same, int64_t i) {
  if (sizeof(T) == 2 && same) return reinterpret_cast<const uint16_t*>(p)[i];
  return reinterpret_cast<const uint32_t*>(p)[i];
}
template <typename T> __device__ __forceinline__ float gate_val(uint32_t raw, int same) {
  if constexpr (sizeof(T) == 2) {
    if (same) { T t; t.bits = (uint16_t)raw; return Elem<T>::to_f(t); }
  }
  return __uint_as_float(raw);
}
template <typename T> __device__ __forceinline__ void gate_st(void* p, int same, int64_t i, float x) {
  if constexpr (sizeof(T) == 2) {
    if (same) { reinterpret_cast<uint16_t*>(p)[i] = Elem<T>::from_f(x).bits; return; }
  }
  reinterpret_cast<float*>(p)[i] = x;
}
__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int imax(int a, int b) { return a > b ? a : b; }

// ---------------------------------------------------------------------------------------------
// 16-byte vectors of T <-> floats
// ---------------------------------------------------------------------------------------------
template <typename T> struct Vec16 {
  u32x4 raw;
  __device__ __forceinline__ float get(int e) const {
    if constexpr (sizeof(T) == 4) {
      return __uint_as_float(raw[e]);
    } else {
      uint32_t w = raw[e >> 1];
      T t; t.bits = (uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu));
      return Elem<T>::to_f(t);
    }
  }
  __device__ __forceinline__ void set(int e, float f) {
    if constexpr (sizeof(T) == 4) {
      raw[e] = __float_as_uint(f);
    } else {
      uint32_t h = Elem<T>::from_f(f).bits;
      uint32_t w = raw[e >> 1];
      raw[e >> 1] = (e & 1) ? ((w & 0xffffu) | (h << 16)) : ((w & 0xffff0000u) | h);
    }
  }
};

template <typename T> __device__ __forceinline__ Vec16<T> ld16(const T* p) {
  Vec16<T> v; v.raw = *reinterpret_cast<const u32x4*>(p); return v;
}
template <typename T> __device__ __forceinline__ void st16(T* p, const Vec16<T>& v) {
  *reinterpret_cast<u32x4*>(p) = v.raw;
}
// fp32 values of a 16-byte piece and back (bf16: two elements per 32-bit word, one conversion instruction per word)
template <typename T> __device__ __forceinline__ void unpack16(const Vec16<T>& v, float* f) {
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = __uint_as_float(v.raw[e]);
  } else if constexpr (std::is_same<T, bf16_t>::value) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[2 * e] = __uint_as_float(v.raw[e] << 16);
      f[2 * e + 1] = __uint_as_float(v.raw[e] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int e = 0; e < Elem<T>::kVec; ++e) f[e] = v.get(e);
  }
}
template <typename T> __device__ __forceinline__ Vec16<T> pack16(const float* f) {
  Vec16<T> r;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) r.raw[e] = __float_as_uint(f[e]);
  } else if constexpr (std::is_same<T, bf16_t>::value) {
#pragma unroll
    for (int e = 0; e < 4; ++e) r.raw[e] = f32x2_to_bf16x2(f[2 * e], f[2 * e + 1]);
  } else {
    r.raw = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < Elem<T>::kVec; ++e) r.set(e, f[e]);
  }
  return r;
}
// every element of a 16-byte piece times one factor (bf16: two elements per conversion instruction)
template <typename T> __device__ __forceinline__ Vec16<T> scale16(const Vec16<T>& v, float s) {
  Vec16<T> r;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) r.raw[e] = __float_as_uint(__uint_as_float(v.raw[e]) * s);
  } else if constexpr (std::is_same<T, bf16_t>::value) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      r.raw[e] = f32x2_to_bf16x2(__uint_as_float(v.raw[e] << 16) * s, __uint_as_float(v.raw[e] & 0xffff0000u) * s);
  } else {
    r = v;
#pragma unroll
    for (int e = 0; e < Elem<T>::kVec; ++e) r.set(e, v.get(e) * s);
  }
  return r;
}
template <typename T> __device__ __forceinline__ Vec16<T> zero16() {
  Vec16<T> v; v.raw = u32x4{0u, 0u, 0u, 0u}; return v;
}

// ---------------------------------------------------------------------------------------------
// global -> LDS tile loads.  The tile has 64 rows (tokens) and COLS columns; rows >= nvalid are
// zero filled (zero padding of a ragged last chunk is exact for the gated delta rule).
// ---------------------------------------------------------------------------------------------
// each row multiplied by rowscale[row] (fp32, in LDS)
template <typename T, int COLS>
__device__ __forceinline__ void load_tile_scaled(T* lds, int ld, const T* g, int64_t row_stride, int nvalid,
                                                 const float* rowscale, int tid) {
  constexpr int V = Elem<T>::kVec, CPR = COLS / V;
  for (int c = tid; c < kChunk * CPR; c += kThreads) {
    const int row = c / CPR, cc = c % CPR;
    Vec16<T> v = zero16<T>();
    if (row < nvalid) {
      v = ld16(g + (int64_t)row * row_stride + cc * V);
      v = scale16<T>(v, rowscale[row]);
    }
    st16(lds + row * ld + cc * V, v);
  }
}

// ---------------------------------------------------------------------------------------------
// MFMA wrappers
// ---------------------------------------------------------------------------------------------
// One operand fragment: the 16 bytes a lane feeds to the matrix core for one k-group
// (bf16: 8 k values -> one 32x32x16 instruction; fp32: 4 k values -> four 32x32x2 instructions).
template <typename T> struct KGroup { static constexpr int kLen = (sizeof(T) == 2) ? 16 : 8; };

// Transposing read from LDS (ds_read_b64_tr_b16): every lane names 8 bytes (4 16-bit elements); within each group of
// 16 lanes, lane 4 a + b receives element b of the lanes 4 e + a, e = 0..3.  Read as a 4 x 16 block of elements whose
// row e is held, 4 columns each, by the lanes 4 e .. 4 e + 3: lane n of the group gets column n, rows 0..3.
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 lds_read_tr16(const void* p) {
  const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
  return __builtin_bit_cast(u32x2, v);
}

// contiguous: p points at element [row][k0]; the lane reads kVec consecutive k
template <typename T> __device__ __forceinline__ u32x4 frag_contig(const T* p) {
  return *reinterpret_cast<const u32x4*>(p);
}
// strided: p points at element [k0][col] of a [k][ld] array; the lane gathers kVec values ld apart
template <typename T> __device__ __forceinline__ u32x4 frag_strided(const T* p, int ld) {
  u32x4 r;
  if constexpr (sizeof(T) == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = __float_as_uint(p[e * ld]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      uint32_t lo = p[(2 * e) * ld].bits, hi = p[(2 * e + 1) * ld].bits;
      r[e] = lo | (hi << 16);
    }
  }
  return r;
}

// strided, 16-bit types: tile points at element [k0][first of the wave's 32 columns] of a [k][ld] array in LDS; the lane
// receives its 8 consecutive k (k0 + 8 (lane >> 5) ..) of column lane & 31 from two transposing reads instead of
// gathering eight two-byte elements
template <typename T> __device__ __forceinline__ u32x4 frag_strided_tr(const T* tile, int ld) {
  static_assert(sizeof(T) == 2, "16-bit types");
  const int lane = threadIdx.x & 63;
  const int gr = lane >> 4, i = lane & 15, e = i >> 2, q = i & 3, hh = gr >> 1;
  const T* base = tile + (8 * hh + e) * ld + (gr & 1) * 16 + 4 * q;
  const u32x2 r0 = lds_read_tr16(base), r1 = lds_read_tr16(base + 4 * ld);
  return u32x4{r0[0], r0[1], r1[0], r1[1]};
}

template <typename T> __device__ __forceinline__ void mfma_kgroup(f32x16& acc, u32x4 a, u32x4 b) {
  if constexpr (sizeof(T) == 2) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc,
                                                  0, 0, 0);
  } else {
#pragma unroll
    for (int m = 0; m < 4; ++m)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[m]), __uint_as_float(b[m]), acc, 0, 0, 0);
  }
}

// acc(32x32) += A(32 x KLEN) * B(KLEN x 32), operands in LDS.
//   A_KC = true : A[i][k] at A[i*lda + k]   (pass A = &tile[i0][k0])
//   A_KC = false: A[i][k] at A[k*lda + i]   (pass A = &tile[k0][i0])
//   B_KC = true : B[k][j] at B[j*ldb + k]   (pass B = &tile[j0][k0])
//   B_KC = false: B[k][j] at B[k*ldb + j]   (pass B = &tile[k0][j0])
template <typename T, int KLEN, bool A_KC, bool B_KC>
__device__ __forceinline__ void mma32(f32x16& acc, const T* A, int lda, const T* B, int ldb) {
  constexpr int G = KGroup<T>::kLen, V = Elem<T>::kVec;
  static_assert(KLEN % G == 0, "contraction length must be a multiple of the k-group");
  const int lane = threadIdx.x & 63, r32 = lane & 31, half = lane >> 5;
#pragma unroll
  for (int kg = 0; kg < KLEN / G; ++kg) {
    const int k = kg * G + half * V;
    u32x4 a, b;
    if constexpr (A_KC) a = frag_contig(A + r32 * lda + k);
    else if constexpr (sizeof(T) == 2) a = frag_strided_tr(A + kg * G * lda, lda);
    else a = frag_strided(A + k * lda + r32, lda);
    if constexpr (B_KC) b = frag_contig(B + r32 * ldb + k);
    else if constexpr (sizeof(T) == 2) b = frag_strided_tr(B + kg * G * ldb, ldb);
    else b = frag_strided(B + k * ldb + r32, ldb);
    mfma_kgroup<T>(acc, a, b);
  }
}

// ---------------------------------------------------------------------------------------------
// Chaining two contractions through registers.  An accumulator tile C (rows i in registers, column j = lane%32)
// already has the lane layout of a B operand whose contraction index is C's row index: D += A * C needs no LDS
// round trip.  Per k-group the lane's registers cover rows
//     bf16: r = 8kg..8kg+7  ->  16kg + {4h..4h+3, 8+4h..8+4h+3}      fp32: r = 4kg..4kg+3  ->  8kg + 4h..4h+3
// (h = lane/32), so the A operand must be gathered with the same k order: frag_a_split.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ f32x16 acc_zero();
template <typename T> struct AccK { static constexpr int kGroups = (sizeof(T) == 2) ? 2 : 4; };  // per 32-row tile

template <typename T, int KG> __device__ __forceinline__ u32x4 frag_b_from_acc(const f32x16& c) {
  u32x4 b;
  if constexpr (sizeof(T) == 2) {
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e] = f32x2_to_bf16x2(c[8 * KG + 2 * e], c[8 * KG + 2 * e + 1]);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e] = __float_as_uint(c[4 * KG + e]);
  }
  return b;
}
// p points at A[row][first contraction index of the k-group]
template <typename T> __device__ __forceinline__ u32x4 frag_a_split(const T* p) {
  const int half = (threadIdx.x & 63) >> 5;
  if constexpr (sizeof(T) == 2) {
    const u32x2 lo = *reinterpret_cast<const u32x2*>(p + 4 * half);
    const u32x2 hi = *reinterpret_cast<const u32x2*>(p + 8 + 4 * half);
    return u32x4{lo[0], lo[1], hi[0], hi[1]};
  } else {
    return *reinterpret_cast<const u32x4*>(p + 4 * half);
  }
}
// all k-groups of one 32x32 accumulator tile packed as operand fragments ("fragment order").  The same 1024
// elements, stored as [k-group][lane][16 bytes], are also the on-memory format in which kernels hand tiles to
// each other: a lane writes/reads 16 contiguous bytes per k-group and never goes through LDS.
// Place of a lane's 16-byte piece inside a stored tile, in pieces: [k-group][half-wave][32 places].  For 16-bit types
// the pieces of block (g, h) are rotated by 4 (2 g + h) places, so that the transposing read, which visits the same
// four rows in all four blocks at once, finds them on different LDS banks (without the rotation they are 512 bytes
// apart: a four-way conflict); a plain load or store still touches every place of a block exactly once.
template <typename T> __device__ __forceinline__ int frag_slot(int g, int lane) {
  if constexpr (sizeof(T) == 2) return g * 64 + (lane & 32) + ((lane + 4 * (2 * g + (lane >> 5))) & 31);
  else return g * 64 + lane;
}
// the tile row (lane % 32 of its owner) of the piece at place p of a stored tile
template <typename T> __device__ __forceinline__ int frag_piece_row(int p) {
  if constexpr (sizeof(T) == 2) return ((p & 31) - 4 * ((p >> 5) & 3)) & 31;
  else return p & 31;
}
template <typename T> struct AccB {
  static constexpr int kG = AccK<T>::kGroups;
  static constexpr int kVecElems = 16 / (int)sizeof(T);   // elements per lane per k-group
  u32x4 f[kG];
  __device__ __forceinline__ void pack(const f32x16& c) {
    f[0] = frag_b_from_acc<T, 0>(c);
    f[1] = frag_b_from_acc<T, 1>(c);
    if constexpr (sizeof(T) == 4) { f[2] = frag_b_from_acc<T, 2>(c); f[3] = frag_b_from_acc<T, 3>(c); }
  }
  __device__ __forceinline__ void negate() {
#pragma unroll
    for (int g = 0; g < kG; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) f[g][e] ^= (sizeof(T) == 2 ? 0x80008000u : 0x80000000u);
  }
  // accumulator values (fp32) of the tile this fragment set was packed from
  __device__ __forceinline__ f32x16 unpack() const {
    f32x16 c;
    if constexpr (sizeof(T) == 2) {
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          c[8 * g + 2 * e] = __uint_as_float(f[g][e] << 16);
          c[8 * g + 2 * e + 1] = __uint_as_float(f[g][e] & 0xffff0000u);
        }
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) c[4 * g + e] = __uint_as_float(f[g][e]);
    }
    return c;
  }
  // tile = first element of this 32x32 tile in a fragment-order buffer (1024 elements per tile)
  __device__ __forceinline__ void store(T* tile) const {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int g = 0; g < kG; ++g) *reinterpret_cast<u32x4*>(tile + frag_slot<T>(g, lane) * kVecElems) = f[g];
  }
  // streaming variant for global tiles that are read again only by a later kernel: the data goes to memory without
  // staying in the L2, which is left to the loads (measured gain on the kernels that stream many tiles: 7-10 %)
  __device__ __forceinline__ void store_stream(T* tile) const {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int g = 0; g < kG; ++g)
      __builtin_nontemporal_store(f[g], reinterpret_cast<u32x4*>(tile + frag_slot<T>(g, lane) * kVecElems));
  }
  __device__ __forceinline__ void load(const T* tile) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int g = 0; g < kG; ++g) f[g] = *reinterpret_cast<const u32x4*>(tile + frag_slot<T>(g, lane) * kVecElems);
  }
  // The fragments of X^T from a tile in LDS that holds X in fragment order: what load() followed by a turn through
  // the matrix core and pack() gives, without either.  Element (lane a, register index b) of a fragment-order tile
  // sits at [k-group of b][a][position of b]; a lane of the transposed set needs a run of consecutive a for one b,
  // which is a column of 16-byte rows: 16-bit types read it with the transposing LDS read, four a at a time.
  __device__ __forceinline__ void load_t(const T* tile) {
    const int lane = threadIdx.x & 63;
    if constexpr (sizeof(T) == 2) {
      const int gr = lane >> 4, i = lane & 15, e = i >> 2, q = i & 3, hh = gr >> 1;
      // this lane fetches columns 4 (q >> 1) .. + 3 of rows 16 g + 8 t + 4 hh + e of the stored block (gr & 1, q & 1),
      // which is rotated by 4 (2 (gr & 1) + (q & 1)) places
      const int rot = 4 * hh + e + 4 * (2 * (gr & 1) + (q & 1));
      const T* base = tile + (((gr & 1) * 64 + 32 * (q & 1)) * 8 + 4 * (q >> 1));
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const u32x2 r = lds_read_tr16(base + ((16 * g + 8 * t + rot) & 31) * 8);
          f[g][2 * t] = r[0];
          f[g][2 * t + 1] = r[1];
        }
    } else {
      const int m = lane & 31, h = lane >> 5;
      const T* base = tile + (((m >> 3) * 64 + 32 * ((m & 7) >> 2) + 4 * h) * 4 + (m & 3));
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) f[g][e] = __float_as_uint(Elem<T>::to_f(base[(8 * g + e) * 4]));
    }
  }
  // From a row-major tile in LDS (x = &X[first row][first column], rows ld elements apart, ld a multiple of 4):
  // lane <-> column, registers <-> row, i.e. X as a B operand contracted over its rows, or, unpack()ed, X in the
  // accumulator layout.
  __device__ __forceinline__ void load_cols(const T* x, int ld) {
    const int lane = threadIdx.x & 63;
    if constexpr (sizeof(T) == 2) {
      const int gr = lane >> 4, i = lane & 15, e = i >> 2, q = i & 3, hh = gr >> 1;
      const T* base = x + (4 * hh + e) * ld + (gr & 1) * 16 + 4 * q;
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const u32x2 r = lds_read_tr16(base + (16 * g + 8 * t) * ld);
          f[g][2 * t] = r[0];
          f[g][2 * t + 1] = r[1];
        }
    } else {
      const int m = lane & 31, h = lane >> 5;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) f[g][e] = __float_as_uint(Elem<T>::to_f(x[(8 * g + 4 * h + e) * ld + m]));
    }
  }
  // As load_cols for 16-bit types, but the 8 rows a lane holds of k-group g are consecutive, 16 g + 8 (lane >> 5) + 0..7:
  // the k order of an A operand that is read with one 16-byte read per k-group straight from a row-major tile.
  __device__ __forceinline__ void load_cols_consecutive(const T* x, int ld) {
    static_assert(sizeof(T) == 2, "16-bit types");
    const int lane = threadIdx.x & 63;
    const int gr = lane >> 4, i = lane & 15, e = i >> 2, q = i & 3, hh = gr >> 1;
    const T* base = x + (8 * hh + e) * ld + (gr & 1) * 16 + 4 * q;
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const u32x2 r = lds_read_tr16(base + (16 * g + 4 * t) * ld);
        f[g][2 * t] = r[0];
        f[g][2 * t + 1] = r[1];
      }
  }
};
// d(32x32) += A[32 rows][32 k] * B(32 k x 32) with B packed from an accumulator; arow = &A[row of this lane][k0]
template <typename T> __device__ __forceinline__ void mma32_accb(f32x16& d, const T* arow, const AccB<T>& b) {
  constexpr int G = KGroup<T>::kLen;
#pragma unroll
  for (int kg = 0; kg < AccK<T>::kGroups; ++kg) mfma_kgroup<T>(d, frag_a_split<T>(arow + G * kg), b.f[kg]);
}
// both operands in fragment order: d += A(32 x 32k) * B(32k x 32)
template <typename T> __device__ __forceinline__ void mma32_ff(f32x16& d, const AccB<T>& a, const AccB<T>& b) {
#pragma unroll
  for (int kg = 0; kg < AccK<T>::kGroups; ++kg) mfma_kgroup<T>(d, a.f[kg], b.f[kg]);
}
// fragments of a tile stored in LDS with the contraction index contiguous: row = &tile[row of this lane][k0]
template <typename T> __device__ __forceinline__ void frags_from_lds(AccB<T>& out, const T* row) {
  constexpr int G = KGroup<T>::kLen;
#pragma unroll
  for (int kg = 0; kg < AccK<T>::kGroups; ++kg) out.f[kg] = frag_a_split<T>(row + G * kg);
}

// A row-major [rows][COLS] tile in LDS without padding, as a direct global -> LDS copy leaves it (64 lanes x 16 bytes
// per instruction, contiguous).  Its rows are a multiple of 64 bytes apart, so the lanes of a fragment read, one row
// each, would meet on a few of the 64 banks.  The 16-byte pieces of row r are therefore stored permuted, piece c at
// position pos(r, c) = c ^ key(r) (an involution: the copy applies it to its source addresses), with the key chosen so
// that 16 consecutive rows cover all the banks.
template <typename T, int COLS> struct SwizzledTile {
  static constexpr int kVec = 16 / (int)sizeof(T), kPieces = COLS / kVec;   // pieces per row
  static_assert(kPieces >= 4 && (kPieces & (kPieces - 1)) == 0, "rows of 4, 8, 16, ... pieces");
  static __device__ __forceinline__ int key(int r) {
    if constexpr (kPieces >= 16) return r & 15;
    else return (r / (16 / kPieces)) & (kPieces - 1);
  }
  static __device__ __forceinline__ int pos(int r, int c) { return c ^ key(r); }
  // A-operand fragments of columns [k0, k0 + 32) of row r (lane <-> row r, registers <-> the 32 columns)
  static __device__ __forceinline__ void frags(AccB<T>& out, const T* tile, int r, int k0) {
    const int half = (threadIdx.x & 63) >> 5, c0 = k0 / kVec;
    const T* row = tile + r * COLS;
#pragma unroll
    for (int kg = 0; kg < AccK<T>::kGroups; ++kg) {
      if constexpr (sizeof(T) == 2) {
        const u32x2 lo = *reinterpret_cast<const u32x2*>(row + pos(r, c0 + 2 * kg) * 8 + 4 * half);
        const u32x2 hi = *reinterpret_cast<const u32x2*>(row + pos(r, c0 + 2 * kg + 1) * 8 + 4 * half);
        out.f[kg] = u32x4{lo[0], lo[1], hi[0], hi[1]};
      } else {
        out.f[kg] = *reinterpret_cast<const u32x4*>(row + pos(r, c0 + 2 * kg + half) * 4);
      }
    }
  }
};

// Cross-lane transpose through the matrix core.  A tile held as fragments with (lane <-> a, registers <-> b)
// multiplied by the identity comes back as an accumulator with (lane <-> b, registers <-> a): C = X * I read as
// A operand X[a][b].  Exact (products with 1.0, sums with 0).  Costs kGroups MFMA k-groups per 32x32 tile.
template <typename T> struct IdentityFrag {
  u32x4 f[AccK<T>::kGroups];
  __device__ __forceinline__ void init() {
    const int lane = threadIdx.x & 63, n = lane & 31, half = lane >> 5;
#pragma unroll
    for (int g = 0; g < AccK<T>::kGroups; ++g) {
      if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int k0 = 16 * g + 8 * ((2 * e) >> 2) + 4 * half + ((2 * e) & 3);
          const int k1 = 16 * g + 8 * ((2 * e + 1) >> 2) + 4 * half + ((2 * e + 1) & 3);
          f[g][e] = (k0 == n ? 0x3f80u : 0u) | (k1 == n ? 0x3f800000u : 0u);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) f[g][e] = (8 * g + 4 * half + e == n) ? 0x3f800000u : 0u;
      }
    }
  }
};
template <typename T>
__device__ __forceinline__ f32x16 mfma_transpose(const AccB<T>& x, const IdentityFrag<T>& id) {
  f32x16 c = acc_zero();
#pragma unroll
  for (int kg = 0; kg < AccK<T>::kGroups; ++kg) mfma_kgroup<T>(c, x.f[kg], id.f[kg]);
  return c;
}

__device__ __forceinline__ f32x16 acc_zero() {
  f32x16 z;
#pragma unroll
  for (int r = 0; r < 16; ++r) z[r] = 0.f;
  return z;
}
// coordinates of accumulator register r of this lane inside the 32x32 tile
__device__ __forceinline__ int acc_row(int r) { return 8 * (r >> 2) + 4 * ((threadIdx.x & 63) >> 5) + (r & 3); }
__device__ __forceinline__ int acc_col() { return threadIdx.x & 31; }

// accumulator tile -> LDS, transposed: dst[(j0+j)*ld + i0 + i].  Registers 4g..4g+3 are four consecutive rows, so a
// lane writes four contiguous elements at a time (ld must be a multiple of 4 elements).  dst may also be global
// memory; with ld = 0 it is the address of the lane's own row.
template <typename T> __device__ __forceinline__ void acc_to_lds_t(const f32x16& acc, T* dst, int ld, int i0, int j0) {
  T* col = dst + (j0 + acc_col()) * ld + i0 + 4 * ((threadIdx.x & 63) >> 5);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    if constexpr (sizeof(T) == 2) {
      *reinterpret_cast<u32x2*>(col + 8 * g) =
          u32x2{f32x2_to_bf16x2(acc[4 * g], acc[4 * g + 1]), f32x2_to_bf16x2(acc[4 * g + 2], acc[4 * g + 3])};
    } else {
      *reinterpret_cast<f32x4*>(col + 8 * g) = f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    }
  }
}
// accumulator tile -> global memory, transposed, for 16-bit types: `row` is this lane's own row of the destination
// (column acc_col() of the tile) at the tile's first column.  acc_to_lds_t with ld = 0 writes it in 8-byte pieces: the
// lower half-wave has columns 8g..8g+3 of a row, the upper one 8g+4..8g+7.  Here the half-waves trade pieces first
// (v_permlane32_swap: the upper half of the first register with the lower half of the second), so that the lower one
// holds columns 16p..16p+7 and the upper one 16p+8..16p+15: two 16-byte stores per lane instead of four of 8 bytes.
// Every lane of the wave must call it (the trade); `live` says whether this lane's row exists.
template <typename T> __device__ __forceinline__ void acc_store_t_rows16(const f32x16& acc, T* row, bool live) {
  static_assert(sizeof(T) == 2, "16-bit types");
  const int half = (threadIdx.x & 63) >> 5;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    u32x4 w;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const uint32_t x = f32x2_to_bf16x2(acc[8 * p + 2 * e], acc[8 * p + 2 * e + 1]);          // group 2p
      const uint32_t y = f32x2_to_bf16x2(acc[8 * p + 4 + 2 * e], acc[8 * p + 4 + 2 * e + 1]);  // group 2p + 1
      const auto r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
      w[e] = r[0];
      w[2 + e] = r[1];
    }
    if (live) *reinterpret_cast<u32x4*>(row + 16 * p + 8 * half) = w;   // every lane trades, lanes of rows past the end do not store
  }
}
// accumulator tile -> LDS, row-major, by way of the matrix core: the tile is rounded to T, transposed (exact) and
// then written like a transposed tile, four contiguous elements per lane and store instead of one.
template <typename T>
__device__ __forceinline__ void acc_to_lds_rm(const f32x16& acc, const IdentityFrag<T>& id, T* dst, int ld, int i0, int j0) {
  AccB<T> b;
  b.pack(acc);
  acc_to_lds_t(mfma_transpose<T>(b, id), dst, ld, j0, i0);
}
// 16 per-row values (fp32, in LDS at arr[i0 + row]) for the rows of this lane's accumulator registers
__device__ __forceinline__ f32x16 rows_ld(const float* arr, int i0) {
  const float* p = arr + i0 + 4 * ((threadIdx.x & 63) >> 5);
  f32x16 v;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p + 8 * g);
    v[4 * g] = t[0]; v[4 * g + 1] = t[1]; v[4 * g + 2] = t[2]; v[4 * g + 3] = t[3];
  }
  return v;
}
// Data-parallel-primitive moves between lanes run at VALU speed; wave shuffles (ds_bpermute) go through the LDS
// crossbar and cost ~10x more.
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// sum over aligned groups of N neighbouring lanes (N a power of two <= 32), every lane gets the result
template <int N> __device__ __forceinline__ float lane_group_sum(float v) {
  if constexpr (N >= 2) v += dpp_mov<0xB1>(v);
  if constexpr (N >= 4) v += dpp_mov<0x4E>(v);
  if constexpr (N >= 8) v += dpp_mov<0x141>(v);
  if constexpr (N >= 16) v += dpp_mov<0x140>(v);
  if constexpr (N >= 32) v += __shfl_xor(v, 16);
  return v;
}

// Row sums of a 32x32 tile given as per-lane products x[r] (accumulator layout).  A halving butterfly over the 16
// lanes of a DPP row: at each step a lane keeps the pair sums of the registers whose index bit matches its own lane bit, so 16 sums cost 15 exchanges instead of 64.  Lane l returns the sum over its DPP row of
// register r = l & 15, i.e. a partial sum (16 of the 32 columns) of tile row acc_row(l & 15).
__device__ __forceinline__ float rows16_partial(const f32x16& x) {
  const int lane = threadIdx.x;
  const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4, b3 = lane & 8;
  // both candidate sums are formed and one is kept: a select between two register elements would be folded into a
  // dynamically indexed element read, which the backend expands into a 16-way compare/select chain
  float a[8], b[4], c[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float lo = x[2 * i] + dpp_mov<0xB1>(x[2 * i]), hi = x[2 * i + 1] + dpp_mov<0xB1>(x[2 * i + 1]);
    a[i] = b0 ? hi : lo;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = a[2 * i] + dpp_mov<0x4E>(a[2 * i]), hi = a[2 * i + 1] + dpp_mov<0x4E>(a[2 * i + 1]);
    b[i] = b1 ? hi : lo;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {   // row_ror:4
    const float lo = b[2 * i] + dpp_mov<0x124>(b[2 * i]), hi = b[2 * i + 1] + dpp_mov<0x124>(b[2 * i + 1]);
    c[i] = b2 ? hi : lo;
  }
  const float lo = c[0] + dpp_mov<0x128>(c[0]), hi = c[1] + dpp_mov<0x128>(c[1]);   // row_ror:8
  return b3 ? hi : lo;
}
// rowacc[wave][i0 + i] += sum_j x[i][j] for the 32 rows of the tile.  rowacc is an LDS array [4 waves][64 rows]:
// every wave owns a slot and every row of a slot is always updated by the same lane, so no atomics are needed and the
// result does not depend on the order in which waves arrive (readers add the four slots in a fixed order).
__device__ __forceinline__ void rows_add(const f32x16& x, float* rowacc, int i0) {
  float s = rows16_partial(x);
  s += __shfl_xor(s, 16);     // the other half of the 32 columns
  const int lane = threadIdx.x & 63;
  if ((lane & 16) == 0) rowacc[(threadIdx.x >> 6) * 64 + i0 + acc_row(lane & 15)] += s;
}
// sum over the four wave slots of such an array, for the rows of this lane's accumulator registers
__device__ __forceinline__ f32x16 rows_ld(const float* arr, int i0);
__device__ __forceinline__ f32x16 rows_ld4(const float* arr, int i0) {
  f32x16 a = rows_ld(arr, i0);
#pragma unroll
  for (int w = 1; w < 4; ++w) {
    const f32x16 b = rows_ld(arr + 64 * w, i0);
#pragma unroll
    for (int r = 0; r < 16; ++r) a[r] += b[r];
  }
  return a;
}

// One wave: 32x32 accumulator tile -> 32 global rows of 32 columns (tile row i at g + i*row_stride), written as
// 16-byte pieces after a pass through a wave-private LDS patch of 32 x kPatchLd elements.  Element-wise stores of
// an accumulator tile (2 bytes per lane, 16 instructions) are several times slower than these.
template <typename T> struct Patch { static constexpr int kLd = 32 + 16 / (int)sizeof(T), kElems = 32 * kLd; };
// What global memory holds at the rows such a tile will be added to: requested by rows_request() well before
// acc_store_rows() adds and writes back, so that the requests of several tiles are in flight together and none of
// them is issued behind a store (loads and stores complete in one order: a load issued after a store is not seen
// before that store has been acknowledged).  Rows past the end repeat the last valid one: the same loads on every path.
template <typename T> struct RowPieces {
  static constexpr int kN = 32 * (32 / Elem<T>::kVec) / 64;   // 16-byte pieces per lane
  Vec16<T> y[kN];
};
template <typename T>
__device__ __forceinline__ void rows_request(RowPieces<T>& r, const T* g, int64_t row_stride, int rows_valid) {
  constexpr int V = Elem<T>::kVec, PPR = 32 / V;
  const int lane = threadIdx.x & 63;
  if (rows_valid <= 0) return;   // wave-uniform; no row of the tile exists (its first row may lie past the tensor's end)
#pragma unroll
  for (int i = 0; i < RowPieces<T>::kN; ++i) {
    const int p = lane + 64 * i, row = imin(p / PPR, rows_valid - 1), cc = p % PPR;
    r.y[i] = ld16(g + (int64_t)row * row_stride + cc * V);
  }
}
// The same requests for either of two sources, chosen by the wave-uniform `frag` on the addresses: the rows of
// rows_request, or a 32x32 tile in fragment order (what AccB::load reads; as_frag() gives it that type).  A branch
// between the two kinds of request would join with loaded registers, and the compiler waits for them there.  Unlike
// rows_request this asks also when the tile has no valid row: `g` must then point 32 rows past a block whose rows
// exist (rows_valid >= -31: the row index goes back into that block).
template <typename T>
__device__ __forceinline__ void rows_or_tile_request(RowPieces<T>& r, bool frag, const T* tile, const T* g,
                                                     int64_t row_stride, int rows_valid) {
  constexpr int V = Elem<T>::kVec, PPR = 32 / V;
  static_assert(RowPieces<T>::kN == AccB<T>::kG, "a lane holds as many 16-byte pieces of a tile either way");
  int lane = threadIdx.x & 63;
  GDN_KEEP_HERE(lane);   // the offsets are formed here: shared with an equal expression far above they would sit in a
                         // register (or in scratch memory) through the phases between
  // a uniform base and one 32-bit offset per piece (never negative: the rows are counted from 32 rows before g)
  const T* base = frag ? tile : g - 32 * row_stride;
#pragma unroll
  for (int i = 0; i < RowPieces<T>::kN; ++i) {
    const int p = lane + 64 * i, row = imin(p / PPR, rows_valid - 1), cc = p % PPR;
    const uint32_t off = frag ? (uint32_t)(frag_slot<T>(i, lane) * AccB<T>::kVecElems)
                              : (uint32_t)((row + 32) * (int)row_stride + cc * V);
    r.y[i] = ld16(base + off);
  }
}
template <typename T> __device__ __forceinline__ AccB<T> as_frag(const RowPieces<T>& r) {
  AccB<T> f;
#pragma unroll
  for (int i = 0; i < AccB<T>::kG; ++i) f.f[i] = r.y[i].raw;
  return f;
}
// ADD: the rows are added to `held` (what memory held, see rows_request) before they are written.
template <typename T, bool ADD>
__device__ __forceinline__ void acc_store_rows(const f32x16& acc, const IdentityFrag<T>& id, T* patch, T* g,
                                               int64_t row_stride, int rows_valid, const RowPieces<T>& held) {
  constexpr int PLD = Patch<T>::kLd, V = Elem<T>::kVec, PPR = 32 / V, NP = RowPieces<T>::kN;
  const int lane = threadIdx.x & 63;
  if (rows_valid <= 0) return;   // wave-uniform
  GDN_WAVE_LDS_SYNC();   // earlier readers of the patch are done
  acc_to_lds_rm(acc, id, patch, PLD, 0, 0);
  GDN_WAVE_LDS_SYNC();
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = lane + 64 * i, row = p / PPR, cc = p % PPR;
    Vec16<T> x = ld16(patch + row * PLD + cc * V);
    if constexpr (ADD) {
      float fx[V], fy[V];
      unpack16<T>(x, fx);
      unpack16<T>(held.y[i], fy);
#pragma unroll
      for (int e = 0; e < V; ++e) fx[e] += fy[e];
      x = pack16<T>(fx);
    }
    if (row < rows_valid) st16(g + (int64_t)row * row_stride + cc * V, x);
  }
  GDN_WAVE_LDS_SYNC();   // the patch may be overwritten (also by a direct global->LDS load) once every lane has read it
}
template <typename T, bool ADD>
__device__ __forceinline__ void acc_store_rows(const f32x16& acc, const IdentityFrag<T>& id, T* patch, T* g,
                                               int64_t row_stride, int rows_valid) {
  static_assert(!ADD, "adding needs the rows requested beforehand");
  RowPieces<T> none;
  acc_store_rows<T, false>(acc, id, patch, g, row_stride, rows_valid, none);
}

// sum over the 32 lanes that share a half-wave (all columns of one accumulator row)
__device__ __forceinline__ float half_wave_sum(float v) {
  v += __shfl_xor(v, 16);
  v += __shfl_xor(v, 8);
  v += __shfl_xor(v, 4);
  v += __shfl_xor(v, 2);
  v += __shfl_xor(v, 1);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  v += __shfl_xor(v, 32);
  return half_wave_sum(v);
}

// A [64, DK] q or k tile on its way into LDS, in two steps so that the requests of both tiles (and of the gates) are
// in flight together instead of one 16-byte piece at a time: tile_qk_request() issues this thread's loads (rows past
// the end of the sequence are zero), tile_qk_finish() applies the optional l2 norm (y = x rsqrt(sum x^2 + 1e-6) over
// the row, modeling_qwen3_5.py:392-395; fp32 arithmetic, result rounded to T; a row sits on DK/VEC neighbouring lanes
// that combine their partial sums with data-parallel-primitive moves), writes the tile to
// LDS and, on request, the normalised rows (row stride y_stride) and 1/|x| (stride rstd_stride) to global memory.
// NT: the threads that move the tile (tid = 0 .. NT - 1).
template <typename T, int DK, int NT = kThreads> struct TileQK {
  static constexpr int V = Elem<T>::kVec, CPR = DK / V, PT = 64 * CPR / NT;   // lanes per row; pieces per thread
  static_assert((64 * CPR) % NT == 0, "every thread takes the same number of pieces");
  Vec16<T> x[PT];
};
template <typename T, int DK, int NT>
__device__ __forceinline__ void tile_qk_request(TileQK<T, DK, NT>& t, const T* g, int64_t row_stride, int nvalid, int tid) {
  constexpr int V = TileQK<T, DK, NT>::V, CPR = TileQK<T, DK, NT>::CPR;
#pragma unroll
  for (int i = 0; i < TileQK<T, DK, NT>::PT; ++i) {
    const int c = tid + i * NT, row = c / CPR, cc = c % CPR;
    t.x[i] = ld16(g + (int64_t)imin(row, nvalid - 1) * row_stride + cc * V);   // the same load on every path
  }
}
template <typename T, int DK, int NT>
__device__ __forceinline__ void tile_qk_finish(TileQK<T, DK, NT>& t, T* lds, int ld, int nvalid, int tid, bool l2norm,
                                               T* y_out, int64_t y_stride, float* rstd_out, int64_t rstd_stride) {
  constexpr int V = TileQK<T, DK, NT>::V, CPR = TileQK<T, DK, NT>::CPR;
#pragma unroll
  for (int i = 0; i < TileQK<T, DK, NT>::PT; ++i) {
    const int c = tid + i * NT, row = c / CPR, cc = c % CPR;
    const bool ok = row < nvalid;
    Vec16<T> x = ok ? t.x[i] : zero16<T>();
    if (l2norm) {   // uniform: every lane takes part in the shuffles
      float f[V], ss = 0.f;
      unpack16<T>(x, f);
#pragma unroll
      for (int e = 0; e < V; ++e) ss += f[e] * f[e];
      ss = lane_group_sum<CPR>(ss);
      const float r = __builtin_amdgcn_rsqf(ss + 1e-6f);   // the instruction alone: its argument is never subnormal
#pragma unroll
      for (int e = 0; e < V; ++e) f[e] *= r;
      x = pack16<T>(f);
      if (ok && y_out != nullptr) st16(y_out + (int64_t)row * y_stride + cc * V, x);
      if (ok && rstd_out != nullptr && cc == 0) rstd_out[(int64_t)row * rstd_stride] = r;
    }
    st16(lds + row * ld + cc * V, x);
  }
}

// ---------------------------------------------------------------------------------------------
// Packed-sequence bookkeeping.  chunk_offsets[n] = number of 64-token chunks before sequence n
// (chunk_offsets[N] = total); built on the device by gdn_chunk_table_kernel so that no host sync is
// needed.  Without cu_seqlens every batch row is a sequence of T tokens.
// ---------------------------------------------------------------------------------------------
struct SeqInfo {
  int n;        // sequence index
  int64_t bos;  // first token (index into the flattened [B*T] token axis)
  int len;      // tokens in this sequence
  int chunk;    // chunk index inside the sequence
  int nvalid;   // valid tokens of this chunk (1..64), 0 if the chunk does not exist
};

__device__ __forceinline__ SeqInfo locate_chunk(int gchunk, const int64_t* cu_seqlens, const int* chunk_offsets,
                                                int N, int T) {
  SeqInfo s;
  if (cu_seqlens == nullptr) {
    const int nt = (T + kChunk - 1) / kChunk;
    s.n = gchunk / nt;
    s.chunk = gchunk % nt;
    s.bos = (int64_t)s.n * T;
    s.len = T;
    s.nvalid = s.n < N ? imin(kChunk, T - s.chunk * kChunk) : 0;
    return s;
  }
  if (gchunk >= chunk_offsets[N]) { s.n = 0; s.bos = 0; s.len = 0; s.chunk = 0; s.nvalid = 0; return s; }
  int lo = 0, hi = N - 1;  // last n with chunk_offsets[n] <= gchunk
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (chunk_offsets[mid] <= gchunk) lo = mid; else hi = mid - 1;
  }
  s.n = lo;
  s.bos = cu_seqlens[lo];
  s.len = (int)(cu_seqlens[lo + 1] - s.bos);
  s.chunk = gchunk - chunk_offsets[lo];
  s.nvalid = imin(kChunk, s.len - s.chunk * kChunk);
  return s;
}

// Rows of packed outputs that belong to no sequence: with cu_seqlens on the device the host cannot check that the last
// entry equals the number of tokens, and the kernels visit listed chunks only, so rows past cu_seqlens[N] would keep
// whatever the allocation held.  One workgroup per 64 rows; those before the end of the last sequence leave at once.
struct TailRows {
  void* base[6];              // null entries are skipped
  int64_t row_stride[6];      // bytes between consecutive tokens
  int row_bytes[6];           // bytes to clear per token (a multiple of 2)
};
static __global__ void zero_tail_rows_kernel(const int64_t* __restrict__ cu, int N, int64_t tokens, TailRows t) {
  const int64_t covered = cu[N], lo = (int64_t)blockIdx.x * 64, hi = lo + 64 < tokens ? lo + 64 : tokens;
  if (hi <= covered) return;
  const int64_t first = lo > covered ? lo : covered;
  for (int a = 0; a < 6; ++a) {
    if (t.base[a] == nullptr) continue;
    unsigned char* b = static_cast<unsigned char*>(t.base[a]);
    if (t.row_bytes[a] % 4 == 0 && t.row_stride[a] % 4 == 0) {
      const int words = t.row_bytes[a] / 4;
      for (int64_t i = threadIdx.x; i < (hi - first) * words; i += blockDim.x)
        reinterpret_cast<uint32_t*>(b + (first + i / words) * t.row_stride[a])[i % words] = 0u;
    } else {   // rows of an odd number of 16-bit values
      const int halves = t.row_bytes[a] / 2;
      for (int64_t i = threadIdx.x; i < (hi - first) * halves; i += blockDim.x)
        reinterpret_cast<uint16_t*>(b + (first + i / halves) * t.row_stride[a])[i % halves] = 0;
    }
  }
}
static inline void launch_zero_tail_rows(const int64_t* cu, int N, int64_t tokens, const TailRows& t, hipStream_t st) {
  if (cu == nullptr || tokens <= 0) return;
  hipLaunchKernelGGL(zero_tail_rows_kernel, dim3((unsigned)((tokens + 63) / 64)), dim3(256), 0, st, cu, N, tokens, t);
}

}  // namespace gdn
