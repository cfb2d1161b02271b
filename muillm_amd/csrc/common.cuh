// Shared device helpers for the gfx950 decode kernels: 128-bit streaming loads,
// 16-bit <-> fp32 conversion, wave64 reductions built from DPP + readlane.
//
// Everything here assumes wavefront size 64 (CDNA4) and is compiled for gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/muillm_amd.h"
#include "../../include/muillm_amd_tune.h"

namespace mui {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------
// element types: storage is 16 bits, arithmetic is fp32
// ---------------------------------------------------------------------------------------
struct F16 {
  static constexpr int kDtype = MUI_DTYPE_F16;
  // low / high half of a packed 32-bit word -> fp32
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(f16x2, w).x;
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(f16x2, w).y;
  }
  static __device__ __forceinline__ float one(uint16_t b) {
    return (float)__builtin_bit_cast(_Float16, b);
  }
  // fp32 -> 16 bit storage, round-to-nearest-even (single rounding)
  static __device__ __forceinline__ uint16_t pack(float v) {
    return __builtin_bit_cast(uint16_t, (_Float16)v);
  }
  // two values -> one packed word (a in the low half): one v_cvt_pk_f16_f32, same rounding
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
};

struct BF16 {
  static constexpr int kDtype = MUI_DTYPE_BF16;
  static __device__ __forceinline__ float lo(uint32_t w) {
    return __builtin_bit_cast(float, w << 16);
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return __builtin_bit_cast(float, w & 0xffff0000u);
  }
  static __device__ __forceinline__ float one(uint16_t b) {
    return __builtin_bit_cast(float, ((uint32_t)b) << 16);
  }
  // fp32 -> bf16, round-to-nearest-even: the hardware convert of gfx950 (v_cvt_pk_bf16_f32)
  static __device__ __forceinline__ uint16_t pack(float v) {
    return __builtin_bit_cast(uint16_t, (__bf16)v);
  }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
  }
};

template <typename T>
__device__ __forceinline__ void unpack8(const u32x4 w, float (&f)[8]) {
  f[0] = T::lo(w.x); f[1] = T::hi(w.x);
  f[2] = T::lo(w.y); f[3] = T::hi(w.y);
  f[4] = T::lo(w.z); f[5] = T::hi(w.z);
  f[6] = T::lo(w.w); f[7] = T::hi(w.w);
}

template <typename T>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
  u32x4 w;
  w.x = (uint32_t)T::pack(f[0]) | ((uint32_t)T::pack(f[1]) << 16);
  w.y = (uint32_t)T::pack(f[2]) | ((uint32_t)T::pack(f[3]) << 16);
  w.z = (uint32_t)T::pack(f[4]) | ((uint32_t)T::pack(f[5]) << 16);
  w.w = (uint32_t)T::pack(f[6]) | ((uint32_t)T::pack(f[7]) << 16);
  return w;
}

// ---------------------------------------------------------------------------------------
// loads. Weights are read exactly once per call, so they are streamed with the
// non-temporal hint; small reused vectors (x, gamma) use ordinary cached loads.
// ---------------------------------------------------------------------------------------
// Every pointer these helpers see is device memory, so the global address space is named
// explicitly: where the compiler cannot infer it (a pointer selected between two kernel
// arguments, for instance) it would otherwise emit flat loads, which also occupy the LDS
// counter and serialise against LDS traffic.
typedef const __attribute__((address_space(1))) u32x4* global_u32x4_ptr;
typedef const __attribute__((address_space(1))) u32x2* global_u32x2_ptr;
__device__ __forceinline__ u32x4 ld16_stream(const void* p) {
  return __builtin_nontemporal_load((global_u32x4_ptr)p);
}
__device__ __forceinline__ u32x4 ld16(const void* p) { return *(global_u32x4_ptr)p; }
__device__ __forceinline__ u32x2 ld8_stream(const void* p) {
  return __builtin_nontemporal_load((global_u32x2_ptr)p);
}
__device__ __forceinline__ u32x2 ld8(const void* p) { return *(global_u32x2_ptr)p; }
__device__ __forceinline__ uint32_t ld4(const void* p) {
  return *(const __attribute__((address_space(1))) uint32_t*)p;
}
__device__ __forceinline__ uint16_t ld2(const void* p) {
  return *(const __attribute__((address_space(1))) uint16_t*)p;
}

template <bool STREAM>
__device__ __forceinline__ u32x4 ld16_sel(const void* p) {
  if constexpr (STREAM) return ld16_stream(p); else return ld16(p);
}

// ---------------------------------------------------------------------------------------
// wave64 reductions. Within a row of 16 lanes the butterfly runs on DPP (no LDS traffic);
// the four row totals are then fetched with v_readlane, giving a wave-uniform result.
// ---------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  int i = __builtin_bit_cast(int, v);
  i = __builtin_amdgcn_update_dpp(0, i, CTRL, 0xf, 0xf, false);
  return __builtin_bit_cast(float, i);
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i within 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i within 16

// every lane of each 16-lane row ends up holding that row's total
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<kDppXor1>(v);
  v += dpp_f32<kDppXor2>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppMirror>(v);
  return v;
}
__device__ __forceinline__ float row16_max(float v) {
  v = fmaxf(v, dpp_f32<kDppXor1>(v));
  v = fmaxf(v, dpp_f32<kDppXor2>(v));
  v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_f32<kDppMirror>(v));
  return v;
}

__device__ __forceinline__ float readlane_f32(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// total over all 64 lanes, uniform across the wave
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  return (readlane_f32(v, 0) + readlane_f32(v, 16)) + (readlane_f32(v, 32) + readlane_f32(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = row16_max(v);
  return fmaxf(fmaxf(readlane_f32(v, 0), readlane_f32(v, 16)),
               fmaxf(readlane_f32(v, 32), readlane_f32(v, 48)));
}

// Reduce N values (N = 2, 4, 8 or 16) over each 16-lane row at once. Every DPP exchange step
// also halves the number of values a lane carries (the lower lane of a pair keeps the first
// half, the upper lane the second half, each adds what its partner sends), so the whole
// reduction costs about 3 N instructions instead of 4 N adds + N broadcasts. Afterwards v[0]
// of lane i holds the row's total of value (i % 16) / (16 / N). Pair order mirror(16) ->
// mirror(8) -> xor 2 -> xor 1 keeps partners on the same value subset at every step.
template <int CTRL, int HALF, int N>
__device__ __forceinline__ void row16_scatter_step(float (&v)[N], bool upper) {
#pragma unroll
  for (int i = 0; i < HALF; ++i) {
    const float keep = upper ? v[i + HALF] : v[i];
    const float send = upper ? v[i] : v[i + HALF];
    v[i] = keep + dpp_f32<CTRL>(send);
  }
}
template <int N>
__device__ __forceinline__ void row16_reduce_scatter(float (&v)[N], int lane) {
  static_assert(N == 2 || N == 4 || N == 8 || N == 16, "N must be 2, 4, 8 or 16");
  row16_scatter_step<kDppMirror, N / 2, N>(v, (lane & 8) != 0);
  if constexpr (N >= 4) row16_scatter_step<kDppHalfMirror, N / 4, N>(v, (lane & 4) != 0);
  else v[0] += dpp_f32<kDppHalfMirror>(v[0]);
  if constexpr (N >= 8) row16_scatter_step<kDppXor2, N / 8, N>(v, (lane & 2) != 0);
  else v[0] += dpp_f32<kDppXor2>(v[0]);
  if constexpr (N >= 16) row16_scatter_step<kDppXor1, N / 16, N>(v, (lane & 1) != 0);
  else v[0] += dpp_f32<kDppXor1>(v[0]);
}

// Pulls [base, base + bytes) into the cache hierarchy with ordinary (cacheable) 128-bit loads and
// drops the data: work for workgroups that would otherwise idle while a latency-bound kernel runs,
// so that the next, bandwidth-bound kernel finds (part of) its weights on chip. The range is cut
// into slabs of slab_bytes; slab s goes to warm workgroup s % n_wg. Workgroups are handed to the
// eight XCDs round-robin by linear workgroup id, and each XCD has its own L2: with n_wg a multiple
// of 8 and the warm workgroups starting at a linear id that is one too, slab s lands in the L2 of
// XCD s % 8 -- where the consumer's workgroup s % 8 (mod 8) will look for it. Loads are issued
// eight at a time with clamped addresses (no load behind a branch).
template <int kBatch = 8>
__device__ __forceinline__ void warm_cache(const char* base, long bytes, int slab_bytes, int wg, int n_wg, int tid,
                                           int n_threads, int delay = 0) {
  // optional head start for the workgroups doing the launch's real work: their first dependent loads
  // go out before this traffic fills the memory queues (one unit = s_sleep 8, about a quarter
  // microsecond)
  for (int i = 0; i < delay; ++i) __builtin_amdgcn_s_sleep(8);
  const long n_slabs = (bytes + slab_bytes - 1) / slab_bytes;
  const long my_slabs = wg < n_slabs ? (n_slabs - wg + n_wg - 1) / n_wg : 0;
  const int per_slab = (slab_bytes / 16 + n_threads - 1) / n_threads;  // loads per thread and slab
  const long n_loads = my_slabs * per_slab;
  for (long i0 = 0; i0 < n_loads; i0 += kBatch) {
    u32x4 v[kBatch];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      long i = i0 + j;
      i = i < n_loads ? i : 0;
      const long slab = wg + (i / per_slab) * n_wg;
      long off = slab * slab_bytes + ((i % per_slab) * (long)n_threads + tid) * 16;
      off = off + 16 <= bytes ? off : 0;
      v[j] = ld16(base + off);
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j) asm volatile("" ::"v"(v[j]));
  }
}

__device__ __forceinline__ float silu_f32(float x) { return x / (1.0f + __expf(-x)); }

// host-side helpers ----------------------------------------------------------------------
// true once mui_tune_lock() has been called: every mui_tune_* call is refused from then on
bool tune_locked();
#define MUI_TUNE_GUARD()                              \
  do {                                                \
    if (mui::tune_locked()) return MUI_ERR_UNSUPPORTED; \
  } while (0)

static inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }
static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

#define MUI_CHECK_ARG(cond)                 \
  do {                                      \
    if (!(cond)) return MUI_ERR_INVALID_ARG; \
  } while (0)

// number of compute units of the current device (cached; this library drives one GPU)
static inline int device_cus() {
  static int cached = 0;
  if (cached == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    cached = cus;
  }
  return cached;
}

// Persistent grid: at most `per_cu` workgroups per CU, and every workgroup gets the same
// number of work items (a ragged last pass would idle most of the chip for one latency).
static inline int balanced_grid(int n_items, int per_cu) {
  const int cap = device_cus() * per_cu;
  if (n_items <= cap) return n_items;
  const int iters = ceil_div(n_items, cap);
  return ceil_div(n_items, iters);
}

static inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? MUI_OK : MUI_ERR_LAUNCH;
}

}  // namespace mui
