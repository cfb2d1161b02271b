// Measurement aid (no counterpart in the reference): a chain of dependent fp16 GEMVs
//   x_{i+1} = W_i . x_i        (W_i: n x k row-major, distinct buffers, k <= 4096, n % 4 == 0)
// launched two ways, to price what a kernel boundary costs against a hand-off in memory:
//   mode 0  ordinary launches: every kernel waits for the one before it (the barrier bit of its
//           dispatch packet), which is what every launch of this library does;
//   mode 1  launches that may start before their predecessor has finished (no barrier bit): a
//           kernel requests its first weight rows at once, then waits on arrival counters that the
//           workgroups of its predecessor bump after their last store, and only then reads x.
// Hand-off protocol of mode 1: the producer stores y with agent-scope (write-through) stores, waits
// for their completion, and adds 1 to one of eight counters (workgroup id mod 8, 256 bytes apart);
// the consumer's lanes 0..7 poll the eight counters (agent-scope loads) until each shows the
// producer's share of workgroups. Every wait is bounded: after spin_limit polls the kernel sets
// *err and goes on, so that every kernel of the chain exits whatever happens. A kernel never waits
// for a kernel launched after it, and the queue hands workgroups out in launch order, so the
// producer's workgroups are always resident or done when a consumer spins.
#include <hip/hip_ext.h>

#include "common.cuh"

namespace mui {

constexpr int kChainThreads = 256;
constexpr int kChainR = 4;
constexpr int kChainCH = 2;
constexpr int kChainCounters = 8;
constexpr int kChainCounterStride = 64;  // in uint32: 256 bytes apart

__device__ __forceinline__ float chain_dot2(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}

// COH: x is read with agent-scope loads (never from a stale line of this XCD's L2)
template <bool HANDOFF, bool COH>
__global__ void __launch_bounds__(kChainThreads) chain_gemv_kernel(
    const uint16_t* w, const uint16_t* x, uint16_t* y, int n, int k, const uint32_t* flag_in,
    uint32_t expected, uint32_t* flag_out, uint32_t* err, int spin_limit) {
  __shared__ float red[2][kChainThreads / kWave][kChainR];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int kc = k >> 3;
  const int n_groups = n / kChainR;
  int coff[kChainCH];
  bool cvalid[kChainCH];
#pragma unroll
  for (int j = 0; j < kChainCH; ++j) {
    const int c = t + kChainThreads * j;
    cvalid[j] = c < kc;
    coff[j] = cvalid[j] ? (c << 3) : 0;
  }
  u32x4 wr[kChainR][kChainCH];
  auto issue = [&](int rg) {
#pragma unroll
    for (int r = 0; r < kChainR; ++r) {
      const uint16_t* rp = w + (long)(rg * kChainR + r) * k;
#pragma unroll
      for (int j = 0; j < kChainCH; ++j) wr[r][j] = ld16_stream(rp + coff[j]);
    }
  };
  int rg = blockIdx.x;
  issue(rg);  // independent of x: in flight while the predecessor drains

  if constexpr (HANDOFF) {
    if (flag_in != nullptr) {
      if (t < kChainCounters) {
        int spins = 0;
        while ((int)(__hip_atomic_load(flag_in + t * kChainCounterStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) -
                     expected) < 0) {
          __builtin_amdgcn_s_sleep(2);
          if (++spins > spin_limit) {
            __hip_atomic_fetch_or(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
        }
      }
      __syncthreads();
    }
  }

  u32x4 xq[kChainCH];
#pragma unroll
  for (int j = 0; j < kChainCH; ++j) {
    if constexpr (HANDOFF && COH) {
      const uint64_t* xp = (const uint64_t*)(x + coff[j]);
      const uint64_t lo = __hip_atomic_load(xp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint64_t hi = __hip_atomic_load(xp + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      xq[j].x = (uint32_t)lo; xq[j].y = (uint32_t)(lo >> 32); xq[j].z = (uint32_t)hi; xq[j].w = (uint32_t)(hi >> 32);
    } else {
      xq[j] = ld16(x + coff[j]);
    }
    const u32x4 zero = {0u, 0u, 0u, 0u};
    xq[j] = cvalid[j] ? xq[j] : zero;
  }

  int buf = 0;
  for (; rg < n_groups; rg += gridDim.x) {
    float acc[kChainR];
#pragma unroll
    for (int r = 0; r < kChainR; ++r) {
      float a = 0.f;
#pragma unroll
      for (int j = 0; j < kChainCH; ++j) {
        a = chain_dot2(wr[r][j].x, xq[j].x, a);
        a = chain_dot2(wr[r][j].y, xq[j].y, a);
        a = chain_dot2(wr[r][j].z, xq[j].z, a);
        a = chain_dot2(wr[r][j].w, xq[j].w, a);
      }
      acc[r] = a;
    }
    const int nxt = rg + gridDim.x;
    if (nxt < n_groups) issue(nxt);
#pragma unroll
    for (int r = 0; r < kChainR; ++r) acc[r] = wave_sum(acc[r]);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < kChainR; ++r) red[buf][wave][r] = acc[r];
    }
    __syncthreads();
    if (t < kChainR) {
      const float v = (red[buf][0][t] + red[buf][1][t]) + (red[buf][2][t] + red[buf][3][t]);
      const uint16_t bits = F16::pack(v);
      if constexpr (HANDOFF)
        __hip_atomic_store(y + rg * kChainR + t, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else
        y[rg * kChainR + t] = bits;
    }
    buf ^= 1;
  }
  if constexpr (HANDOFF) {
    // the storing threads wait until their stores have been acknowledged, then one thread reports
    if (t < kChainR) __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (t == 0)
      __hip_atomic_fetch_add(flag_out + (blockIdx.x % kChainCounters) * kChainCounterStride, 1u, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Second form of the hand-off: a fifth wave does nothing but poll the counters and then fetch x into
// LDS (its loads do not queue behind weight loads: loads return in order within a wave), and the four
// weight waves request PF row groups -- for a 4096 x 4096 matrix on 512 workgroups: everything they
// will ever read -- before they wait for it. n_groups must be a multiple of gridDim.x * PF... not
// required: row groups past the end are clamped and dropped.
template <int PF>
__global__ void __launch_bounds__(kChainThreads + kWave) chain_gemv_pollwave_kernel(
    const uint16_t* w, const uint16_t* x, uint16_t* y, int n, int k, const uint32_t* flag_in,
    uint32_t expected, uint32_t* flag_out, uint32_t* err, int spin_limit) {
  __shared__ float red[2][kChainThreads / kWave][kChainR];
  __shared__ __attribute__((aligned(16))) uint16_t xs[kChainCH * kChainThreads * 8];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int kc = k >> 3;
  const int n_groups = n / kChainR;
  const bool poller = wave == kChainThreads / kWave;
  int coff[kChainCH];
#pragma unroll
  for (int j = 0; j < kChainCH; ++j) {
    const int c = (t & (kChainThreads - 1)) + kChainThreads * j;
    coff[j] = c < kc ? (c << 3) : 0;
  }
  u32x4 wr[PF][kChainR][kChainCH];
  auto issue = [&](int slot, int rg) {
    const int g = rg < n_groups ? rg : n_groups - 1;
#pragma unroll
    for (int r = 0; r < kChainR; ++r) {
      const uint16_t* rp = w + (long)(g * kChainR + r) * k;
#pragma unroll
      for (int j = 0; j < kChainCH; ++j) wr[slot][r][j] = ld16_stream(rp + coff[j]);
    }
  };
  if (!poller) {
#pragma unroll
    for (int f = 0; f < PF; ++f) issue(f, blockIdx.x + f * gridDim.x);
  } else {
    if (flag_in != nullptr && lane < kChainCounters) {
      int spins = 0;
      while ((int)(__hip_atomic_load(flag_in + lane * kChainCounterStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) -
                   expected) < 0) {
        __builtin_amdgcn_s_sleep(1);
        if (++spins > spin_limit) {
          __hip_atomic_fetch_or(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
      }
    }
    // (the wave reconverges here: the loads below follow every lane's last poll)
    // all of x requested before the first value is used: one round trip, not one per chunk
    constexpr int kIter = kChainCH * kChainThreads / kWave;
    uint64_t lo[kIter], hi[kIter];
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      const int c = lane + i * kWave;
      const uint64_t* xp = (const uint64_t*)(x + ((c < kc ? c : 0) << 3));
      lo[i] = __hip_atomic_load(xp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      hi[i] = __hip_atomic_load(xp + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      const int c = lane + i * kWave;
      *(uint64_t*)&xs[(c << 3)] = lo[i];
      *(uint64_t*)&xs[(c << 3) + 4] = hi[i];
    }
  }
  __syncthreads();
  u32x4 xq[kChainCH];
#pragma unroll
  for (int j = 0; j < kChainCH; ++j) {
    const int c = (t & (kChainThreads - 1)) + kChainThreads * j;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    xq[j] = c < kc ? *(const u32x4*)&xs[c << 3] : zero;
  }

  int buf = 0;
  int rg = blockIdx.x;
  for (int it = 0; rg < n_groups; rg += gridDim.x, ++it) {
    float acc[kChainR];
    if (!poller) {
      const int slot = it % PF;
#pragma unroll
      for (int r = 0; r < kChainR; ++r) {
        float a = 0.f;
#pragma unroll
        for (int f = 0; f < PF; ++f) {
          if (f == slot) {
#pragma unroll
            for (int j = 0; j < kChainCH; ++j) {
              a = chain_dot2(wr[f][r][j].x, xq[j].x, a);
              a = chain_dot2(wr[f][r][j].y, xq[j].y, a);
              a = chain_dot2(wr[f][r][j].z, xq[j].z, a);
              a = chain_dot2(wr[f][r][j].w, xq[j].w, a);
            }
          }
        }
        acc[r] = a;
      }
      const int nxt = rg + PF * gridDim.x;
      if (nxt < n_groups) {
#pragma unroll
        for (int f = 0; f < PF; ++f)
          if (f == slot) issue(f, nxt);
      }
#pragma unroll
      for (int r = 0; r < kChainR; ++r) acc[r] = wave_sum(acc[r]);
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < kChainR; ++r) red[buf][wave][r] = acc[r];
      }
    }
    __syncthreads();
    if (t < kChainR) {
      const float v = (red[buf][0][t] + red[buf][1][t]) + (red[buf][2][t] + red[buf][3][t]);
      __hip_atomic_store(y + rg * kChainR + t, F16::pack(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    buf ^= 1;
  }
  if (t < kChainR) __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (t == 0)
    __hip_atomic_fetch_add(flag_out + (blockIdx.x % kChainCounters) * kChainCounterStride, 1u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace mui

using namespace mui;

extern "C" size_t mui_probe_chain_flag_bytes(int n_launches) {
  return n_launches > 0 ? (size_t)n_launches * kChainCounters * kChainCounterStride * sizeof(uint32_t) : 0;
}

// weights: n_mats device pointers (host array) used round-robin; xa / xb: two k-element fp16 buffers
// (launch i reads one and writes the other; n == k); flags: mui_probe_chain_flag_bytes(n_launches)
// bytes of device memory that the CALLER has zeroed; err: one zeroed device uint32.
extern "C" int mui_probe_gemv_chain(mui_stream_t stream, int mode, const void* const* weights, int n_mats,
                                    int n_launches, int n, int k, void* xa, void* xb, void* flags, void* err,
                                    int workgroups, int spin_limit) {
  MUI_CHECK_ARG(weights && n_mats > 0 && n_launches > 0 && xa && xb && err);
  MUI_CHECK_ARG(n == k && k > 0 && k <= kChainCH * kChainThreads * 8 && (k & 7) == 0 && (n % kChainR) == 0);
  MUI_CHECK_ARG(mode == 0 || mode == 5 || mode == 6 || ((mode >= 1 && mode <= 4) && flags));
  MUI_CHECK_ARG(spin_limit > 0 && spin_limit <= (1 << 22));
  const int n_groups = n / kChainR;
  int grid = workgroups > 0 ? workgroups : balanced_grid(n_groups, 3);
  if (grid > n_groups) grid = n_groups;
  // the counters are dealt by workgroup id mod 8: every counter must see the same number of arrivals
  if (mode != 0 && grid % kChainCounters != 0) return MUI_ERR_INVALID_ARG;
  hipStream_t s = (hipStream_t)stream;
  uint32_t* fl = (uint32_t*)flags;
  for (int i = 0; i < n_launches; ++i) {
    const uint16_t* w = (const uint16_t*)weights[i % n_mats];
    const uint16_t* x = (const uint16_t*)((i & 1) ? xb : xa);
    uint16_t* y = (uint16_t*)((i & 1) ? xa : xb);
    if (mode == 5 || mode == 6) {
      // independent GEMVs (every launch reads xa and writes its own half of xb's ... the same y: the
      // results are not used), ordinary (6) or free to overlap (5): what overlap alone is worth
      if (mode == 6)
        hipLaunchKernelGGL((chain_gemv_kernel<false, false>), dim3(grid), dim3(kChainThreads), 0, s, w,
                           (const uint16_t*)xa, (uint16_t*)xb, n, k, (const uint32_t*)nullptr, 0u, (uint32_t*)nullptr,
                           (uint32_t*)err, spin_limit);
      else
        hipExtLaunchKernelGGL((chain_gemv_kernel<false, false>), dim3(grid), dim3(kChainThreads), 0, s, nullptr, nullptr,
                              hipExtAnyOrderLaunch, w, (const uint16_t*)xa, (uint16_t*)xb, n, k, (const uint32_t*)nullptr,
                              0u, (uint32_t*)nullptr, (uint32_t*)err, spin_limit);
    } else if (mode == 0) {
      hipLaunchKernelGGL((chain_gemv_kernel<false, false>), dim3(grid), dim3(kChainThreads), 0, s, w, x, y, n, k,
                         (const uint32_t*)nullptr, 0u, (uint32_t*)nullptr, (uint32_t*)err, spin_limit);
    } else {
      const uint32_t* fin = i == 0 ? nullptr : fl + (size_t)(i - 1) * kChainCounters * kChainCounterStride;
      uint32_t* fout = fl + (size_t)i * kChainCounters * kChainCounterStride;
      const uint32_t expected = (uint32_t)(grid / kChainCounters);
      if (mode == 3)
        hipExtLaunchKernelGGL((chain_gemv_pollwave_kernel<1>), dim3(grid), dim3(kChainThreads + kWave), 0, s, nullptr,
                              nullptr, hipExtAnyOrderLaunch, w, x, y, n, k, fin, expected, fout, (uint32_t*)err,
                              spin_limit);
      else if (mode == 4)
        hipExtLaunchKernelGGL((chain_gemv_pollwave_kernel<2>), dim3(grid), dim3(kChainThreads + kWave), 0, s, nullptr,
                              nullptr, hipExtAnyOrderLaunch, w, x, y, n, k, fin, expected, fout, (uint32_t*)err,
                              spin_limit);
      else if (mode == 1)
        hipExtLaunchKernelGGL((chain_gemv_kernel<true, true>), dim3(grid), dim3(kChainThreads), 0, s, nullptr, nullptr,
                              hipExtAnyOrderLaunch, w, x, y, n, k, fin, expected, fout, (uint32_t*)err, spin_limit);
      else
        hipExtLaunchKernelGGL((chain_gemv_kernel<true, false>), dim3(grid), dim3(kChainThreads), 0, s, nullptr, nullptr,
                              hipExtAnyOrderLaunch, w, x, y, n, k, fin, expected, fout, (uint32_t*)err, spin_limit);
    }
    if (hipGetLastError() != hipSuccess) return MUI_ERR_LAUNCH;
  }
  return MUI_OK;
}

// The same chain dealt alternately to TWO streams (launch i goes to stream i % 2; ordinary launches,
// so a kernel waits for the launch two before it through its own queue and for its predecessor, on
// the other queue, through the arrival counters): two kernels can then be resident at a time -- the
// one that computes and its successor, whose weights are already on their way. mode 0: independent
// GEMVs (no hand-off, results unused: what two queues overlap at best); 1: hand-off as in
// mui_probe_gemv_chain mode 1; 2 / 3: the poll-wave kernel with one / two row groups requested first.
extern "C" int mui_probe_gemv_chain2(mui_stream_t stream_a, mui_stream_t stream_b, int mode,
                                     const void* const* weights, int n_mats, int n_launches, int n, int k, void* xa,
                                     void* xb, void* flags, void* err, int workgroups, int spin_limit) {
  MUI_CHECK_ARG(weights && n_mats > 0 && n_launches > 0 && xa && xb && err && flags);
  MUI_CHECK_ARG(n == k && k > 0 && k <= kChainCH * kChainThreads * 8 && (k & 7) == 0 && (n % kChainR) == 0);
  MUI_CHECK_ARG(mode >= 0 && mode <= 3 && spin_limit > 0 && spin_limit <= (1 << 22));
  const int n_groups = n / kChainR;
  int grid = workgroups > 0 ? workgroups : balanced_grid(n_groups, 3);
  if (grid > n_groups) grid = n_groups;
  if (grid % kChainCounters != 0) return MUI_ERR_INVALID_ARG;
  uint32_t* fl = (uint32_t*)flags;
  for (int i = 0; i < n_launches; ++i) {
    hipStream_t s = (hipStream_t)((i & 1) ? stream_b : stream_a);
    const uint16_t* w = (const uint16_t*)weights[i % n_mats];
    const uint16_t* x = (const uint16_t*)((i & 1) ? xb : xa);
    uint16_t* y = (uint16_t*)((i & 1) ? xa : xb);
    const uint32_t* fin = i == 0 ? nullptr : fl + (size_t)(i - 1) * kChainCounters * kChainCounterStride;
    uint32_t* fout = fl + (size_t)i * kChainCounters * kChainCounterStride;
    const uint32_t expected = (uint32_t)(grid / kChainCounters);
    if (mode == 0)
      hipLaunchKernelGGL((chain_gemv_kernel<false, false>), dim3(grid), dim3(kChainThreads), 0, s, w, (const uint16_t*)xa,
                         (uint16_t*)xb, n, k, (const uint32_t*)nullptr, 0u, (uint32_t*)nullptr, (uint32_t*)err, spin_limit);
    else if (mode == 1)
      hipLaunchKernelGGL((chain_gemv_kernel<true, true>), dim3(grid), dim3(kChainThreads), 0, s, w, x, y, n, k, fin,
                         expected, fout, (uint32_t*)err, spin_limit);
    else if (mode == 2)
      hipLaunchKernelGGL((chain_gemv_pollwave_kernel<1>), dim3(grid), dim3(kChainThreads + kWave), 0, s, w, x, y, n, k,
                         fin, expected, fout, (uint32_t*)err, spin_limit);
    else
      hipLaunchKernelGGL((chain_gemv_pollwave_kernel<2>), dim3(grid), dim3(kChainThreads + kWave), 0, s, w, x, y, n, k,
                         fin, expected, fout, (uint32_t*)err, spin_limit);
    if (hipGetLastError() != hipSuccess) return MUI_ERR_LAUNCH;
  }
  return MUI_OK;
}
