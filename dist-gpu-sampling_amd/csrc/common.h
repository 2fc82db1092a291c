// Shared host/device helpers of libdgs_hip.so (gfx950 only).
#ifndef DGS_CSRC_COMMON_H_
#define DGS_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "dgs_hip.h"

#define DGS_API extern "C" __attribute__((visibility("default")))

namespace dgs {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- host-side error plumbing -------------------------------------------------
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define DGS_REQUIRE(cond, status, ...)  \
  do {                                  \
    if (!(cond)) {                      \
      ::dgs::set_error(__VA_ARGS__);    \
      return (status);                  \
    }                                   \
  } while (0)

#define DGS_HIP_TRY(call)                                                          \
  do {                                                                             \
    hipError_t e_ = (call);                                                        \
    if (e_ != hipSuccess) {                                                        \
      ::dgs::set_error("%s:%d %s failed: %s", __FILE__, __LINE__, #call,           \
                       hipGetErrorString(e_));                                     \
      return DGS_ERR_HIP;                                                          \
    }                                                                              \
  } while (0)

// Checks the launch of the kernel just enqueued.
#define DGS_LAUNCH_CHECK() DGS_HIP_TRY(hipGetLastError())

inline bool width_ok(int32_t b) { return b == 4 || b == 8; }

// Value of a dgs_debug_set option (0 unless a test set it).
int64_t debug_option(int32_t option);

// Carves aligned pieces out of a caller-provided workspace.
struct Carver {
  char* base;
  size_t used;
  explicit Carver(void* p) : base(static_cast<char*>(p)), used(0) {}
  template <typename T>
  T* take(size_t count) {
    used = (used + 255) & ~size_t(255);
    T* r = reinterpret_cast<T*>(base + used);
    used += count * sizeof(T);
    return r;
  }
};
inline size_t carve_size(size_t used, size_t bytes) {
  return ((used + 255) & ~size_t(255)) + bytes;
}

// ---- device-side helpers ------------------------------------------------------

// Typed element of a two-tier view: dev[i] below the threshold, host[i-thr] above.
template <typename T>
struct TierView {
  const T* dev;
  const T* host;
  int64_t thr;
  int64_t n;  // elements in the whole store: what an index is checked against before it is used
  __host__ explicit TierView(const dgs_view& v)
      : dev(static_cast<const T*>(v.dev)), host(static_cast<const T*>(v.host)), thr(v.threshold), n(v.total) {}
  __device__ __forceinline__ T at(int64_t i) const { return i < thr ? dev[i] : host[i - thr]; }
};

// Whether `row` names a row of the CSC offsets array `indptr` (entries row and row + 1 exist).
template <typename T>
__device__ __forceinline__ bool row_in_range(const TierView<T>& indptr, int64_t row) {
  return row >= 0 && row < indptr.n - 1;
}

// Exclusive scan of one value per thread over a block of NT threads (NT multiple of 64).
// Returns the exclusive prefix; *total receives the block sum (same value in all threads).
// `lds` holds NT/64 values of T.
template <int NT, typename T>
__device__ __forceinline__ T block_exclusive_scan(T v, T* total, T* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  T incl = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    T t = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += t;
  }
  if (lane == kWave - 1) lds[wave] = incl;
  __syncthreads();
  T wave_off = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < NT / kWave; ++w) {
    T s = lds[w];
    if (w < wave) wave_off += s;
    sum += s;
  }
  __syncthreads();  // lds may be reused by the caller right after
  *total = sum;
  return wave_off + incl - v;
}

// One block of NT threads: out[t] = exclusive prefix of in[0..t) for t < count, *sum = total
// (valid in thread 0).  Used for the per-tile totals of the multi-block scans (count is small).
template <int NT, typename TIn, typename TOut>
__device__ __forceinline__ void single_block_scan(const TIn* __restrict__ in, TOut* __restrict__ out,
                                                  int64_t count, TOut* sum) {
  __shared__ TOut lds[NT / kWave];
  __shared__ TOut carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int64_t t0 = 0; t0 < count; t0 += NT) {
    const int64_t t = t0 + threadIdx.x;
    const TOut v = t < count ? TOut(in[t]) : TOut(0);
    TOut total;
    const TOut ex = block_exclusive_scan<NT, TOut>(v, &total, lds);
    if (t < count) out[t] = carry + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) *sum = carry;
}

// A length word mirrored into pinned host memory: stored at system scope, so that it leaves the
// GPU's caches at once and a host thread that polls the word (dgs_ticket_wait_words) sees it
// while the kernel is still running.  Every word stands for itself: no order among them is
// promised, and a reader takes each one when it has turned non-negative.
__device__ __forceinline__ void mirror_to_host(int64_t* word, int64_t v) {
  __hip_atomic_store(word, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

template <typename T>
__device__ __forceinline__ void single_block_scan_1024(const T* __restrict__ in, T* __restrict__ out,
                                                       int64_t count, T* sum) {
  single_block_scan<1024, T, T>(in, out, count, sum);
}

// Philox4x32-10 block for the "dgs-philox-1" contract.
struct PhiloxWords { uint32_t w[4]; };
__device__ __forceinline__ PhiloxWords philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                     uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    // one 32x32->64 multiply each (v_mad_u64_u32) instead of separate high and low halves
    const uint64_t p0 = uint64_t(0xD2511F53u) * c0;
    const uint64_t p1 = uint64_t(0xCD9E8D57u) * c2;
    const uint32_t n0 = uint32_t(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = uint32_t(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = uint32_t(p1); c2 = n2; c3 = uint32_t(p0);
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return PhiloxWords{{c0, c1, c2, c3}};
}

// The Philox block of draw j of `row`: depends on nothing but the ids, so a kernel can compute it
// while the loads that tell the range of the draw are still in flight.
__device__ __forceinline__ PhiloxWords philox_draw_words(uint64_t seed, uint32_t stream, int64_t row, uint32_t j) {
  return philox4x32_10(j, stream, uint32_t(uint64_t(row)), uint32_t(uint64_t(row) >> 32), uint32_t(seed),
                       uint32_t(seed >> 32));
}

// A draw's block reduced to [0, n) (1 <= n < 2^32): multiply-shift with rejection over the
// block's four words, the last accepted unconditionally.
__device__ __forceinline__ uint32_t philox_reduce(const PhiloxWords& p, uint32_t n) {
  uint64_t m = uint64_t(p.w[0]) * n;
  if (uint32_t(m) < n) {  // rare: only now is the rejection threshold needed
    const uint32_t t = (0u - n) % n;
#pragma unroll
    for (int i = 1; i < 4; ++i) {
      if (uint32_t(m) >= t) break;
      m = uint64_t(p.w[i]) * n;
    }
  }
  return uint32_t(m >> 32);
}

// Draw j of `row`, reduced to [0, n).
__device__ __forceinline__ uint32_t philox_bounded(uint64_t seed, uint32_t stream, int64_t row,
                                                   uint32_t j, uint32_t n) {
  return philox_reduce(philox_draw_words(seed, stream, row, j), n);
}

}  // namespace dgs
#endif
