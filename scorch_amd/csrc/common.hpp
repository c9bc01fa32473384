// Shared host/device helpers of libscorch_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <type_traits>

#include "../../include/scorch_hip_unstable.h"  // and, through it, scorch_hip.h

namespace scorch {

constexpr int kWaveSize = 64;       // CDNA wavefront
constexpr int kBlockThreads = 256;  // 4 wavefronts per workgroup
constexpr int kWavesPerBlock = kBlockThreads / kWaveSize;

// ---- error reporting --------------------------------------------------------
// One message buffer per host thread; scorch_hip_last_error() returns it.
char *error_buffer();
constexpr size_t kErrorBufferBytes = 512;

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), kErrorBufferBytes, fmt, ap);
  va_end(ap);
  return code;
}

#define SCORCH_REQUIRE(cond, ...)                                   \
  do {                                                              \
    if (!(cond)) return ::scorch::fail(SCORCH_HIP_EINVAL, __VA_ARGS__); \
  } while (0)

#define SCORCH_HIP_CHECK(expr)                                                       \
  do {                                                                               \
    hipError_t err__ = (expr);                                                       \
    if (err__ != hipSuccess)                                                         \
      return ::scorch::fail(SCORCH_HIP_ERUNTIME, "%s failed: %s", #expr,             \
                            hipGetErrorString(err__));                               \
  } while (0)

inline bool aligned_to(const void *p, size_t bytes) {
  return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// Validation shared by every entry point that takes a CSR operand.
inline int check_csr_args(const char *fn, int64_t M, int64_t K, int64_t nnz, const void *row_ptr,
                          const void *col_idx, const void *vals) {
  if (M < 0 || K < 0 || nnz < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld K=%lld nnz=%lld)", fn,
                (long long)M, (long long)K, (long long)nnz);
  if (M >= INT32_MAX || K > INT32_MAX || nnz > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED,
                "%s: M, K and nnz must fit the int32 index arrays (M=%lld K=%lld nnz=%lld)", fn,
                (long long)M, (long long)K, (long long)nnz);
  if (!row_ptr) return fail(SCORCH_HIP_EINVAL, "%s: row_ptr is NULL", fn);
  if (nnz > 0 && (!col_idx || !vals))
    return fail(SCORCH_HIP_EINVAL, "%s: col_idx/vals is NULL with nnz=%lld", fn, (long long)nnz);
  if (nnz > 0 && (M == 0 || K == 0))
    return fail(SCORCH_HIP_EINVAL, "%s: nnz=%lld in an empty matrix", fn, (long long)nnz);
  if (!aligned_to(row_ptr, 4) || !aligned_to(col_idx, 4))
    return fail(SCORCH_HIP_EINVAL, "%s: index arrays must be 4-byte aligned", fn);
  return SCORCH_HIP_OK;
}

// ---- per-kernel timing for benchmarks ---------------------------------------
// Between scorch_hip_timing_begin() and scorch_hip_timing_end() on a host thread,
// every entry point records a HIP event on its stream before its first launch,
// between its launches and after its last (mark_launch); _end returns the
// intervals.  Outside such a bracket mark_launch is one thread-local test.
constexpr int kMaxLaunchMarks = 16;
struct LaunchMarks {
  hipEvent_t ev[kMaxLaunchMarks];
  int count = 0;
  bool created = false, active = false;
};
LaunchMarks *launch_marks();  // the calling thread's

inline void mark_launch(hipStream_t stream) {
  LaunchMarks *m = launch_marks();
  if (m->active && m->count < kMaxLaunchMarks) (void)hipEventRecord(m->ev[m->count++], stream);
}

// ---- arithmetic traits --------------------------------------------------------
// Integer kernels accumulate in the unsigned type of the same width so that
// overflow wraps (the reference's signed overflow wraps in practice).
template <typename T> struct Acc { using type = T; };
template <> struct Acc<int32_t> { using type = uint32_t; };
template <> struct Acc<int64_t> { using type = uint64_t; };

// ---- device helpers ---------------------------------------------------------
template <typename T, int V> struct alignas(sizeof(T) * V) Vec { T v[V]; };

// Sum over the GS lanes of a group (GS a power of two, groups aligned), every lane receiving the
// total, with the pairing x(i) + x(i ^ off) for off = GS / 2 down to 1.  Within a row of 16 lanes
// the exchanges are row rotations carried by the add itself (DPP): once the steps above have made
// the values periodic with period 2 off, lane (i + off) mod 16 holds what lane i ^ off holds.  A
// shuffle instead goes through the LDS pipe and has to be waited for.  Groups below 16 lanes share
// a row with other groups and keep the shuffles.
template <int N>
__device__ __forceinline__ float row_rotated(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + N, 0xf, 0xf, false));
}
template <int GS>
__device__ __forceinline__ float group_sum(float x) {
  if constexpr (GS >= 16) {
#pragma unroll
    for (int off = GS / 2; off >= 16; off >>= 1) x += __shfl_xor(x, off);
    x += row_rotated<8>(x);
    x += row_rotated<4>(x);
    x += row_rotated<2>(x);
    x += row_rotated<1>(x);
  } else {
#pragma unroll
    for (int off = GS / 2; off > 0; off >>= 1) x += __shfl_xor(x, off);
  }
  return x;
}

// A store marked as streaming: data that nothing reads again, which should not push out of the
// L2 what other accesses of the same kernel come back to.
template <typename T>
__device__ __forceinline__ void store_streaming(T *p, T x) {
  __builtin_nontemporal_store(x, p);
}
template <typename T, int V>
__device__ __forceinline__ void store_streaming(T *p, const Vec<T, V> &x) {
  typedef T Native __attribute__((ext_vector_type(V)));
  __builtin_nontemporal_store(__builtin_bit_cast(Native, x), reinterpret_cast<Native *>(p));
}

__device__ __forceinline__ int wave_lane() { return threadIdx.x & (kWaveSize - 1); }

// Value of lane 0's copy in a scalar register: tells the compiler a value is
// wave-uniform so that addresses built from it use scalar arithmetic.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Workgroups are dealt to the 8 XCDs round robin by their linear id, and every
// XCD has its own L2.  xcd_contiguous renumbers the n workgroups of a launch (n a
// multiple of 8, see round_up_8; a kernel lets the surplus ones find nothing to
// do) so that XCD x works through the contiguous range [x n/8, (x + 1) n/8) in
// order: the wavefronts resident on one XCD then work on neighbouring pieces of
// the input, and rows of the gathered operand that neighbouring pieces share
// are found in that XCD's L2 instead of being fetched into all eight.
__device__ __forceinline__ int64_t xcd_contiguous(int64_t id, int64_t n) {
  return (id & 7) * (n >> 3) + (id >> 3);
}
inline int64_t round_up_8(int64_t n) { return (n + 7) / 8 * 8; }

// Orders LDS traffic inside one wavefront: writes by any lane before this point
// are seen by reads of any lane after it.  Enough when the LDS region is
// private to the wavefront (the hardware runs one wavefront's LDS instructions
// in order; this keeps the compiler from moving them), and it does not couple
// the wavefronts of a workgroup the way __syncthreads() does.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Wave-cooperative search: number of i in [0, n) with key(i) < bound, for a
// strictly increasing key.  Each step probes 64 evenly spaced positions, so a
// million-entry array takes four dependent loads instead of twenty.
template <typename KeyFn>
__device__ __forceinline__ int wave_count_below(int n, int64_t bound, KeyFn key) {
  const int lane = wave_lane();
  int lo = 0, hi = n;
  while (lo < hi) {
    const int span = hi - lo;
    const int step = (span + kWaveSize - 1) / kWaveSize;
    const int64_t idx = (int64_t)lo + (int64_t)(lane + 1) * step - 1;
    bool below = false;
    if (idx < hi) below = key((int)idx) < bound;
    const int cnt = __popcll(__ballot(below));
    const int64_t nhi = (int64_t)lo + (int64_t)(cnt + 1) * step - 1;
    lo = lo + cnt * step;
    hi = nhi < hi ? (int)nhi : hi;
  }
  return uniform(lo);
}

}  // namespace scorch

// ---- loading the device code ahead of the first launch ------------------------------------------
// HIP loads a source file's device code when the first kernel of that file is launched on a
// device, which takes about a millisecond: a product whose kernels live in a file that has not
// been used yet pays it.  Every source file defines an empty kernel through this macro;
// scorch_hip_init() asks the runtime for each one's attributes, which loads the file's code for
// the current device without launching anything.
#define SCORCH_DEFINE_PRELOAD(name)                                                                   \
  namespace scorch {                                                                                  \
  __global__ void preload_anchor_##name() {}                                                          \
  hipError_t preload_##name() {                                                                       \
    hipFuncAttributes attributes;                                                                     \
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void *>(&preload_anchor_##name)); \
  }                                                                                                   \
  }
