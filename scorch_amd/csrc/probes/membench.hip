// Probes used by bench.py --probe-memory / --probe-compute: what this GPU
// sustains for a streaming read, for random row gathers, and for matrix and
// vector instructions alone and side by side, measured with kernels that do
// nothing else.  They give the ceilings the kernels are priced against.  Built into libscorch_probes.so, separate from the product library.
#include <hip/hip_runtime.h>

#include <cstdint>

#define PROBE_API extern "C" __attribute__((visibility("default")))

namespace {

__global__ __launch_bounds__(256) void stream_read_kernel(const float4 *__restrict__ src, size_t n4,
                                                          float *sink) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  for (; i + 3 * stride < n4; i += 4 * stride) {
    const float4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc.x += a.x + b.x + c.x + d.x;
    acc.y += a.y + b.y + c.y + d.y;
    acc.z += a.z + b.z + c.z + d.z;
    acc.w += a.w + b.w + c.w + d.w;
  }
  for (; i < n4; i += stride) {
    const float4 a = src[i];
    acc.x += a.x; acc.y += a.y; acc.z += a.z; acc.w += a.w;
  }
  if (acc.x + acc.y + acc.z + acc.w == 12345.678f) sink[0] = acc.x;  // keeps the loads alive
}

// One wavefront gathers `per_wave` rows of 64 * VEC floats at the row numbers
// listed in idx, IN_FLIGHT loads at a time; lane l reads VEC floats at column l * VEC.
template <int VEC, int IN_FLIGHT>
__global__ __launch_bounds__(256) void gather_rows_kernel(const float *__restrict__ table,
                                                          const int *__restrict__ idx, int per_wave,
                                                          float *sink) {
  typedef float vecf __attribute__((ext_vector_type(VEC)));
  const int lane = threadIdx.x & 63;
  const size_t wave = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int *mine = idx + wave * per_wave;
  const int row_floats = 64 * VEC;
  float acc = 0.f;
  for (int k = 0; k < per_wave; k += IN_FLIGHT) {
    vecf b[IN_FLIGHT];
#pragma unroll
    for (int u = 0; u < IN_FLIGHT; ++u) {
      const int j = __builtin_amdgcn_readfirstlane(mine[k + u]);
      b[u] = *reinterpret_cast<const vecf *>(table + (size_t)j * row_floats + lane * VEC);
    }
#pragma unroll
    for (int u = 0; u < IN_FLIGHT; ++u)
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc += b[u][v];
  }
  if (acc == 12345.678f) sink[0] = acc;
}

template <int VEC, int IN_FLIGHT>
int launch_gather(const float *table, const int *idx, int64_t n_gathers, float *sink, hipStream_t s) {
  const int per_wave = 256;
  const int64_t waves = n_gathers / per_wave;
  if (waves % 4) return 1;
  gather_rows_kernel<VEC, IN_FLIGHT><<<dim3((unsigned)(waves / 4)), 256, 0, s>>>(table, idx, per_wave, sink);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}


// Matrix and vector throughput.  MODE 0: eight independent v_mfma_f32_16x16x32_bf16
// per iteration; MODE 1: 64 independent fp32 FMAs per lane and iteration; MODE 2:
// both in the same loop.  Whether mode 2 takes the longer of the two times or
// their sum says whether the matrix cores and the vector ALU of a SIMD run side
// by side.
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_floatx4 __attribute__((ext_vector_type(4)));

template <int MODE>
__global__ __launch_bounds__(256) void compute_kernel(float *sink, int iters) {
  probe_bf16x8 a, b;
  for (int j = 0; j < 8; ++j) {
    a[j] = (__bf16)(float)(threadIdx.x & 3);
    b[j] = (__bf16)1.0f;
  }
  probe_floatx4 acc[8];
  for (int i = 0; i < 8; ++i) acc[i] = probe_floatx4{0.f, 0.f, 0.f, 0.f};
  float x[16];
  for (int i = 0; i < 16; ++i) x[i] = 1.0f + 0.001f * (threadIdx.x + i);
  for (int it = 0; it < iters; ++it) {
    if (MODE != 1) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
    }
    if (MODE != 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = __builtin_fmaf(x[i], 1.0001f, 0.5f);
    }
  }
  float s = 0.f;
  for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  for (int i = 0; i < 16; ++i) s += x[i];
  if (s == 123.456f) sink[0] = s;  // keeps the work alive
}

}  // namespace

// mode 0 / 1 / 2 as above; `workgroups` of 256 threads, `iters` loop iterations.
// Per wavefront and iteration: 8 * 16384 matrix flops, 64 * 64 * 2 vector flops.
PROBE_API int scorch_probe_compute(int mode, int workgroups, int iters, void *sink, void *stream) {
  if (!sink || workgroups <= 0 || iters <= 0 || mode < 0 || mode > 2) return 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float *k = static_cast<float *>(sink);
  if (mode == 0) compute_kernel<0><<<dim3((unsigned)workgroups), 256, 0, s>>>(k, iters);
  else if (mode == 1) compute_kernel<1><<<dim3((unsigned)workgroups), 256, 0, s>>>(k, iters);
  else compute_kernel<2><<<dim3((unsigned)workgroups), 256, 0, s>>>(k, iters);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Reads `bytes` bytes (multiple of 16) once.  grid = number of 256-thread workgroups.
PROBE_API int scorch_probe_stream_read(const void *src, int64_t bytes, int grid, void *sink, void *stream) {
  if (!src || !sink || bytes <= 0 || bytes % 16 || grid <= 0) return 1;
  stream_read_kernel<<<dim3((unsigned)grid), 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const float4 *>(src), (size_t)bytes / 16, static_cast<float *>(sink));
  return hipGetLastError() == hipSuccess ? 0 : 2;
}

// Gathers n_gathers (multiple of 1024) rows of row_bytes in {256, 512, 1024} bytes;
// idx[n_gathers] holds row numbers inside the table; in_flight in {4, 8, 16}.
PROBE_API int scorch_probe_gather_rows(const void *table, const int32_t *idx, int64_t n_gathers,
                                       int row_bytes, int in_flight, void *sink, void *stream) {
  if (!table || !idx || !sink || n_gathers <= 0 || n_gathers % 1024) return 1;
  const float *t = static_cast<const float *>(table);
  float *k = static_cast<float *>(sink);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define CASE(RB, VEC, INF) if (row_bytes == RB && in_flight == INF) return launch_gather<VEC, INF>(t, idx, n_gathers, k, s)
  CASE(256, 1, 4); CASE(256, 1, 8); CASE(256, 1, 16);
  CASE(512, 2, 4); CASE(512, 2, 8); CASE(512, 2, 16);
  CASE(1024, 4, 4); CASE(1024, 4, 8); CASE(1024, 4, 16);
#undef CASE
  return 1;
}
