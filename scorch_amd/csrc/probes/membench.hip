// Memory-system probes used by bench.py --probe: what this GPU sustains for a
// streaming read and for random row gathers, measured with kernels that do
// nothing else.  They give the ceilings the SpMM/SDDMM kernels are priced
// against.  Built into libscorch_probes.so, separate from the product library.
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

}  // namespace

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
