// Measurement aid: a plain streaming read, the rate every HBM-bound kernel here is held against
// besides the published peak.
#include "common.h"

// Visible outside this file on purpose: a store to a file-local variable that nothing reads
// would be removed, and the loads with it.
__device__ float msa_probe_sink;

namespace {

__global__ __launch_bounds__(256) void stream_read_kernel(const float4_t* __restrict__ p,
                                                          int64_t n16) {
  constexpr int U = 8;  // 16-byte loads in flight per thread
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (; i + (U - 1) * stride < n16; i += U * stride) {
    float4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) acc += v[u];
  }
  for (; i < n16; i += stride) acc += __builtin_nontemporal_load(p + i);
  // keeps the loads alive; the comparison is (practically) never true
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) msa_probe_sink = 1.f;
}

}  // namespace

extern "C" int msa_probe_stream_read(const void* p, int64_t bytes, void* stream) {
  MSA_REQUIRE(p != nullptr, MSA_ERR_INVALID_ARG, "msa_probe_stream_read: null pointer");
  MSA_REQUIRE(bytes > 0 && bytes % 16 == 0 && ((uintptr_t)p & 15) == 0, MSA_ERR_INVALID_ARG,
              "msa_probe_stream_read: address and size must be multiples of 16 bytes");
  hipLaunchKernelGGL(stream_read_kernel, dim3(8192), dim3(256), 0, (hipStream_t)stream,
                     (const float4_t*)p, bytes / 16);
  MSA_CHECK_LAUNCH("msa_probe_stream_read");
  return MSA_OK;
}
