// Measurement aid: a plain streaming read, the rate every HBM-bound kernel here is held against
// besides the published peak.
#include "common.h"

// Visible outside this file on purpose: a store to a file-local variable that nothing reads
// would be removed, and the loads with it.
__device__ float msa_probe_sink;

namespace {

// Workgroup b reads the contiguous piece [b * chunk16, (b + 1) * chunk16) of the buffer, 16 loads of
// 16 bytes in flight per thread: the access pattern of the kernels it is compared with (each of
// their workgroups streams its own weight tiles or key / value rows).  A grid-stride sweep of the
// same bytes measured 10-15 % slower at 30-700 MB.
__global__ __launch_bounds__(256) void stream_read_kernel(const float4_t* __restrict__ p,
                                                          int64_t n16, int64_t chunk16) {
  constexpr int U = 16, T = 256;
  const int64_t lo = (int64_t)blockIdx.x * chunk16;
  const int64_t hi = lo + chunk16 < n16 ? lo + chunk16 : n16;
  int64_t i = lo + threadIdx.x;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  for (; i + (U - 1) * T < hi; i += U * T) {
    float4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + u * T);
#pragma unroll
    for (int u = 0; u < U; ++u) acc += v[u];
  }
  for (; i < hi; i += T) acc += __builtin_nontemporal_load(p + i);
  // keeps the loads alive; the comparison is (practically) never true
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) msa_probe_sink = 1.f;
}

}  // namespace

extern "C" int msa_probe_stream_read(const void* p, int64_t bytes, void* stream) {
  MSA_REQUIRE(p != nullptr, MSA_ERR_INVALID_ARG, "msa_probe_stream_read: null pointer");
  MSA_REQUIRE(bytes > 0 && bytes % 16 == 0 && ((uintptr_t)p & 15) == 0, MSA_ERR_INVALID_ARG,
              "msa_probe_stream_read: address and size must be multiples of 16 bytes");
  const int64_t n16 = bytes / 16;
  const int blocks = bytes < (64ll << 20) ? 512 : 2048;
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream,
                     (const float4_t*)p, n16, (n16 + blocks - 1) / blocks);
  MSA_CHECK_LAUNCH("msa_probe_stream_read");
  return MSA_OK;
}
