// Pre-LN LayerNorm forward, fp16 in / fp16 out, fp32 statistics.
// One workgroup per row; the row lives in registers between the two reduction passes, so
// HBM traffic is exactly one read and one write of the row plus gamma/beta.
#include "common.h"

namespace {

constexpr int LN_THREADS = 256;
constexpr int LN_MAX_CHUNKS = 8;  // 8 halves per chunk per thread -> D <= 256*8*8 = 16384

__global__ __launch_bounds__(LN_THREADS) void layernorm_f16_kernel(
    const half_t* __restrict__ x, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, half_t* __restrict__ y, int D, float eps) {
  __shared__ float red[16];
  const int64_t row = blockIdx.x;
  const half_t* xr = x + row * D;
  half_t* yr = y + row * D;
  const int nchunk = D >> 3;  // 16-byte chunks in the row

  half8_t v[LN_MAX_CHUNKS];
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * LN_THREADS;
    if (idx < nchunk) {
      v[c] = *reinterpret_cast<const half8_t*>(xr + (idx << 3));
#pragma unroll
      for (int i = 0; i < 8; ++i) s += (float)v[c][i];
    }
  }
  const float mean = block_sum(s, red) / (float)D;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * LN_THREADS;
    if (idx < nchunk) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float d = (float)v[c][i] - mean;
        q += d * d;
      }
    }
  }
  const float var = block_sum(q, red) / (float)D;
  const float rstd = rsqrtf(var + eps);
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * LN_THREADS;
    if (idx < nchunk) {
      const half8_t g = *reinterpret_cast<const half8_t*>(gamma + (idx << 3));
      const half8_t b = *reinterpret_cast<const half8_t*>(beta + (idx << 3));
      half8_t o;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        o[i] = (half_t)(((float)v[c][i] - mean) * rstd * (float)g[i] + (float)b[i]);
      *reinterpret_cast<half8_t*>(yr + (idx << 3)) = o;
    }
  }
}

}  // namespace

extern "C" int msa_layernorm_f16(const void* x, const void* gamma, const void* beta, void* y,
                                 int64_t rows, int D, float eps, void* stream) {
  MSA_REQUIRE(x && gamma && beta && y, MSA_ERR_INVALID_ARG, "msa_layernorm_f16: null pointer");
  MSA_REQUIRE(rows >= 0 && rows <= 0x7fffffff, MSA_ERR_INVALID_ARG,
              "msa_layernorm_f16: rows=%lld out of range", (long long)rows);
  MSA_REQUIRE(D > 0 && D % 8 == 0 && D <= LN_THREADS * 8 * LN_MAX_CHUNKS, MSA_ERR_INVALID_ARG,
              "msa_layernorm_f16: D=%d must be a multiple of 8 and <= %d", D,
              LN_THREADS * 8 * LN_MAX_CHUNKS);
  if (rows == 0) return MSA_OK;
  hipLaunchKernelGGL(layernorm_f16_kernel, dim3((unsigned)rows), dim3(LN_THREADS), 0,
                     (hipStream_t)stream, (const half_t*)x, (const half_t*)gamma,
                     (const half_t*)beta, (half_t*)y, D, eps);
  MSA_CHECK_LAUNCH("msa_layernorm_f16");
  return MSA_OK;
}
