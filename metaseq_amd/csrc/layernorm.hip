// Pre-LN LayerNorm forward, fp16 in / fp16 out, fp32 statistics, optionally fused with the
// tail of the preceding split-K linear layer (sum of fp32 partials, bias add, residual add),
// and optionally writing the packed activation layout the decode GEMMs read.
// One workgroup per row; the row lives in registers between the reduction passes, so HBM
// traffic is one read and one write of the row plus gamma/beta.
#include "common.h"

namespace {

constexpr int LN_THREADS = 512;
constexpr int LN_MAX_CHUNKS = 4;  // 8 halves per chunk per thread -> D <= 512*8*4 = 16384

// ST > 0: the number of split-K slices is the compile-time constant ST, so that all slice loads
// of a chunk are issued back to back (a run-time trip count makes them one round trip each);
// ST == 0: any S.
// THREADS: workgroup size; a row of D elements needs D / 8 <= THREADS * LN_MAX_CHUNKS.  Decode
// (a few rows) uses wide workgroups to shorten the dependent chain, prefill (thousands of
// rows) narrow ones so that several rows share a compute unit.
template <int ST, int THREADS = LN_THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_f16_kernel(
    const half_t* x, const float* __restrict__ part, int S,
    const half_t* __restrict__ bias, half_t* x_out, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, half_t* __restrict__ y, int M, int D, float eps, int out_mb) {
  __shared__ float red[16];
  const int row = blockIdx.x;
  const int nchunk = D >> 3;  // 16-byte chunks in the row

  half8_t v[LN_MAX_CHUNKS], gv[LN_MAX_CHUNKS], bv[LN_MAX_CHUNKS];
  float s = 0.f;
  // gamma / beta are requested first so that their latency hides behind the reductions
  if (gamma) {
#pragma unroll
    for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
      const int idx = threadIdx.x + c * THREADS;
      if (idx < nchunk) {
        gv[c] = *reinterpret_cast<const half8_t*>(gamma + (idx << 3));
        bv[c] = *reinterpret_cast<const half8_t*>(beta + (idx << 3));
      }
    }
  }
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * THREADS;
    if (idx < nchunk) {
      if (part) {
        // x_out = round(round(round(sum_s part) + bias) + x): the fp16 rounding points of
        // "linear, + bias, + residual" in the reference layer; slices are summed in order
        const float* p = part + (int64_t)row * D + (idx << 3);
        const int64_t slice = (int64_t)M * D;
        const half8_t b = *reinterpret_cast<const half8_t*>(bias + (idx << 3));
        const half8_t r = *reinterpret_cast<const half8_t*>(x + (int64_t)row * D + (idx << 3));
        float4_t a0, a1;
        if (ST > 0) {
          float4_t t0[ST > 0 ? ST : 1], t1[ST > 0 ? ST : 1];
#pragma unroll
          for (int i = 0; i < ST; ++i) {
            t0[i] = *reinterpret_cast<const float4_t*>(p + i * slice);
            t1[i] = *reinterpret_cast<const float4_t*>(p + i * slice + 4);
          }
          a0 = t0[0];
          a1 = t1[0];
#pragma unroll
          for (int i = 1; i < ST; ++i) {
            a0 += t0[i];
            a1 += t1[i];
          }
        } else {
          a0 = *reinterpret_cast<const float4_t*>(p);
          a1 = *reinterpret_cast<const float4_t*>(p + 4);
          for (int i = 1; i < S; ++i) {
            a0 += *reinterpret_cast<const float4_t*>(p + i * slice);
            a1 += *reinterpret_cast<const float4_t*>(p + i * slice + 4);
          }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          float t = round_h(i < 4 ? a0[i] : a1[i - 4]);
          t = round_h(t + (float)b[i]);
          v[c][i] = (half_t)(t + (float)r[i]);
        }
        *reinterpret_cast<half8_t*>(x_out + (int64_t)row * D + (idx << 3)) = v[c];
      } else {
        v[c] = *reinterpret_cast<const half8_t*>(x + (int64_t)row * D + (idx << 3));
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) s += (float)v[c][i];
    }
  }
  if (!gamma) return;
  const float mean = block_sum(s, red) / (float)D;
  float q = 0.f;
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * THREADS;
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
    const int idx = threadIdx.x + c * THREADS;
    if (idx < nchunk) {
      half8_t o;
#pragma unroll
      for (int i = 0; i < 8; ++i)
        o[i] = (half_t)(((float)v[c][i] - mean) * rstd * (float)gv[c][i] + (float)bv[c][i]);
      half_t* dst = out_mb > 0 ? y + packed_act_offset(row, idx << 3, out_mb)
                               : y + (int64_t)row * D + (idx << 3);
      *reinterpret_cast<half8_t*>(dst) = o;
    }
  }
}

// Plain LayerNorm over thousands of rows: a workgroup walks rows blockIdx.x, + gridDim.x, ...
// with gamma and beta held in registers (read once per workgroup, not once per row) and the next
// row requested before the current one is reduced.  Per row the same threads do the same
// arithmetic in the same order as layernorm_f16_kernel<0, THREADS>: the results are its bits.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void layernorm_rows_kernel(
    const half_t* __restrict__ x, const half_t* __restrict__ gamma,
    const half_t* __restrict__ beta, half_t* __restrict__ y, int M, int D, float eps) {
  __shared__ float red[16];
  const int nchunk = D >> 3;
  half8_t v[LN_MAX_CHUNKS], nx[LN_MAX_CHUNKS], gv[LN_MAX_CHUNKS], bv[LN_MAX_CHUNKS];
  auto load_row = [&](int row, half8_t(&dst)[LN_MAX_CHUNKS]) {
#pragma unroll
    for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
      const int idx = threadIdx.x + c * THREADS;
      if (idx < nchunk)
        dst[c] = __builtin_nontemporal_load(
            reinterpret_cast<const half8_t*>(x + (int64_t)row * D + (idx << 3)));
    }
  };
#pragma unroll
  for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
    const int idx = threadIdx.x + c * THREADS;
    if (idx < nchunk) {
      gv[c] = *reinterpret_cast<const half8_t*>(gamma + (idx << 3));
      bv[c] = *reinterpret_cast<const half8_t*>(beta + (idx << 3));
    }
  }
  int row = blockIdx.x;
  if (row < M) load_row(row, v);
  for (; row < M; row += gridDim.x) {
    const int next = row + gridDim.x;
    if (next < M) load_row(next, nx);  // uniform
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
      const int idx = threadIdx.x + c * THREADS;
      if (idx < nchunk) {
#pragma unroll
        for (int i = 0; i < 8; ++i) s += (float)v[c][i];
      }
    }
    const float mean = block_sum(s, red) / (float)D;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < LN_MAX_CHUNKS; ++c) {
      const int idx = threadIdx.x + c * THREADS;
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
      const int idx = threadIdx.x + c * THREADS;
      if (idx < nchunk) {
        half8_t o;
#pragma unroll
        for (int i = 0; i < 8; ++i)
          o[i] = (half_t)(((float)v[c][i] - mean) * rstd * (float)gv[c][i] + (float)bv[c][i]);
        *reinterpret_cast<half8_t*>(y + (int64_t)row * D + (idx << 3)) = o;
      }
    }
#pragma unroll
    for (int c = 0; c < LN_MAX_CHUNKS; ++c) v[c] = nx[c];
  }
}

int check(const char* name, int64_t rows, int D, unsigned flags) {
  MSA_REQUIRE(rows >= 0 && rows <= 0x7fffffff, MSA_ERR_INVALID_ARG, "%s: rows=%lld out of range",
              name, (long long)rows);
  MSA_REQUIRE(D > 0 && D % 8 == 0 && D <= LN_THREADS * 8 * LN_MAX_CHUNKS, MSA_ERR_INVALID_ARG,
              "%s: D=%d must be a multiple of 8 and <= %d", name, D,
              LN_THREADS * 8 * LN_MAX_CHUNKS);
  MSA_REQUIRE((flags & ~MSA_OUT_PACKED) == 0, MSA_ERR_INVALID_ARG, "%s: unsupported flags 0x%x",
              name, flags);
  MSA_REQUIRE(!(flags & MSA_OUT_PACKED) || (rows <= MSA_PACKED_MAX_ROWS && D % 32 == 0),
              MSA_ERR_INVALID_ARG,
              "%s: packed output needs rows <= %d and D %% 32 == 0 (rows=%lld D=%d)", name,
              MSA_PACKED_MAX_ROWS, (long long)rows, D);
  return MSA_OK;
}

}  // namespace

extern "C" int msa_layernorm_f16(const void* x, const void* gamma, const void* beta, void* y,
                                 int64_t rows, int D, float eps, unsigned flags, void* stream) {
  MSA_REQUIRE(x && gamma && beta && y, MSA_ERR_INVALID_ARG, "msa_layernorm_f16: null pointer");
  int rc = check("msa_layernorm_f16", rows, D, flags);
  if (rc) return rc;
  if (rows == 0) return MSA_OK;
  const int out_mb = (flags & MSA_OUT_PACKED) ? packed_row_blocks(rows) : 0;
  // many rows: the narrowest workgroup that covers the row
  const int threads = rows <= 64 || D > 256 * 8 * LN_MAX_CHUNKS ? LN_THREADS
                      : D > 128 * 8 * LN_MAX_CHUNKS             ? 256
                                                                : 128;
  if (rows > 64 && out_mb == 0) {
    // up to 2048 threads per CU worth of workgroups, each walking its share of the rows
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0)
      cus = 256;
    const int64_t wgs = (int64_t)cus * (2048 / threads);
    const dim3 grid((unsigned)(rows < wgs ? rows : wgs));
    auto rk = threads == LN_THREADS ? layernorm_rows_kernel<LN_THREADS>
              : threads == 256      ? layernorm_rows_kernel<256>
                                    : layernorm_rows_kernel<128>;
    hipLaunchKernelGGL(rk, grid, dim3(threads), 0, (hipStream_t)stream, (const half_t*)x,
                       (const half_t*)gamma, (const half_t*)beta, (half_t*)y, (int)rows, D, eps);
    MSA_CHECK_LAUNCH("msa_layernorm_f16");
    return MSA_OK;
  }
  auto kernel = threads == LN_THREADS ? layernorm_f16_kernel<0, LN_THREADS>
                : threads == 256      ? layernorm_f16_kernel<0, 256>
                                      : layernorm_f16_kernel<0, 128>;
  hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(threads), 0, (hipStream_t)stream,
                     (const half_t*)x, (const float*)nullptr, 0, (const half_t*)nullptr,
                     (half_t*)nullptr, (const half_t*)gamma, (const half_t*)beta, (half_t*)y,
                     (int)rows, D, eps, out_mb);
  MSA_CHECK_LAUNCH("msa_layernorm_f16");
  return MSA_OK;
}

extern "C" int msa_residual_layernorm_f16(const float* part, int S, const void* bias, void* x,
                                          const void* gamma, const void* beta, void* y,
                                          int64_t rows, int D, float eps, unsigned flags,
                                          void* stream) {
  MSA_REQUIRE(part && bias && x, MSA_ERR_INVALID_ARG, "msa_residual_layernorm_f16: null pointer");
  MSA_REQUIRE(S >= 1, MSA_ERR_INVALID_ARG, "msa_residual_layernorm_f16: S=%d", S);
  MSA_REQUIRE((gamma == nullptr) == (beta == nullptr) && (gamma == nullptr) == (y == nullptr),
              MSA_ERR_INVALID_ARG,
              "msa_residual_layernorm_f16: gamma, beta and y must be given together");
  int rc = check("msa_residual_layernorm_f16", rows, D, flags);
  if (rc) return rc;
  if (rows == 0) return MSA_OK;
  const int out_mb = (flags & MSA_OUT_PACKED) ? packed_row_blocks(rows) : 0;
  auto kernel = S == 1   ? layernorm_f16_kernel<1>
                : S == 2 ? layernorm_f16_kernel<2>
                : S == 4 ? layernorm_f16_kernel<4>
                : S == 8 ? layernorm_f16_kernel<8>
                         : layernorm_f16_kernel<0>;
  hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(LN_THREADS), 0, (hipStream_t)stream,
                     (const half_t*)x, part, S, (const half_t*)bias, (half_t*)x,
                     (const half_t*)gamma, (const half_t*)beta, (half_t*)y, (int)rows, D, eps,
                     out_mb);
  MSA_CHECK_LAUNCH("msa_residual_layernorm_f16");
  return MSA_OK;
}
