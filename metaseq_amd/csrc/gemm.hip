// y[M,N] = epilogue(x[M,K] . W[N,K]^T) on fp16 MFMA with fp32 accumulation.
//
// Two kernels behind one entry point:
//   * skinny (M <= 64, the decode step): HBM-bound weight streaming.  A workgroup owns 16
//     rows of W; its 4 waves take interleaved 32-wide K steps, load W straight from HBM into
//     MFMA A-operand registers (16 bytes per lane, 64 contiguous bytes per row per
//     instruction), multiply against the M activation rows (B operand) and reduce across
//     waves through LDS in a fixed order, so results are run-to-run deterministic.
//   * tiled (any M, the prefill): 128x128x32 LDS double-buffered tiles, 4 waves of 64x64,
//     32x32x16 MFMA.
// Both share one epilogue that reproduces the reference's fp16 rounding points, and a QKV
// mode that scatters K/V into the per-layer cache and scales Q.
#include <math.h>

#include "common.h"

namespace {

enum { MODE_PLAIN = 0, MODE_QKV = 1 };

struct Epilogue {
  const half_t* bias;
  const half_t* residual;
  half_t* y;
  int N;
  unsigned flags;
  // MODE_QKV
  half_t* q_out;
  half_t* Kc;
  half_t* Vc;
  int T, H, hd, S0, S_cap;
  float qscale;
};

// 4 consecutive output columns n..n+3 of row m
template <int MODE>
__device__ __forceinline__ void epilogue4(const Epilogue& e, int64_t m, int n, float4_t acc) {
  float t[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) t[i] = round_h(acc[i]);
  if (e.bias) {
    const half4_t b = *reinterpret_cast<const half4_t*>(e.bias + n);
#pragma unroll
    for (int i = 0; i < 4; ++i) t[i] = round_h(t[i] + (float)b[i]);
  }
  if (MODE == MODE_PLAIN) {
    if (e.flags & MSA_EPI_RELU) {
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = fmaxf(t[i], 0.f);
    }
    if (e.residual) {
      const half4_t r = *reinterpret_cast<const half4_t*>(e.residual + m * e.N + n);
#pragma unroll
      for (int i = 0; i < 4; ++i) t[i] = round_h(t[i] + (float)r[i]);
    }
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (half_t)t[i];
    *reinterpret_cast<half4_t*>(e.y + m * e.N + n) = o;
  } else {
    const int D = e.H * e.hd;
    const int part = n / D, c = n - part * D;  // 0 = K, 1 = V, 2 = Q
    half4_t o;
    if (part == 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)(t[i] * e.qscale);
      *reinterpret_cast<half4_t*>(e.q_out + m * D + c) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)t[i];
      const int h = c / e.hd, d = c - h * e.hd;
      const int64_t b = m / e.T, tt = m - b * e.T;
      half_t* dst = (part == 0 ? e.Kc : e.Vc) +
                    ((b * e.H + h) * (int64_t)e.S_cap + e.S0 + tt) * e.hd + d;
      *reinterpret_cast<half4_t*>(dst) = o;
    }
  }
}

// ---- int8 -> fp16 dequantisation in registers --------------------------------------
// 8 int8 (two dwords) times an fp16 per-row scale -> 8 fp16, each round(q * scale).
__device__ __forceinline__ half8_t dequant8(uint32_t lo, uint32_t hi, half_t scale) {
  half8_t r;
  const uint32_t w[2] = {lo, hi};
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = (int)(int8_t)((w[j] >> (8 * i)) & 0xff);
      r[j * 4 + i] = (half_t)((float)q * (float)scale);
    }
  }
  return r;
}

// ---- skinny kernel --------------------------------------------------------------------
constexpr int SK_THREADS = 256;
constexpr int SK_WAVES = 4;
constexpr int SK_ROWS = 16;  // W rows per workgroup
constexpr int SK_U = 4;      // K steps in flight per wave

template <int MB, bool W8, int MODE>
__global__ __launch_bounds__(SK_THREADS) void linear_skinny_kernel(
    const half_t* __restrict__ x, const void* __restrict__ Wv, const half_t* __restrict__ scales,
    int M, int N, int K, Epilogue epi) {
  __shared__ float4_t part[SK_WAVES][MB][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * SK_ROWS;
  const int nks = K >> 5;  // 32-wide K steps

  const half_t* xrow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    int m = mb * 16 + r;
    if (m >= M) m = M - 1;  // rows past M are computed on valid memory and discarded
    xrow[mb] = x + (int64_t)m * K + g * 8;
  }
  float4_t acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  if (!W8) {
    const half_t* wrow = (const half_t*)Wv + (int64_t)(n0 + r) * K + g * 8;
    int ks = wave;
    for (; ks + SK_WAVES * (SK_U - 1) < nks; ks += SK_WAVES * SK_U) {
      half8_t a[SK_U], b[SK_U][MB];
#pragma unroll
      for (int u = 0; u < SK_U; ++u) {
        const int k = (ks + SK_WAVES * u) << 5;
        a[u] = *reinterpret_cast<const half8_t*>(wrow + k);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) b[u][mb] = *reinterpret_cast<const half8_t*>(xrow[mb] + k);
      }
#pragma unroll
      for (int u = 0; u < SK_U; ++u)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u], b[u][mb], acc[mb], 0, 0, 0);
    }
    for (; ks < nks; ks += SK_WAVES) {
      const int k = ks << 5;
      const half8_t a = *reinterpret_cast<const half8_t*>(wrow + k);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const half8_t b = *reinterpret_cast<const half8_t*>(xrow[mb] + k);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[mb], 0, 0, 0);
      }
    }
  } else {
    // int8 weights: one 8-byte load per lane per K step, dequantised in registers
    const int8_t* wrow = (const int8_t*)Wv + (int64_t)(n0 + r) * K + g * 8;
    const half_t sc = scales[n0 + r];
    for (int ks = wave; ks < nks; ks += SK_WAVES) {
      const int k = ks << 5;
      const uint2 w = *reinterpret_cast<const uint2*>(wrow + k);
      const half8_t a = dequant8(w.x, w.y, sc);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const half8_t b = *reinterpret_cast<const half8_t*>(xrow[mb] + k);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[mb], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int mb = 0; mb < MB; ++mb) part[wave][mb][lane] = acc[mb];
  __syncthreads();
  for (int idx = threadIdx.x; idx < MB * 64; idx += SK_THREADS) {
    const int mb = idx >> 6, l = idx & 63;
    float4_t s = part[0][mb][l];
#pragma unroll
    for (int w = 1; w < SK_WAVES; ++w) s += part[w][mb][l];
    // MFMA 16x16 output: lane l holds column (l & 15) of B = activation row m, and rows
    // 4*(l >> 4) .. +3 of A = output features n.
    const int m = mb * 16 + (l & 15);
    const int n = n0 + ((l >> 4) << 2);
    if (m < M) epilogue4<MODE>(epi, m, n, s);
  }
}

// ---- tiled kernel ---------------------------------------------------------------------
constexpr int TL_BM = 128, TL_BN = 128, TL_BK = 32, TL_LD = TL_BK + 8, TL_THREADS = 256;

template <bool W8, int MODE>
__global__ __launch_bounds__(TL_THREADS) void linear_tiled_kernel(
    const half_t* __restrict__ x, const void* __restrict__ Wv, const half_t* __restrict__ scales,
    int64_t M, int N, int K, Epilogue epi) {
  __shared__ __attribute__((aligned(16))) half_t lx[2][TL_BM * TL_LD];
  __shared__ __attribute__((aligned(16))) half_t lw[2][TL_BN * TL_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int li = lane & 31, lg = lane >> 5;
  const int64_t m0 = (int64_t)blockIdx.y * TL_BM;
  const int n0 = blockIdx.x * TL_BN;
  const int nkt = K / TL_BK;

  // staging: each thread moves two 16-byte chunks of each operand tile
  int srow[2], scol[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + TL_THREADS * i;
    srow[i] = c >> 2;
    scol[i] = (c & 3) << 3;
  }
  half8_t rx[2], rw[2];

  auto load_tile = [&](int kt) {
    const int k0 = kt * TL_BK;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t m = m0 + srow[i];
      if (m < M)
        rx[i] = *reinterpret_cast<const half8_t*>(x + m * K + k0 + scol[i]);
      else
        rx[i] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      const int n = n0 + srow[i];
      if (n < N) {
        if (!W8) {
          rw[i] = *reinterpret_cast<const half8_t*>((const half_t*)Wv + (int64_t)n * K + k0 +
                                                    scol[i]);
        } else {
          const uint2 w =
              *reinterpret_cast<const uint2*>((const int8_t*)Wv + (int64_t)n * K + k0 + scol[i]);
          rw[i] = dequant8(w.x, w.y, scales[n]);
        }
      } else {
        rw[i] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<half8_t*>(&lx[buf][srow[i] * TL_LD + scol[i]]) = rx[i];
      *reinterpret_cast<half8_t*>(&lw[buf][srow[i] * TL_LD + scol[i]]) = rw[i];
    }
  };

  float16_t acc[2][2];  // [tn][tm]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

  load_tile(0);
  store_tile(0);
  __syncthreads();
  for (int kt = 0; kt < nkt; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nkt) load_tile(kt + 1);
#pragma unroll
    for (int ks = 0; ks < TL_BK / 16; ++ks) {
      half8_t fa[2], fb[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fa[t] = *reinterpret_cast<const half8_t*>(
            &lw[buf][(wn * 64 + t * 32 + li) * TL_LD + ks * 16 + lg * 8]);
        fb[t] = *reinterpret_cast<const half8_t*>(
            &lx[buf][(wm * 64 + t * 32 + li) * TL_LD + ks * 16 + lg * 8]);
      }
#pragma unroll
      for (int tn = 0; tn < 2; ++tn)
#pragma unroll
        for (int tm = 0; tm < 2; ++tm)
          acc[tn][tm] =
              __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[tn], fb[tm], acc[tn][tm], 0, 0, 0);
    }
    if (kt + 1 < nkt) store_tile(buf ^ 1);
    __syncthreads();
  }

  // MFMA 32x32 output: lane holds column (lane & 31) of B = activation row, and for register
  // v the A row 8*(v/4) + 4*(lane >> 5) + (v & 3) = output feature.
#pragma unroll
  for (int tn = 0; tn < 2; ++tn)
#pragma unroll
    for (int tm = 0; tm < 2; ++tm) {
      const int64_t m = m0 + wm * 64 + tm * 32 + li;
      if (m >= M) continue;
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        const int n = n0 + wn * 64 + tn * 32 + blk * 8 + lg * 4;
        if (n >= N) continue;
        const float4_t v = {acc[tn][tm][blk * 4 + 0], acc[tn][tm][blk * 4 + 1],
                            acc[tn][tm][blk * 4 + 2], acc[tn][tm][blk * 4 + 3]};
        epilogue4<MODE>(epi, m, n, v);
      }
    }
}

template <bool W8, int MODE>
int launch_linear(const void* x, const void* W, const void* scales, int64_t M, int N, int K,
                  const Epilogue& epi, hipStream_t s) {
  if (M <= 64 && N % SK_ROWS == 0) {
    const dim3 grid(N / SK_ROWS), block(SK_THREADS);
    const int MB = (int)((M + 15) / 16);
#define MSA_SK(mb)                                                                              \
  hipLaunchKernelGGL((linear_skinny_kernel<mb, W8, MODE>), grid, block, 0, s, (const half_t*)x, \
                     W, (const half_t*)scales, (int)M, N, K, epi)
    switch (MB) {
      case 1: MSA_SK(1); break;
      case 2: MSA_SK(2); break;
      case 3: MSA_SK(3); break;
      default: MSA_SK(4); break;
    }
#undef MSA_SK
  } else {
    const dim3 grid((N + TL_BN - 1) / TL_BN, (unsigned)((M + TL_BM - 1) / TL_BM));
    hipLaunchKernelGGL((linear_tiled_kernel<W8, MODE>), grid, dim3(TL_THREADS), 0, s,
                       (const half_t*)x, W, (const half_t*)scales, M, N, K, epi);
  }
  return MSA_OK;
}

int check_linear_args(const char* name, const void* x, const void* W, const void* y, int64_t M,
                      int N, int K) {
  MSA_REQUIRE(x && W && y, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(M >= 0 && M < (1ll << 31) && N > 0 && K > 0, MSA_ERR_INVALID_ARG,
              "%s: bad shape M=%lld N=%d K=%d", name, (long long)M, N, K);
  MSA_REQUIRE(K % 32 == 0 && N % 8 == 0, MSA_ERR_INVALID_ARG,
              "%s: K=%d must be a multiple of 32 and N=%d a multiple of 8", name, K, N);
  MSA_REQUIRE((M + TL_BM - 1) / TL_BM <= 65535, MSA_ERR_INVALID_ARG, "%s: M=%lld too large", name,
              (long long)M);
  return MSA_OK;
}

template <bool W8>
int linear_entry(const char* name, const void* x, const void* W, const void* scales,
                 const void* bias, const void* residual, void* y, int64_t M, int N, int K,
                 unsigned flags, void* stream) {
  int rc = check_linear_args(name, x, W, y, M, N, K);
  if (rc) return rc;
  MSA_REQUIRE(!W8 || scales, MSA_ERR_INVALID_ARG, "%s: null scales", name);
  MSA_REQUIRE((flags & ~MSA_EPI_RELU) == 0, MSA_ERR_INVALID_ARG, "%s: unknown flags 0x%x", name,
              flags);
  if (M == 0) return MSA_OK;
  Epilogue e{};
  e.bias = (const half_t*)bias;
  e.residual = (const half_t*)residual;
  e.y = (half_t*)y;
  e.N = N;
  e.flags = flags;
  launch_linear<W8, MODE_PLAIN>(x, W, scales, M, N, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

template <bool W8>
int qkv_entry(const char* name, const void* x, const void* W, const void* scales, const void* bqkv,
              void* q_out, void* Kc, void* Vc, int B, int T, int H, int hd, int S0, int S_cap,
              int K, void* stream) {
  MSA_REQUIRE(q_out && Kc && Vc, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(B > 0 && T > 0 && H > 0 && hd > 0 && hd % 8 == 0 && S0 >= 0, MSA_ERR_INVALID_ARG,
              "%s: bad shape B=%d T=%d H=%d hd=%d S0=%d", name, B, T, H, hd, S0);
  MSA_REQUIRE((int64_t)S0 + T <= S_cap, MSA_ERR_CAPACITY,
              "%s: S0 + T = %d exceeds the cache capacity %d", name, S0 + T, S_cap);
  const int64_t M = (int64_t)B * T;
  const int N = 3 * H * hd;
  int rc = check_linear_args(name, x, W, q_out, M, N, K);
  if (rc) return rc;
  MSA_REQUIRE(!W8 || scales, MSA_ERR_INVALID_ARG, "%s: null scales", name);
  Epilogue e{};
  e.bias = (const half_t*)bqkv;
  e.N = N;
  e.q_out = (half_t*)q_out;
  e.Kc = (half_t*)Kc;
  e.Vc = (half_t*)Vc;
  e.T = T;
  e.H = H;
  e.hd = hd;
  e.S0 = S0;
  e.S_cap = S_cap;
  e.qscale = (float)pow((double)hd, -0.5);  // the reference's head_dim ** -0.5, cast to fp32
  launch_linear<W8, MODE_QKV>(x, W, scales, M, N, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

}  // namespace

extern "C" size_t msa_linear_workspace_bytes(int64_t, int, int) { return 0; }

extern "C" int msa_linear_f16(const void* x, const void* W, const void* bias, const void* residual,
                              void* y, int64_t M, int N, int K, unsigned flags, void*, size_t,
                              void* stream) {
  return linear_entry<false>("msa_linear_f16", x, W, nullptr, bias, residual, y, M, N, K, flags,
                             stream);
}

extern "C" int msa_linear_w8a16(const void* x, const int8_t* Wq, const void* scales,
                                const void* bias, const void* residual, void* y, int64_t M, int N,
                                int K, unsigned flags, void*, size_t, void* stream) {
  return linear_entry<true>("msa_linear_w8a16", x, Wq, scales, bias, residual, y, M, N, K, flags,
                            stream);
}

extern "C" int msa_qkv_proj_f16(const void* x, const void* Wqkv, const void* bqkv, void* q_out,
                                void* Kcache, void* Vcache, int B, int T, int H, int hd, int S0,
                                int S_cap, int K, void*, size_t, void* stream) {
  return qkv_entry<false>("msa_qkv_proj_f16", x, Wqkv, nullptr, bqkv, q_out, Kcache, Vcache, B, T,
                          H, hd, S0, S_cap, K, stream);
}

extern "C" int msa_qkv_proj_w8a16(const void* x, const int8_t* Wq, const void* scales,
                                  const void* bqkv, void* q_out, void* Kcache, void* Vcache, int B,
                                  int T, int H, int hd, int S0, int S_cap, int K, void*, size_t,
                                  void* stream) {
  return qkv_entry<true>("msa_qkv_proj_w8a16", x, Wq, scales, bqkv, q_out, Kcache, Vcache, B, T, H,
                         hd, S0, S_cap, K, stream);
}
