// Decode attention (one new query per row) over the contiguous per-layer KV cache
// [B, H, S_cap, hd]; queries with T > 1 go to the MFMA kernel in attention_prefill.hip.
//
// One workgroup per (batch row, head).  The workgroup streams the K rows of its head
// once (16-byte loads, hd/8 lanes per key row, so each wave instruction reads whole 128- or
// 256-byte rows), forms the fp16-rounded scores in LDS, normalises them with an fp32 softmax
// whose probabilities are rounded to fp16 exactly like the reference's cast-back, then streams
// the V rows once.  With T == 1 (a decode step) the kernel moves 2*S*hd*2 bytes per (b, h)
// and nothing else: it is bound by HBM bandwidth.
#include <math.h>

#include "common.h"

namespace {

template <int HD>
__global__ void attention_kernel(const half_t* __restrict__ q, const half_t* __restrict__ Kc,
                                 const half_t* __restrict__ Vc,
                                 const uint8_t* __restrict__ key_pad_mask, int64_t mask_stride,
                                 half_t* __restrict__ out, int H, int T, int S0, int S_cap,
                                 int out_mb, const int32_t* __restrict__ len_dev) {
  constexpr int LPR = HD / 8;    // lanes per key row (16 bytes each)
  constexpr int RPW = 64 / LPR;  // key rows per wave instruction
  extern __shared__ float smem[];
  float* sc = smem;  // [n_keys] scores, then probabilities
  __shared__ float red[16];
  __shared__ float oacc[16][HD];

  const int bh = blockIdx.x, t = blockIdx.y;
  const int b = bh / H, h = bh - b * H;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int sub = lane % LPR, rsel = lane / LPR;
  if (len_dev) {  // per-row cache lengths kept on the device (ragged batches, graph replay)
    S0 = len_dev[b];
    if (S0 < 0) return;  // inactive row: nothing to attend, the output row keeps its contents
    S0 = min(S0, S_cap - 1);
  }
  const int n_keys = S0 + t + 1;
  const int D = H * HD;

  const half_t* kbase = Kc + (int64_t)bh * S_cap * HD + sub * 8;
  const half_t* vbase = Vc + (int64_t)bh * S_cap * HD + sub * 8;
  const uint8_t* mrow = key_pad_mask ? key_pad_mask + (int64_t)b * mask_stride : nullptr;

  const half8_t qv =
      *reinterpret_cast<const half8_t*>(q + ((int64_t)b * T + t) * D + h * HD + sub * 8);
  float qf[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];

  // ---- scores ----
  constexpr int U = 8;  // key rows in flight per lane group
  const int kstride = nw * RPW;
  float lmax = -INFINITY;
  auto score = [&](const half8_t& kv, int kk) {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d = fmaf(qf[i], (float)kv[i], d);
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, MSA_WAVE);
    float s = round_h(d);
    if (mrow && mrow[kk]) s = -INFINITY;
    if (sub == 0) sc[kk] = s;
    lmax = fmaxf(lmax, s);
  };
  // U rows per lane group are requested before the first is used, also in the last (or only)
  // round, where rows past the end re-read the last key and are not scored: a short history
  // (few rounds, or less than one) is one memory latency, not one per row
  const int last = n_keys - 1;
  int key = wave * RPW + rsel;
  for (; key + (U - 1) * kstride < n_keys; key += U * kstride) {  // whole rounds
    half8_t kv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      kv[u] = __builtin_nontemporal_load(
          reinterpret_cast<const half8_t*>(kbase + (int64_t)(key + u * kstride) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u) score(kv[u], key + u * kstride);
  }
  if (key < n_keys) {
    half8_t kv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      kv[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
          kbase + (int64_t)min(key + u * kstride, last) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (key + u * kstride < n_keys) score(kv[u], key + u * kstride);
  }

  // the first V rows are requested before the softmax so that HBM stays busy through it
  half8_t vpre[U];
  const int vkey0 = wave * RPW + rsel;
#pragma unroll
  for (int u = 0; u < U; ++u)
    vpre[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
        vbase + (int64_t)min(vkey0 + u * kstride, last) * HD));
  const float m = block_max(lmax, red);  // barriers inside also publish sc[]

  // ---- softmax in fp32, probabilities rounded to fp16 ----
  float lsum = 0.f;
  for (int i = threadIdx.x; i < n_keys; i += blockDim.x) {
    const float e = expf(sc[i] - m);
    sc[i] = e;
    lsum += e;
  }
  const float denom = block_sum(lsum, red);
  for (int i = threadIdx.x; i < n_keys; i += blockDim.x) sc[i] = round_h(sc[i] / denom);
  __syncthreads();

  // ---- weighted sum of V rows ----
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // rows past the end are skipped, not weighted by zero: what a clamped load returns is a real
  // row, but a probability read past the end of sc[] is not a number to multiply with
  auto weigh = [&](const half8_t& vv, int kk) {
    if (kk < n_keys) {
      const float p = sc[kk];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(p, (float)vv[i], acc[i]);
    }
  };
#pragma unroll
  for (int u = 0; u < U; ++u) weigh(vpre[u], vkey0 + u * kstride);
  for (key = vkey0 + U * kstride; key + (U - 1) * kstride < n_keys; key += U * kstride) {
    half8_t vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      vv[u] = __builtin_nontemporal_load(
          reinterpret_cast<const half8_t*>(vbase + (int64_t)(key + u * kstride) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float p = sc[key + u * kstride];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(p, (float)vv[u][i], acc[i]);
    }
  }
  if (key < n_keys) {
    half8_t vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      vv[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
          vbase + (int64_t)min(key + u * kstride, last) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u) weigh(vv[u], key + u * kstride);
  }
  // combine the RPW row groups of a wave, then the waves, in a fixed order
#pragma unroll
  for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], o, MSA_WAVE);
  if (rsel == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) oacc[wave][sub * 8 + i] = acc[i];
  }
  __syncthreads();
  for (int d = threadIdx.x; d < HD; d += blockDim.x) {
    float s = 0.f;
    for (int w = 0; w < nw; ++w) s += oacc[w][d];
    if (out_mb > 0)  // packed activation layout of the decode GEMMs (T == 1: row = b)
      out[packed_act_offset(b, h * HD + d, out_mb)] = (half_t)s;
    else
      out[((int64_t)b * T + t) * D + h * HD + d] = (half_t)s;
  }
}

}  // namespace

extern "C" int msa_attention_f16(const void* q, const void* Kcache, const void* Vcache,
                                 const uint8_t* key_pad_mask, int64_t mask_stride, void* out, int B,
                                 int H, int hd, int T, int S0, int S_cap, unsigned flags,
                                 const int32_t* len_dev, void* stream) {
  MSA_REQUIRE(q && Kcache && Vcache && out, MSA_ERR_INVALID_ARG, "msa_attention_f16: null pointer");
  MSA_REQUIRE(B > 0 && H > 0 && T > 0 && S0 >= 0, MSA_ERR_INVALID_ARG,
              "msa_attention_f16: bad shape B=%d H=%d T=%d S0=%d", B, H, T, S0);
  MSA_REQUIRE(hd == 64 || hd == 128, MSA_ERR_INVALID_ARG,
              "msa_attention_f16: head_dim %d not supported (64 or 128)", hd);
  MSA_REQUIRE((int64_t)S0 + T <= S_cap, MSA_ERR_CAPACITY,
              "msa_attention_f16: S0 + T = %d exceeds the cache capacity %d", S0 + T, S_cap);
  MSA_REQUIRE(S0 + T <= 8192, MSA_ERR_CAPACITY,
              "msa_attention_f16: %d keys exceed the 8192 the score buffer holds", S0 + T);
  MSA_REQUIRE(!key_pad_mask || mask_stride >= S0 + T, MSA_ERR_INVALID_ARG,
              "msa_attention_f16: mask_stride %lld shorter than %d keys", (long long)mask_stride,
              S0 + T);
  MSA_REQUIRE(T <= 65535, MSA_ERR_INVALID_ARG, "msa_attention_f16: T=%d too large", T);
  MSA_REQUIRE((flags & ~MSA_OUT_PACKED) == 0, MSA_ERR_INVALID_ARG,
              "msa_attention_f16: unsupported flags 0x%x", flags);
  MSA_REQUIRE(!(flags & MSA_OUT_PACKED) || (T == 1 && B <= 64), MSA_ERR_INVALID_ARG,
              "msa_attention_f16: packed output needs T == 1 and B <= 64 (T=%d B=%d)", T, B);
  const int out_mb = (flags & MSA_OUT_PACKED) ? (B + 15) / 16 : 0;
  MSA_REQUIRE(!len_dev || T == 1, MSA_ERR_INVALID_ARG,
              "msa_attention_f16: a device-side length needs T == 1");
  MSA_REQUIRE(!len_dev || S_cap <= 8192, MSA_ERR_CAPACITY,
              "msa_attention_f16: S_cap %d exceeds the 8192 the score buffer holds", S_cap);
  const int64_t BH = (int64_t)B * H;
  if (T > 1) {
    MSA_REQUIRE(BH <= 0x7fffffff, MSA_ERR_INVALID_ARG, "msa_attention_f16: B*H too large");
    msa_launch_prefill_attention(q, Kcache, Vcache, key_pad_mask, mask_stride, out, B, H, hd, T,
                                 S0, S_cap, (hipStream_t)stream);
    MSA_CHECK_LAUNCH("msa_attention_f16");
    return MSA_OK;
  }
  // few (b,h) pairs: spend more waves on each so the chip still fills
  const int threads = (T == 1 && BH < 512) ? 1024 : 256;
  const size_t lds = (size_t)(len_dev ? S_cap : S0 + T) * sizeof(float);
  const dim3 grid((unsigned)BH, (unsigned)T);
  hipStream_t s = (hipStream_t)stream;
  if (hd == 64)
    hipLaunchKernelGGL(attention_kernel<64>, grid, dim3(threads), lds, s, (const half_t*)q,
                       (const half_t*)Kcache, (const half_t*)Vcache, key_pad_mask, mask_stride,
                       (half_t*)out, H, T, S0, S_cap, out_mb, len_dev);
  else
    hipLaunchKernelGGL(attention_kernel<128>, grid, dim3(threads), lds, s, (const half_t*)q,
                       (const half_t*)Kcache, (const half_t*)Vcache, key_pad_mask, mask_stride,
                       (half_t*)out, H, T, S0, S_cap, out_mb, len_dev);
  MSA_CHECK_LAUNCH("msa_attention_f16");
  return MSA_OK;
}
