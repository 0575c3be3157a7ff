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


// ---- split form: few (batch row, head) pairs, long histories ------------------------------------
// One workgroup per (b, h) leaves most of the chip idle when B*H is small, and a single CU pulls
// its K and V rows at a fraction of the HBM rate.  Here a decode step's attention is two
// launches: the scores of NS key ranges per (b, h) go to a scratch array, then one workgroup
// per (b, h) and 32-column slice of the head repeats the softmax over all scores (a few KB from
// L2) and streams its slice of the V rows.  Nothing is merged between workgroups, and every sum
// is formed in the order of attention_kernel at 1024 threads (what a small B*H runs there), so
// the two forms give identical bits.
constexpr int SPLIT_NS = 8;  // key ranges per (b, h) of the score kernel

template <int HD>
__global__ __launch_bounds__(256) void attention_scores_kernel(
    const half_t* __restrict__ q, const half_t* __restrict__ Kc,
    const uint8_t* __restrict__ key_pad_mask, int64_t mask_stride, float* __restrict__ scores,
    int H, int S0, int S_cap, const int32_t* __restrict__ len_dev) {
  constexpr int LPR = HD / 8, RPW = 64 / LPR;
  constexpr int U = 16;  // rows in flight per lane group: the ranges are short, latency is the cost
  const int bh = blockIdx.x / SPLIT_NS, split = blockIdx.x - bh * SPLIT_NS;
  const int b = bh / H, h = bh - b * H;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPR, rsel = lane / LPR;
  if (len_dev) {
    S0 = len_dev[b];
    if (S0 < 0) return;
    S0 = min(S0, S_cap - 1);
  }
  const int n_keys = S0 + 1;
  const int chunk = (n_keys + SPLIT_NS - 1) / SPLIT_NS;
  const int begin = split * chunk, end = min(n_keys, begin + chunk);
  if (begin >= end) return;
  const half_t* kbase = Kc + (int64_t)bh * S_cap * HD + sub * 8;
  const uint8_t* mrow = key_pad_mask ? key_pad_mask + (int64_t)b * mask_stride : nullptr;
  float* srow = scores + (int64_t)bh * S_cap;
  const half8_t qv =
      *reinterpret_cast<const half8_t*>(q + (int64_t)b * H * HD + h * HD + sub * 8);
  float qf[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) qf[i] = (float)qv[i];
  auto score = [&](const half8_t& kv, int kk) {  // the arithmetic of attention_kernel's score
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d = fmaf(qf[i], (float)kv[i], d);
#pragma unroll
    for (int o = LPR / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, MSA_WAVE);
    float sv = round_h(d);
    if (mrow && mrow[kk]) sv = -INFINITY;
    if (sub == 0) srow[kk] = sv;
  };
  const int kstride = 4 * RPW, last = end - 1;
  for (int key = begin + wave * RPW + rsel; key < end; key += U * kstride) {
    half8_t kv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      kv[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
          kbase + (int64_t)min(key + u * kstride, last) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (key + u * kstride < end) score(kv[u], key + u * kstride);
  }
}

template <int HD>
__global__ __launch_bounds__(16 * (64 / (HD / 8)) * 4) void attention_values_kernel(
    const float* __restrict__ scores, const half_t* __restrict__ Vc, half_t* __restrict__ out,
    int BH, int H, int S0, int S_cap, int out_mb, const int32_t* __restrict__ len_dev) {
  constexpr int LPR = HD / 8, RPW = 64 / LPR;
  constexpr int U = 16;  // rows in flight per lane group: the ranges are short, latency is the cost
  constexpr int CHAINS = 16 * RPW;       // (wave, row group) pairs of attention_kernel at 16 waves
  constexpr int SL = 4, NC = LPR / SL;   // lanes per row of a 32-column slice; slices per head
  constexpr int THREADS = CHAINS * SL;   // 256 (hd 128) or 512 (hd 64)
  constexpr int VT = 1024 / THREADS;     // threads of attention_kernel that one thread stands for
  extern __shared__ float smem[];
  float* sc = smem;  // [n_keys] scores, then probabilities
  __shared__ float red[16];
  __shared__ float chain_acc[CHAINS][32];
  // the slices of one (b, h) get workgroup numbers that are equal modulo 8: they run on one XCD
  // and share its L2 lines of the V rows
  const int id = blockIdx.x;
  const int bh = (id / (8 * NC)) * 8 + (id & 7), slice = (id >> 3) % NC;
  if (bh >= BH) return;
  const int b = bh / H, h = bh - b * H;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  if (len_dev) {
    S0 = len_dev[b];
    if (S0 < 0) return;
    S0 = min(S0, S_cap - 1);
  }
  const int n_keys = S0 + 1, last = n_keys - 1;
  const int chain = t / SL, sub = slice * SL + t % SL;  // sub: the lane's 8 columns of the head
  const half_t* vbase = Vc + (int64_t)bh * S_cap * HD + sub * 8;
  // the first V rows are requested before the softmax
  half8_t vpre[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    vpre[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
        vbase + (int64_t)min(chain + u * CHAINS, last) * HD));

  const float* srow = scores + (int64_t)bh * S_cap;
  float lmax = -INFINITY;
  for (int i = t; i < n_keys; i += THREADS) {
    const float v = srow[i];
    sc[i] = v;
    lmax = fmaxf(lmax, v);
  }
  const float m = block_max(lmax, red);  // barriers inside also publish sc[]
  // softmax sums in the order of 1024 threads: thread t stands for threads t + THREADS * j
  float wsum[VT];
#pragma unroll
  for (int j = 0; j < VT; ++j) {
    float lsum = 0.f;
    for (int i = t + THREADS * j; i < n_keys; i += 1024) {
      const float e = expf(sc[i] - m);
      sc[i] = e;
      lsum += e;
    }
    wsum[j] = wave_sum(lsum);
  }
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < VT; ++j) red[wave + (THREADS / 64) * j] = wsum[j];
  }
  __syncthreads();
  float denom = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) denom += red[i];
  for (int i = t; i < n_keys; i += THREADS) sc[i] = round_h(sc[i] / denom);
  __syncthreads();

  // chain c walks keys c, c + CHAINS, ... like (wave c / RPW, row group c % RPW) there
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  auto weigh = [&](const half8_t& vv, int kk) {
    if (kk < n_keys) {
      const float p = sc[kk];
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(p, (float)vv[i], acc[i]);
    }
  };
#pragma unroll
  for (int u = 0; u < U; ++u) weigh(vpre[u], chain + u * CHAINS);
  for (int key = chain + U * CHAINS; key < n_keys; key += U * CHAINS) {
    half8_t vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      vv[u] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(
          vbase + (int64_t)min(key + u * CHAINS, last) * HD));
#pragma unroll
    for (int u = 0; u < U; ++u) weigh(vv[u], key + u * CHAINS);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) chain_acc[chain][(t % SL) * 8 + i] = acc[i];
  __syncthreads();
  if (t < 32) {
    // per wave the row groups as a pairwise tree (the xor shuffles there), then the waves in turn
    float s = 0.f;
    for (int w = 0; w < 16; ++w) {
      float g[RPW];
#pragma unroll
      for (int r = 0; r < RPW; ++r) g[r] = chain_acc[w * RPW + r][t];
#pragma unroll
      for (int o = 1; o < RPW; o <<= 1)
#pragma unroll
        for (int r = 0; r < RPW; r += 2 * o) g[r] += g[r + o];
      s += g[0];
    }
    const int col = h * HD + slice * 32 + t;
    if (out_mb > 0)
      out[packed_act_offset(b, col, out_mb)] = (half_t)s;
    else
      out[(int64_t)b * H * HD + col] = (half_t)s;
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
  MSA_REQUIRE(!(flags & MSA_OUT_PACKED) || (T == 1 && B <= MSA_PACKED_MAX_ROWS),
              MSA_ERR_INVALID_ARG,
              "msa_attention_f16: packed output needs T == 1 and B <= %d (T=%d B=%d)",
              MSA_PACKED_MAX_ROWS, T, B);
  const int out_mb = (flags & MSA_OUT_PACKED) ? packed_row_blocks(B) : 0;
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

extern "C" int64_t msa_attention_split_workspace_bytes(int B, int H, int S_cap) {
  if (B < 1 || H < 1 || S_cap < 1) return 0;
  return (int64_t)B * H * S_cap * (int64_t)sizeof(float);
}

extern "C" int msa_attention_prefers_split(int B, int H, int hd, int n_keys) {
  // Measured: the two launches cost two rounds of fixed latencies (launch, first loads, the
  // softmax over all scores) and win only once a pair's K and V rows keep a single CU busy for
  // several times that: from about 4096 keys at head_dim 128 (B*H = 32: 41.7 -> 37.9 us; 8000
  // keys: 79 -> 64 us), and only for very few pairs (B*H = 128 is slower at every length).
  return (int64_t)B * H <= 64 && (int64_t)n_keys * hd >= 512 * 1024;
}

extern "C" int msa_attention_split_f16(const void* q, const void* Kcache, const void* Vcache,
                                       const uint8_t* key_pad_mask, int64_t mask_stride, void* out,
                                       void* workspace, int B, int H, int hd, int S0, int S_cap,
                                       unsigned flags, const int32_t* len_dev, void* stream) {
  const char* name = "msa_attention_split_f16";
  MSA_REQUIRE(q && Kcache && Vcache && out && workspace, MSA_ERR_INVALID_ARG, "%s: null pointer",
              name);
  MSA_REQUIRE(B > 0 && H > 0 && S0 >= 0, MSA_ERR_INVALID_ARG, "%s: bad shape B=%d H=%d S0=%d", name,
              B, H, S0);
  MSA_REQUIRE(hd == 64 || hd == 128, MSA_ERR_INVALID_ARG,
              "%s: head_dim %d not supported (64 or 128)", name, hd);
  MSA_REQUIRE((int64_t)S0 + 1 <= S_cap, MSA_ERR_CAPACITY,
              "%s: S0 + 1 = %d exceeds the cache capacity %d", name, S0 + 1, S_cap);
  MSA_REQUIRE((len_dev ? S_cap : S0 + 1) <= 8192, MSA_ERR_CAPACITY,
              "%s: more keys than the 8192 the score buffer holds", name);
  MSA_REQUIRE(!key_pad_mask || mask_stride >= S0 + 1, MSA_ERR_INVALID_ARG,
              "%s: mask_stride %lld shorter than %d keys", name, (long long)mask_stride, S0 + 1);
  MSA_REQUIRE((flags & ~MSA_OUT_PACKED) == 0, MSA_ERR_INVALID_ARG, "%s: unsupported flags 0x%x",
              name, flags);
  MSA_REQUIRE(!(flags & MSA_OUT_PACKED) || B <= MSA_PACKED_MAX_ROWS, MSA_ERR_INVALID_ARG,
              "%s: packed output needs B <= %d (B=%d)", name, MSA_PACKED_MAX_ROWS, B);
  const int64_t BH = (int64_t)B * H;
  MSA_REQUIRE(BH * SPLIT_NS <= 0x7fffffff, MSA_ERR_INVALID_ARG, "%s: B*H too large", name);
  const int out_mb = (flags & MSA_OUT_PACKED) ? packed_row_blocks(B) : 0;
  const size_t lds = (size_t)(len_dev ? S_cap : S0 + 1) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  const dim3 g1((unsigned)(BH * SPLIT_NS));
  const int nc = hd / 32;
  const dim3 g2((unsigned)(((BH + 7) / 8) * 8 * nc));
  if (hd == 64) {
    hipLaunchKernelGGL(attention_scores_kernel<64>, g1, dim3(256), 0, s, (const half_t*)q,
                       (const half_t*)Kcache, key_pad_mask, mask_stride, (float*)workspace, H, S0,
                       S_cap, len_dev);
    MSA_CHECK_LAUNCH(name);
    hipLaunchKernelGGL(attention_values_kernel<64>, g2, dim3(512), lds, s,
                       (const float*)workspace, (const half_t*)Vcache, (half_t*)out, (int)BH, H, S0,
                       S_cap, out_mb, len_dev);
  } else {
    hipLaunchKernelGGL(attention_scores_kernel<128>, g1, dim3(256), 0, s, (const half_t*)q,
                       (const half_t*)Kcache, key_pad_mask, mask_stride, (float*)workspace, H, S0,
                       S_cap, len_dev);
    MSA_CHECK_LAUNCH(name);
    hipLaunchKernelGGL(attention_values_kernel<128>, g2, dim3(256), lds, s,
                       (const float*)workspace, (const half_t*)Vcache, (half_t*)out, (int)BH, H, S0,
                       S_cap, out_mb, len_dev);
  }
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}
