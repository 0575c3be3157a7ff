// Per-row vocabulary reductions of the greedy generation loop: fp32 log-sum-exp over fp16
// logits, masked arg-max with lowest-index tie-break, and target log-probability gather.
// One workgroup per logits row; the row (V * 2 bytes) is read twice from cache/HBM.
#include <math.h>

#include "common.h"

namespace {

constexpr int SM_THREADS = 1024;

struct RowStats {
  float max;  // max of z = logit / temperature over the whole row
  float lse;  // log(sum(exp(z - max)))   (so log_softmax(z) = z - max - lse)
};

// visits every element of a logits row as z = logit (/ temperature), 8 halves per load where the
// row is 16-byte aligned
template <typename F>
__device__ __forceinline__ void for_each_z(const half_t* __restrict__ row, int V, float temp,
                                           bool scale, F f) {
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int nv = V >> 3;
    for (int c = threadIdx.x; c < nv; c += blockDim.x) {
      const half8_t v = *reinterpret_cast<const half8_t*>(row + (c << 3));
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float z = (float)v[i];
        if (scale) z = z / temp;
        f((c << 3) + i, z);
      }
    }
    for (int i = (nv << 3) + threadIdx.x; i < V; i += blockDim.x) {
      float z = (float)row[i];
      if (scale) z = z / temp;
      f(i, z);
    }
  } else {
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      float z = (float)row[i];
      if (scale) z = z / temp;
      f(i, z);
    }
  }
}

__device__ __forceinline__ RowStats row_logsumexp(const half_t* __restrict__ row, int V,
                                                  float temp, bool scale, float* red) {
  float mx = -INFINITY;
  bool nan = false;
  for_each_z(row, V, temp, scale, [&](int, float z) {
    nan |= (z != z);
    mx = fmaxf(mx, z);
  });
  mx = block_max(mx, red);
  const float any_nan = block_max(nan ? 1.f : 0.f, red);
  float s = 0.f;
  for_each_z(row, V, temp, scale, [&](int, float z) { s += expf(z - mx); });
  s = block_sum(s, red);
  RowStats r;
  r.max = mx;
  r.lse = any_nan > 0.f ? NAN : logf(s);
  return r;
}

__global__ __launch_bounds__(SM_THREADS) void greedy_select_kernel(
    const half_t* __restrict__ logits, int64_t ld, int V, float temperature, bool scale,
    IdList banned, IdList stop, uint8_t* __restrict__ finished,
    const uint8_t* __restrict__ row_mode, int force_eos_all, int eos,
    int64_t* __restrict__ tok, int64_t tok_stride, float* __restrict__ score,
    int64_t score_stride, const int32_t* __restrict__ len_dev) {
  __shared__ float wm[16], ws[16], wbest[16], wnan[16];
  __shared__ int widx[16];
  const int b = blockIdx.x;
  const half_t* row = logits + (int64_t)b * ld;
  const unsigned rm = row_mode ? row_mode[b] : 0u;
  const bool only_eos = force_eos_all || (finished && finished[b]) || (rm & MSA_ROW_ONLY_EOS);
  const bool ban_early = rm & MSA_ROW_BAN_EARLY;  // eos and the stop ids are not eligible

  // single pass: running log-sum-exp over ALL ids, and the best eligible id (log-softmax is
  // monotone in z, so the arg-max of the masked log-probs is the arg-max of the masked z)
  float m = -INFINITY, s = 0.f, best = -INFINITY;
  int bidx = 0x7fffffff;
  bool nan = false;
  auto visit = [&](int i, float z) {  // arg-max bookkeeping of one id
    nan |= (z != z);
    bool ok = !(only_eos && i != eos) && !(ban_early && i == eos);
    for (int j = 0; j < banned.n; ++j) ok &= (banned.id[j] != i);
    if (ban_early)
      for (int j = 0; j < stop.n; ++j) ok &= (stop.id[j] != i);
    const float cand = ok ? z : -INFINITY;
    if (cand > best || (cand == best && i < bidx)) {
      best = cand;
      bidx = i;
    }
  };
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int nv = V >> 3;
    constexpr int UNR = 4;  // chunks requested together: one memory round trip per UNR chunks
    for (int c0 = threadIdx.x; c0 < nv; c0 += blockDim.x * UNR) {
      half8_t vv[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        vv[u] = *reinterpret_cast<const half8_t*>(row + (min(c0 + u * (int)blockDim.x, nv - 1) << 3));
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int c = c0 + u * blockDim.x;
        if (c >= nv) break;
        float z[8], cm = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          z[i] = (float)vv[u][i];
          if (scale) z[i] = z[i] / temperature;
          cm = fmaxf(cm, z[i]);
          visit((c << 3) + i, z[i]);
        }
        if (cm > m) {  // rescale once per 8 ids
          s *= __expf(m - cm);
          m = cm;
        }
        if (m > -INFINITY) {
#pragma unroll
          for (int i = 0; i < 8; ++i) s += __expf(z[i] - m);
        }
      }
    }
    for (int i = (nv << 3) + threadIdx.x; i < V; i += blockDim.x) {
      float z = (float)row[i];
      if (scale) z = z / temperature;
      visit(i, z);
      lse_merge(m, s, z, 1.f);
    }
  } else {
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      float z = (float)row[i];
      if (scale) z = z / temperature;
      visit(i, z);
      lse_merge(m, s, z, 1.f);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lse_merge(m, s, __shfl_xor(m, o, MSA_WAVE), __shfl_xor(s, o, MSA_WAVE));
    const float ob = __shfl_xor(best, o, MSA_WAVE);
    const int oi = __shfl_xor(bidx, o, MSA_WAVE);
    if (ob > best || (ob == best && oi < bidx)) {
      best = ob;
      bidx = oi;
    }
    nan |= (bool)__shfl_xor((int)nan, o, MSA_WAVE);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    wm[wave] = m;
    ws[wave] = s;
    wbest[wave] = best;
    widx[wave] = bidx;
    wnan[wave] = nan ? 1.f : 0.f;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      lse_merge(m, s, wm[w], ws[w]);
      if (wbest[w] > best || (wbest[w] == best && widx[w] < bidx)) {
        best = wbest[w];
        bidx = widx[w];
      }
      nan |= wnan[w] > 0.f;
    }
    // lprob = (z - max) - log(sum(exp(z - max))); a NaN anywhere, or no eligible finite id,
    // leaves every eligible log-prob at -inf and the lowest index wins
    float lp = (best - m) - logf(s);
    if (nan || !(best > -INFINITY)) {
      lp = -INFINITY;
      bidx = 0;
    }
    const int col = len_dev ? *len_dev : 0;  // column offset kept on the device (graph replay)
    tok[b * tok_stride + col] = bidx;
    score[b * score_stride + col] = lp;
    if (finished) {
      bool f = bidx == eos;
      for (int j = 0; j < stop.n; ++j) f |= (stop.id[j] == bidx);
      if (f) finished[b] = 1;
    }
  }
}

__global__ __launch_bounds__(SM_THREADS) void target_logprob_kernel(
    const half_t* __restrict__ logits, int64_t ld, int V, float temperature, bool scale,
    const int64_t* __restrict__ target, float* __restrict__ out) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const half_t* row = logits + r * ld;
  const RowStats st = row_logsumexp(row, V, temperature, scale, red);
  if (threadIdx.x == 0) {
    int64_t t = target[r];
    t = t < 0 ? 0 : (t >= V ? V - 1 : t);
    float z = (float)row[t];
    if (scale) z = z / temperature;
    out[r] = (z - st.max) - st.lse;
  }
}

// Merges the per-workgroup partials that the vocabulary projection's selection epilogue
// wrote for one row and finishes the step exactly as greedy_select_kernel does.
__global__ __launch_bounds__(256) void select_combine_kernel(
    const SelectPartial* __restrict__ partials, int n_parts, IdList stop,
    uint8_t* __restrict__ finished, int eos, int64_t* __restrict__ tok, int64_t tok_stride,
    float* __restrict__ score, int64_t score_stride, const int32_t* __restrict__ len_dev) {
  __shared__ float wm[4], ws[4], wbest[4], wnan[4];
  __shared__ int widx[4];
  const int b = blockIdx.x;
  float m = -INFINITY, s = 0.f, best = -INFINITY;
  int bidx = 0x7fffffff;
  bool nan = false;
  for (int i = threadIdx.x; i < n_parts; i += blockDim.x) {
    const SelectPartial p = partials[(int64_t)b * n_parts + i];
    lse_merge(m, s, p.m, p.s);
    if (p.best > best || (p.best == best && p.bidx < bidx)) {
      best = p.best;
      bidx = p.bidx;
    }
    nan |= p.nan > 0.f;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lse_merge(m, s, __shfl_xor(m, o, MSA_WAVE), __shfl_xor(s, o, MSA_WAVE));
    const float ob = __shfl_xor(best, o, MSA_WAVE);
    const int oi = __shfl_xor(bidx, o, MSA_WAVE);
    if (ob > best || (ob == best && oi < bidx)) {
      best = ob;
      bidx = oi;
    }
    nan |= (bool)__shfl_xor((int)nan, o, MSA_WAVE);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    wm[wave] = m;
    ws[wave] = s;
    wbest[wave] = best;
    widx[wave] = bidx;
    wnan[wave] = nan ? 1.f : 0.f;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      lse_merge(m, s, wm[w], ws[w]);
      if (wbest[w] > best || (wbest[w] == best && widx[w] < bidx)) {
        best = wbest[w];
        bidx = widx[w];
      }
      nan |= wnan[w] > 0.f;
    }
    float lp = (best - m) - logf(s);
    if (nan || !(best > -INFINITY)) {
      lp = -INFINITY;
      bidx = 0;
    }
    const int col = len_dev ? *len_dev : 0;
    tok[b * tok_stride + col] = bidx;
    score[b * score_stride + col] = lp;
    if (finished) {
      bool f = bidx == eos;
      for (int j = 0; j < stop.n; ++j) f |= (stop.id[j] == bidx);
      if (f) finished[b] = 1;
    }
  }
}

}  // namespace

int msa_launch_select_combine(const SelectPartial* partials, int n_parts, int B,
                              const IdList& stop, uint8_t* finished, int eos, int64_t* tok,
                              int64_t tok_stride, float* score, int64_t score_stride,
                              const int32_t* len_dev, hipStream_t stream) {
  hipLaunchKernelGGL(select_combine_kernel, dim3(B), dim3(256), 0, stream, partials, n_parts,
                     stop, finished, eos, tok, tok_stride, score, score_stride, len_dev);
  return 0;
}

extern "C" int msa_greedy_select_f16(const void* logits, int64_t ld_logits, int B, int V,
                                     float temperature, const int32_t* banned_host, int n_banned,
                                     const int32_t* stop_host, int n_stop, uint8_t* finished,
                                     const uint8_t* row_mode, int force_eos_all, int eos_idx,
                                     int64_t* tok,
                                     int64_t tok_stride, float* score, int64_t score_stride,
                                     const int32_t* len_dev, void* stream) {
  MSA_REQUIRE(logits && tok && score, MSA_ERR_INVALID_ARG, "msa_greedy_select_f16: null pointer");
  MSA_REQUIRE(B > 0 && V > 0 && ld_logits >= V, MSA_ERR_INVALID_ARG,
              "msa_greedy_select_f16: bad shape B=%d V=%d ld=%lld", B, V, (long long)ld_logits);
  MSA_REQUIRE(n_banned >= 0 && n_banned <= 16 && (n_banned == 0 || banned_host),
              MSA_ERR_INVALID_ARG, "msa_greedy_select_f16: n_banned=%d (0..16)", n_banned);
  MSA_REQUIRE(n_stop >= 0 && n_stop <= 16 && (n_stop == 0 || stop_host), MSA_ERR_INVALID_ARG,
              "msa_greedy_select_f16: n_stop=%d (0..16)", n_stop);
  MSA_REQUIRE(eos_idx >= 0 && eos_idx < V, MSA_ERR_INVALID_ARG,
              "msa_greedy_select_f16: eos_idx=%d outside the vocabulary", eos_idx);
  MSA_REQUIRE(temperature >= 0.f, MSA_ERR_INVALID_ARG, "msa_greedy_select_f16: temperature < 0");
  const bool scale = temperature > 0.f && temperature != 1.0f;
  IdList banned{}, stop{};
  banned.n = n_banned;
  for (int i = 0; i < n_banned; ++i) banned.id[i] = banned_host[i];
  stop.n = n_stop;
  for (int i = 0; i < n_stop; ++i) stop.id[i] = stop_host[i];
  hipLaunchKernelGGL(greedy_select_kernel, dim3(B), dim3(SM_THREADS), 0, (hipStream_t)stream,
                     (const half_t*)logits, ld_logits, V, temperature, scale, banned, stop,
                     finished, row_mode, force_eos_all, eos_idx, tok, tok_stride, score,
                     score_stride, len_dev);
  MSA_CHECK_LAUNCH("msa_greedy_select_f16");
  return MSA_OK;
}

extern "C" int msa_target_logprob_f16(const void* logits, int64_t ld_logits, int64_t rows, int V,
                                      float temperature, const int64_t* target, float* out,
                                      void* stream) {
  MSA_REQUIRE(logits && target && out, MSA_ERR_INVALID_ARG, "msa_target_logprob_f16: null pointer");
  MSA_REQUIRE(rows >= 0 && rows < (1ll << 31) && V > 0 && ld_logits >= V, MSA_ERR_INVALID_ARG,
              "msa_target_logprob_f16: bad shape rows=%lld V=%d ld=%lld", (long long)rows, V,
              (long long)ld_logits);
  if (rows == 0) return MSA_OK;
  const bool scale = temperature > 0.f && temperature != 1.0f;
  hipLaunchKernelGGL(target_logprob_kernel, dim3((unsigned)rows), dim3(SM_THREADS), 0,
                     (hipStream_t)stream, (const half_t*)logits, ld_logits, V, temperature, scale,
                     target, out);
  MSA_CHECK_LAUNCH("msa_target_logprob_f16");
  return MSA_OK;
}
