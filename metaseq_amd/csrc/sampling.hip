// Per-row vocabulary reductions of the greedy generation loop: fp32 log-sum-exp over fp16
// logits, masked arg-max with lowest-index tie-break, and target log-probability gather.
// One workgroup per logits row; the row (V * 2 bytes) is read twice from cache/HBM.
#include <atomic>
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


// fp32 log-softmax of fp16 logits rows; row (o, i) is read at o * in_outer + i * ld and written
// at o * out_outer + i * ld_out
__global__ __launch_bounds__(SM_THREADS) void log_softmax_kernel(
    const half_t* __restrict__ logits, int64_t in_outer, int64_t ld, int n_inner, int V,
    float temperature, bool scale, float* __restrict__ out, int64_t out_outer, int64_t ld_out) {
  __shared__ float red[16];
  const int o = blockIdx.x / n_inner, i = blockIdx.x % n_inner;
  const half_t* row = logits + o * in_outer + i * ld;
  float* orow = out + o * out_outer + i * ld_out;
  const RowStats st = row_logsumexp(row, V, temperature, scale, red);
  for_each_z(row, V, temperature, scale, [&](int id, float z) { orow[id] = (z - st.max) - st.lse; });
}

// ---- nucleus (top-p) sampling --------------------------------------------------------------
// One workgroup per row.  The nucleus boundary is found without sorting, by a radix descent over
// the bit pattern of the probabilities (positive floats order like their bit patterns): four
// passes over the row, each adding the mass of the ids that match the bits decided so far into
// a 256-bucket histogram.  Masses are accumulated as 2^-48 fixed-point integers, so the sums
// are exact and do not depend on the order of the additions (run-to-run deterministic although
// the buckets are filled with LDS atomics).  Ties at the boundary are cut by id.  Nothing of the
// row is kept between passes: a pass re-reads the fp16 logits (L2) and recomputes p.
// The draw is an exponential race: arg-max of p / noise over the nucleus, noise ~ Exp(1) per id,
// which picks id v with probability p[v] / mass(nucleus).
constexpr int SP_THREADS = 1024;
constexpr int SP_CACHE_IDS = 40000;  // ids whose values stay in LDS between the passes
constexpr int SP_TIE_BLOCKS = 64;  // rounds of SP_THREADS ids the one-pass tie search covers
constexpr float SP_FIXED = 281474976710656.f;  // 2^48

struct Penalties {
  int64_t* counts;            // [B, V] generated-token counts (updated) or NULL
  const int64_t* counts_src;  // [B, V] prompt-token counts or NULL
  float presence, frequency, presence_src, frequency_src;
  const float* rows;  // [B, 4] per-row presence, frequency, presence_src, frequency_src, or NULL
};

// Adds `mass` to hist[bucket] for the active lanes of a wave: the wave first sums the masses of
// the lanes that name the same bucket (up to four buckets, lowest lane first), so that one LDS
// atomic per bucket remains; what four buckets do not cover is added per lane.
__device__ __forceinline__ void hist_add_wave(unsigned long long* hist, bool active,
                                              unsigned bucket, unsigned long long mass) {
  const int lane = threadIdx.x & 63;
  unsigned long long todo = __ballot(active);
  for (int trip = 0; todo != 0 && trip < 4; ++trip) {
    const int leader = __builtin_ctzll(todo);
    const unsigned lb = (unsigned)__shfl((int)bucket, leader, MSA_WAVE);
    const bool mine = active && bucket == lb;
    unsigned long long m = mine ? mass : 0ull;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m += __shfl_xor(m, o, MSA_WAVE);
    if (lane == leader) atomicAdd(&hist[lb], m);
    active = active && !mine;
    todo = __ballot(active);
  }
  if (active) atomicAdd(&hist[bucket], mass);
}

__device__ __forceinline__ void argbest(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

__global__ __launch_bounds__(SP_THREADS) void sample_topp_kernel(
    const half_t* __restrict__ logits, int64_t ld, int V, float temperature_all,
    const float* __restrict__ temperature_rows, IdList banned, IdList stop,
    uint8_t* __restrict__ finished, const uint8_t* __restrict__ row_mode, int force_eos_all,
    int eos, const float* __restrict__ topp_rows, float topp_all,
    const float* __restrict__ noise, Penalties pen, float* __restrict__ lprobs_out,
    int64_t ld_lprobs, int64_t* __restrict__ tok, int64_t tok_stride,
    float* __restrict__ score, int64_t score_stride, int cap) {
  // e(id) of the first `cap` ids, kept from the first pass for the six that follow (dynamic
  // LDS, 4 * cap bytes): an LDS read in place of the load, the exact division by the
  // temperature, the masks and the penalties.  Every pass walks the ids in the same
  // thread-to-id mapping, so a thread only ever reads back what it wrote itself.
  extern __shared__ __attribute__((aligned(16))) float e_cache[];
  if (pen.rows) {  // this row's own penalty weights (rows of a batch from different requests)
    const float* w = pen.rows + 4 * (int64_t)blockIdx.x;
    pen.presence = w[0], pen.frequency = w[1], pen.presence_src = w[2], pen.frequency_src = w[3];
  }
  __shared__ float red[16];
  __shared__ float rbest[16], rprob[16];
  __shared__ int ridx[16];
  __shared__ unsigned long long hist[256];
  __shared__ unsigned sh_bucket;
  __shared__ unsigned long long sh_above;
  __shared__ unsigned long long wsum[4];
  __shared__ int sh_found, sh_limit;
  __shared__ unsigned tcnt[SP_TIE_BLOCKS];
  __shared__ unsigned long long tmask[SP_THREADS / 64];
  const int b = blockIdx.x;
  const half_t* row = logits + (int64_t)b * ld;
  const unsigned rm = row_mode ? row_mode[b] : 0u;
  if (rm & MSA_ROW_SKIP) return;  // the whole workgroup: this row is not part of the call
  const bool only_eos = force_eos_all || (finished && finished[b]) || (rm & MSA_ROW_ONLY_EOS);
  const bool ban_early = rm & MSA_ROW_BAN_EARLY;
  const float topp = topp_rows ? topp_rows[b] : topp_all;
  const float temperature = temperature_rows ? temperature_rows[b] : temperature_all;
  const bool scale = temperature > 0.f && temperature != 1.0f;

  // e(id) = z - penalties for an eligible id, -inf otherwise; nan_out collects NaN logits
  auto eligible = [&](int id) {
    bool ok = !(only_eos && id != eos) && !(ban_early && id == eos);
    for (int t = 0; t < banned.n; ++t) ok &= (banned.id[t] != id);
    if (ban_early)
      for (int t = 0; t < stop.n; ++t) ok &= (stop.id[t] != id);
    return ok;
  };
  auto e_of = [&](int id, bool& nan_out) {
    float z = (float)row[id];
    if (scale) z = z / temperature;
    nan_out |= (z != z);
    if (!eligible(id)) return -INFINITY;
    if (pen.counts) {
      const float cnt = (float)pen.counts[(int64_t)b * V + id];
      z -= cnt * pen.frequency + (cnt > 0.f ? pen.presence : 0.f);
    }
    if (pen.counts_src) {
      const float cnt = (float)pen.counts_src[(int64_t)b * V + id];
      z -= cnt * pen.frequency_src + (cnt > 0.f ? pen.presence_src : 0.f);
    }
    return z;
  };

  // ---- softmax statistics: over the eligible ids (after penalties), and over every id of the
  // raw z for the log-softmax that the greedy branch's score is taken from ----
  bool nan = false;
  float mx = -INFINITY, mx_all = -INFINITY;
  #pragma unroll 8
  for (int id = threadIdx.x; id < V; id += SP_THREADS) {
    const float e = e_of(id, nan);
    if (id < cap) e_cache[id] = e;
    mx = fmaxf(mx, e);
    float z = (float)row[id];
    if (scale) z = z / temperature;
    mx_all = fmaxf(mx_all, z);
  }
  auto e_at = [&](int id) {
    bool unused = false;
    return id < cap ? e_cache[id] : e_of(id, unused);
  };
  mx = block_max(mx, red);
  mx_all = block_max(mx_all, red);
  const bool dead = block_max(nan ? 1.f : 0.f, red) > 0.f || !(mx > -INFINITY);
  const bool sampling = noise != nullptr && topp > 0.f && temperature > 0.f && !dead;
  // the log-softmax over all ids of the raw values: the greedy score and the stored row
  const bool need_all = lprobs_out != nullptr || !sampling;
  float s = 0.f, s_all = 0.f;
  if (!dead) {
    #pragma unroll 8
    for (int id = threadIdx.x; id < V; id += SP_THREADS) {
      const float e = e_at(id);
      s += e > -INFINITY ? expf(e - mx) : 0.f;
      if (need_all) {
        float z = (float)row[id];
        if (scale) z = z / temperature;
        s_all += expf(z - mx_all);
      }
    }
  }
  s = block_sum(s, red);
  s_all = block_sum(s_all, red);
  const float inv = dead ? 0.f : 1.f / s;
  auto p_of = [&](int id) {
    const float e = e_at(id);
    return e > -INFINITY ? expf(e - mx) * inv : 0.f;
  };

  // ---- nucleus: ids in order of decreasing p (ties: increasing id) belong while the mass
  // before them is < topp.  T = the smallest probability whose strictly-greater mass is below
  // topp: everything above T is in, of the ids equal to T those below tie_limit.
  unsigned tbits = 0;
  int tie_limit = V;
  if (sampling) {
    const unsigned long long P =
        topp >= 1.f ? ~0ull : (unsigned long long)((double)topp * (double)SP_FIXED);
    unsigned prefix = 0;            // bits decided so far (the top 8 * level bits)
    unsigned long long above = 0;   // mass of the ids whose decided bits are greater
    for (int level = 0; level < 4; ++level) {
      const int shift = 24 - 8 * level;
      if (threadIdx.x < 256) hist[threadIdx.x] = 0;
      __syncthreads();
      // At level 0 (sign and seven exponent bits) nearly all ids fall into two or three
      // buckets: a thread first adds up its own ids' masses in a table of four buckets, a wave
      // then those of its lanes, and one LDS atomic per wave and bucket remains (1024 lanes
      // adding 64-bit masses to the same few LDS words cost more than everything else here).
      unsigned tb[4] = {~0u, ~0u, ~0u, ~0u};
      unsigned long long tm[4] = {0ull, 0ull, 0ull, 0ull};
      #pragma unroll 8
      for (int id = threadIdx.x; id < V; id += SP_THREADS) {
        const float pv = p_of(id);
        const unsigned u = __float_as_uint(pv);
        if (pv > 0.f && (level == 0 || (u >> (shift + 8)) == prefix)) {
          const unsigned bucket = (u >> shift) & 255u;
          const unsigned long long mass = (unsigned long long)(pv * SP_FIXED);
          bool done = false;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (!done && (tb[j] == bucket || tb[j] == ~0u)) {
              tb[j] = bucket;
              tm[j] += mass;
              done = true;
            }
          if (!done) atomicAdd(&hist[bucket], mass);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) hist_add_wave(hist, tb[j] != ~0u, tb[j], tm[j]);
      __syncthreads();
      // the lowest non-empty bucket that still has less than topp above it: thread j < 256
      // looks at bucket 255 - j, with the mass of the buckets above it in front of it
      if (threadIdx.x == 0) sh_found = -1;
      unsigned long long h = 0, before = 0;
      if (threadIdx.x < 256) {
        h = hist[255 - threadIdx.x];
        unsigned long long inc = h;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const unsigned long long up = __shfl_up(inc, o, MSA_WAVE);
          if ((int)(threadIdx.x & 63) >= o) inc += up;
        }
        if ((threadIdx.x & 63) == 63) wsum[threadIdx.x >> 6] = inc;
        before = inc - h;
      }
      __syncthreads();
      if (threadIdx.x < 256) {
        for (int w = 0; w < (int)(threadIdx.x >> 6); ++w) before += wsum[w];
        before += above;
        if (h != 0 && before < P) atomicMax(&sh_found, (int)threadIdx.x);
      }
      __syncthreads();
      if (threadIdx.x < 256 && (int)threadIdx.x == sh_found) {
        sh_bucket = 255u - threadIdx.x;
        sh_above = before;
      }
      if (threadIdx.x == 0 && sh_found < 0) {
        sh_bucket = 0u;
        sh_above = above;
      }
      __syncthreads();
      prefix = (prefix << 8) | sh_bucket;
      above = sh_above;
      __syncthreads();
    }
    tbits = prefix;
    const float T = __uint_as_float(tbits);
    const unsigned long long Tfx = (unsigned long long)(T * SP_FIXED);
    const unsigned long long tie_mass = hist[tbits & 255u];
    const long long n_ties = Tfx ? (long long)(tie_mass / Tfx) : 0;
    // the i-th tied id (from 0) has above + i * T before it
    long long n_in = n_ties;
    if (Tfx && P != ~0ull && above < P) n_in = min(n_ties, (long long)((P - above + Tfx - 1) / Tfx));
    if (n_in < n_ties && V <= SP_TIE_BLOCKS * SP_THREADS) {
      // The smallest id bound below which exactly n_in tied ids lie.  Ids in increasing order
      // are (round k of the loop, wave, lane) in lexicographic order: count the tied ids of
      // every round, find the round that holds the n_in-th, then its wave and lane.  (fp16
      // logits make ties at the boundary the rule, not the exception.)
      if (threadIdx.x < SP_TIE_BLOCKS) tcnt[threadIdx.x] = 0;
      __syncthreads();
      for (int id = threadIdx.x, k = 0; id - (int)threadIdx.x < V; id += SP_THREADS, ++k) {
        const bool tied = id < V && __float_as_uint(p_of(min(id, V - 1))) == tbits;
        const unsigned long long m = __ballot(tied);
        if ((threadIdx.x & 63) == 0 && m) atomicAdd(&tcnt[k], (unsigned)__popcll(m));
      }
      __syncthreads();
      if (threadIdx.x == 0) {
        long long cum = 0;
        int kk = -1;
        if (n_in > 0)
          for (int k = 0; k < SP_TIE_BLOCKS; ++k) {
            if (cum + tcnt[k] >= n_in) {
              kk = k;
              break;
            }
            cum += tcnt[k];
          }
        sh_found = kk;
        sh_above = (unsigned long long)(n_in - cum);  // which of that round's tied ids (from 1)
        sh_limit = 0;                                  // n_in == 0: no tied id is in
      }
      __syncthreads();
      const int kk = sh_found;
      if (kk >= 0) {
        const int id = kk * SP_THREADS + (int)threadIdx.x;
        const bool tied = id < V && __float_as_uint(p_of(min(id, V - 1))) == tbits;
        const unsigned long long m = __ballot(tied);
        if ((threadIdx.x & 63) == 0) tmask[threadIdx.x >> 6] = m;
        __syncthreads();
        if (threadIdx.x == 0) {
          long long need = (long long)sh_above;
          for (int w = 0; w < SP_THREADS / 64; ++w) {
            unsigned long long mw = tmask[w];
            const int c = __popcll(mw);
            if (need > c) {
              need -= c;
              continue;
            }
            for (; need > 1; --need) mw &= mw - 1;  // drop the lowest set bits
            sh_limit = kk * SP_THREADS + w * 64 + __builtin_ctzll(mw) + 1;
            break;
          }
        }
      }
      __syncthreads();
      tie_limit = sh_limit;
    } else if (n_in < n_ties) {  // larger vocabularies: bisection, a pass over the row per step
      int lo = 0, hi = V;
      while (lo < hi) {
        const int mid = lo + ((hi - lo) >> 1);
        float cnt = 0.f;
        for (int id = threadIdx.x; id < mid; id += SP_THREADS)
          cnt += __float_as_uint(p_of(id)) == tbits ? 1.f : 0.f;
        if ((long long)block_sum(cnt, red) >= n_in)
          hi = mid;
        else
          lo = mid + 1;
      }
      tie_limit = lo;
    }
  }

  // ---- the masked log-probabilities of the row, if asked for: log-softmax over all ids, the
  // ineligible ones at -inf, then the penalties (frequency, then presence) - before the counts
  // are updated below
  if (lprobs_out) {
    float* lrow = lprobs_out + (int64_t)b * ld_lprobs;
    const float log_s = dead ? 0.f : logf(s_all);
    for (int id = threadIdx.x; id < V; id += SP_THREADS) {
      float v = -INFINITY;
      if (!dead && eligible(id)) {
        float z = (float)row[id];
        if (scale) z = z / temperature;
        v = (z - mx_all) - log_s;
        if (pen.counts) {
          const float cnt = (float)pen.counts[(int64_t)b * V + id];
          v = v - cnt * pen.frequency;
          v = v - (cnt > 0.f ? pen.presence : 0.f);
        }
        if (pen.counts_src) {
          const float cnt = (float)pen.counts_src[(int64_t)b * V + id];
          v = v - cnt * pen.frequency_src;
          v = v - (cnt > 0.f ? pen.presence_src : 0.f);
        }
      }
      lrow[id] = v;
    }
  }

  // ---- the draw: exponential race over the nucleus; when not sampling, the arg-max of the
  // penalised values themselves (exp() may map two close values to one probability)
  float best = -INFINITY, bestp = 0.f;
  int bidx = 0x7fffffff;
  if (!dead) {
    #pragma unroll 8
    for (int id = threadIdx.x; id < V; id += SP_THREADS) {
      const float e = e_at(id);
      if (!(e > -INFINITY)) continue;
      const float pv = expf(e - mx) * inv;
      float key = e;
      if (sampling) {
        if (!(pv > 0.f)) continue;
        const unsigned u = __float_as_uint(pv);
        if (!(u > tbits || (u == tbits && id < tie_limit))) continue;
        key = pv / noise[(int64_t)b * V + id];
      }
      if (key > best || (key == best && id < bidx)) {
        best = key;
        bidx = id;
        bestp = pv;
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, MSA_WAVE), op = __shfl_xor(bestp, o, MSA_WAVE);
    const int oi = __shfl_xor(bidx, o, MSA_WAVE);
    if (ov > best || (ov == best && oi < bidx)) {
      best = ov;
      bidx = oi;
      bestp = op;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    rbest[threadIdx.x >> 6] = best;
    ridx[threadIdx.x >> 6] = bidx;
    rprob[threadIdx.x >> 6] = bestp;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SP_THREADS / 64; ++w)
      if (rbest[w] > best || (rbest[w] == best && ridx[w] < bidx)) {
        best = rbest[w];
        bidx = ridx[w];
        bestp = rprob[w];
      }
    // sampling: the log of the probability among the eligible ids (the reference takes it from
    // softmax(lprobs)); greedy: the penalised log-softmax value itself (lprobs.max())
    float lp = logf(bestp);
    if (!sampling && !dead && bidx != 0x7fffffff) {
      bool unused = false;
      lp = (e_of(bidx, unused) - mx_all) - logf(s_all);
    }
    if (dead || bidx == 0x7fffffff) {  // as the greedy kernel: token 0 with score -inf
      bidx = 0;
      lp = -INFINITY;
    }
    tok[b * tok_stride] = bidx;
    score[b * score_stride] = lp;
    if (pen.counts) pen.counts[(int64_t)b * V + bidx] += 1;
    if (finished) {
      bool f = bidx == eos;
      for (int j = 0; j < stop.n; ++j) f |= (stop.id[j] == bidx);
      if (f) finished[b] = 1;
    }
  }
}

// Raises sample_topp_kernel's dynamic LDS limit, once per device.
bool allow_cache_lds(int bytes) {
  static std::atomic<uint64_t> done{0};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return true;
  if (hipFuncSetAttribute((const void*)sample_topp_kernel,
                          hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  done.fetch_or(bit, std::memory_order_release);
  return true;
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

extern "C" int msa_sample_topp_f16(const void* logits, int64_t ld_logits, int B, int V,
                                   float temperature, const float* temperature_rows,
                                   const int32_t* banned_host, int n_banned,
                                   const int32_t* stop_host, int n_stop, uint8_t* finished,
                                   const uint8_t* row_mode, int force_eos_all, int eos_idx,
                                   const float* topp_rows, float topp_all, const float* noise,
                                   int64_t* counts, const int64_t* counts_src,
                                   float alpha_presence, float alpha_frequency,
                                   float alpha_presence_src, float alpha_frequency_src,
                                   const float* penalty_rows, float* lprobs_out,
                                   int64_t ld_lprobs, int64_t* tok,
                                   int64_t tok_stride, float* score, int64_t score_stride,
                                   void* stream) {
  const char* name = "msa_sample_topp_f16";
  MSA_REQUIRE(logits && tok && score, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(B > 0 && V > 0 && ld_logits >= V, MSA_ERR_INVALID_ARG,
              "%s: bad shape B=%d V=%d ld=%lld", name, B, V, (long long)ld_logits);
  MSA_REQUIRE(!lprobs_out || ld_lprobs >= V, MSA_ERR_INVALID_ARG,
              "%s: log-probability rows of stride %lld < V=%d", name, (long long)ld_lprobs, V);
  MSA_REQUIRE(n_banned >= 0 && n_banned <= 16 && (n_banned == 0 || banned_host),
              MSA_ERR_INVALID_ARG, "%s: n_banned=%d (0..16)", name, n_banned);
  MSA_REQUIRE(n_stop >= 0 && n_stop <= 16 && (n_stop == 0 || stop_host), MSA_ERR_INVALID_ARG,
              "%s: n_stop=%d (0..16)", name, n_stop);
  MSA_REQUIRE(eos_idx >= 0 && eos_idx < V, MSA_ERR_INVALID_ARG,
              "%s: eos_idx=%d outside the vocabulary", name, eos_idx);
  MSA_REQUIRE(temperature >= 0.f, MSA_ERR_INVALID_ARG, "%s: temperature < 0", name);
  IdList banned{}, stop{};
  banned.n = n_banned;
  for (int i = 0; i < n_banned; ++i) banned.id[i] = banned_host[i];
  stop.n = n_stop;
  for (int i = 0; i < n_stop; ++i) stop.id[i] = stop_host[i];
  Penalties pen{};
  pen.counts = counts;
  pen.counts_src = counts_src;
  pen.presence = alpha_presence;
  pen.frequency = alpha_frequency;
  pen.presence_src = alpha_presence_src;
  pen.frequency_src = alpha_frequency_src;
  pen.rows = penalty_rows;
  // as many ids' values as the CU's LDS holds beside the kernel's own 3 KB stay in LDS
  // between the passes (none if the limit cannot be raised)
  int cap = min(V, SP_CACHE_IDS);
  if (cap * 4 > 48 * 1024 && !allow_cache_lds(SP_CACHE_IDS * 4)) cap = 48 * 1024 / 4;
  hipLaunchKernelGGL(sample_topp_kernel, dim3(B), dim3(SP_THREADS), (size_t)cap * 4,
                     (hipStream_t)stream, (const half_t*)logits, ld_logits, V, temperature,
                     temperature_rows, banned, stop, finished, row_mode, force_eos_all, eos_idx,
                     topp_rows, topp_all, noise, pen, lprobs_out, ld_lprobs, tok, tok_stride,
                     score, score_stride, cap);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

extern "C" int msa_log_softmax_f16(const void* logits, int64_t in_outer_stride, int64_t ld_logits,
                                   int n_outer, int n_inner, int V, float temperature,
                                   float* out, int64_t out_outer_stride, int64_t ld_out,
                                   void* stream) {
  const char* name = "msa_log_softmax_f16";
  MSA_REQUIRE(logits && out, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(n_outer >= 0 && n_inner >= 0 && V > 0 && ld_logits >= V && ld_out >= V &&
                  (int64_t)n_outer * n_inner < (1ll << 31),
              MSA_ERR_INVALID_ARG, "%s: bad shape %d x %d rows of V=%d", name, n_outer, n_inner,
              V);
  MSA_REQUIRE(temperature >= 0.f, MSA_ERR_INVALID_ARG, "%s: temperature < 0", name);
  if (n_outer == 0 || n_inner == 0) return MSA_OK;
  const bool scale = temperature > 0.f && temperature != 1.0f;
  hipLaunchKernelGGL(log_softmax_kernel, dim3((unsigned)(n_outer * n_inner)), dim3(SM_THREADS), 0,
                     (hipStream_t)stream, (const half_t*)logits, in_outer_stride, ld_logits,
                     n_inner, V, temperature, scale, out, out_outer_stride, ld_out);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}
