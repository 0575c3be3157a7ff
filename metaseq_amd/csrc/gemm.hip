// y[M,N] = epilogue(x[M,K] . W[N,K]^T) on fp16 MFMA with fp32 accumulation.
//
// Weights live in HBM in a tile-packed layout (see pack kernels below): the 16 x 32 block of
// W that one v_mfma_f32_16x16x32_f16 consumes as its A operand is one contiguous KB, stored in
// the order the 64 lanes read it, and the blocks of one 16-row tile follow each other along K.
// A wave instruction therefore reads one whole KB and a tile's K sweep is one linear stream.
//
// Five kernels:
//   * stream (M <= 32 packed rows, the decode step; also the fused vocabulary projection +
//     selection up to 64 rows): HBM-bound.  A workgroup of 8 waves owns a contiguous range of
//     16-row tiles (and, with split-K, one K range); it walks the tiles 3 or 4 at a time, the
//     waves taking interleaved K steps.  Activations come in the matching packed fragment
//     layout from L2 and every activation fragment is reused for the tiles of the group.
//     Fragments are double buffered several steps deep and the prefetch runs across tile-group
//     boundaries, so the memory pipe never drains while a finished group is reduced across
//     the waves through LDS (fixed order: results are run-to-run deterministic).
//   * shared-activation stream (33 .. 64 packed rows): the same weight streaming, with the
//     activation fragments staged once per workgroup in LDS and shared by four waves.
//   * large tiled, fp16 weights (prefill-sized M): 256 x 256 per workgroup of four waves of
//     128 x 128 with their accumulators in the AGPR bank, both operands global -> LDS directly.
//   * large tiled, int8 weights: 256 x 256 x 64 per workgroup of eight waves, weights straight
//     from the packed layout into registers (dequantised there), activations through LDS.
//   * tiled (shapes in between): 128 x 128 x 32 LDS double-buffered tiles, 4 waves of 64 x 64,
//     v_mfma_f32_32x32x16_f16.
// All share one epilogue that reproduces the reference's fp16 rounding points, and a QKV mode
// that scatters K/V into the per-layer cache and scales Q.
#include <math.h>

#include <atomic>
#include <type_traits>
#include <utility>
#include <mutex>

#include "common.h"

namespace {

enum { MODE_PLAIN = 0, MODE_QKV = 1, MODE_SELECT = 2 };

struct Epilogue {
  const half_t* bias;
  const half_t* residual;
  half_t* y;
  int N;
  unsigned flags;
  int out_mb;  // > 0: y is written in the packed activation layout with this many 16-row blocks
  // MODE_QKV
  half_t* q_out;
  half_t* Kc;
  half_t* Vc;
  int T, H, hd, S0, S_cap;
  int hd_shift;  // log2(hd) if hd is a power of two, else -1
  const int32_t* len_dev;  // if set (T == 1): per-row append positions on the device (< 0: skip)
  float qscale;
  // MODE_SELECT: greedy selection over the output row instead of (or besides) storing it
  SelectPartial* partials;  // [M][gridDim.x]
  const uint8_t* finished;  // rows that may only emit eos
  const uint8_t* row_mode;  // optional per-row MSA_ROW_* bits
  IdList banned;
  IdList early;  // eos and the stop ids: not eligible for rows with MSA_ROW_BAN_EARLY
  float temperature;  // logits are divided by it when `scale`
  int scale, force_eos_all, eos;
};

// running selection state of one thread for one activation row (see SelectPartial)
struct SelectState {
  float m = -INFINITY, s = 0.f, best = -INFINITY;
  int bidx = 0x7fffffff;
  bool nan = false;
};

// 4 consecutive vocabulary ids n..n+3 of row m: the logit is round(acc), as the stored tensor
// would hold it; log-softmax is monotone, so the arg-max of the masked log-probs is the
// arg-max of the masked logits (lowest id on ties).
__device__ __forceinline__ void select_update4(SelectState& st, const Epilogue& e, int64_t m,
                                               int n, float4_t acc) {
  float z[4], cm = -INFINITY;
  const unsigned rm = e.row_mode ? e.row_mode[m] : 0u;
  const bool only_eos =
      e.force_eos_all || (e.finished && e.finished[m]) || (rm & MSA_ROW_ONLY_EOS);
  const int n_early = (rm & MSA_ROW_BAN_EARLY) ? e.early.n : 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    z[i] = round_h(acc[i]);
    if (e.scale) z[i] = z[i] / e.temperature;
    st.nan |= (z[i] != z[i]);
    cm = fmaxf(cm, z[i]);
    const int id = n + i;
    bool ok = !(only_eos && id != e.eos);
    for (int j = 0; j < e.banned.n; ++j) ok &= (e.banned.id[j] != id);
    for (int j = 0; j < n_early; ++j) ok &= (e.early.id[j] != id);
    const float cand = ok ? z[i] : -INFINITY;
    if (cand > st.best || (cand == st.best && id < st.bidx)) {
      st.best = cand;
      st.bidx = id;
    }
  }
  if (cm > st.m) {
    st.s *= __expf(st.m - cm);
    st.m = cm;
  }
  if (st.m > -INFINITY) {
#pragma unroll
    for (int i = 0; i < 4; ++i) st.s += __expf(z[i] - st.m);
  }
  if (e.y) {
    half4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (half_t)acc[i];
    *reinterpret_cast<half4_t*>(e.y + m * e.N + n) = o;
  }
}

__device__ __forceinline__ void select_merge(SelectState& a, float om, float os, float ob, int oi,
                                             bool onan) {
  lse_merge(a.m, a.s, om, os);
  if (ob > a.best || (ob == a.best && oi < a.bidx)) {
    a.best = ob;
    a.bidx = oi;
  }
  a.nan |= onan;
}

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
    if (e.out_mb > 0)
      *reinterpret_cast<half4_t*>(e.y + packed_act_offset((int)m, n, e.out_mb)) = o;
    else
      *reinterpret_cast<half4_t*>(e.y + m * e.N + n) = o;
  } else {
    // index arithmetic in 32 bits, without 64-bit division: the row count is below 2^31, the
    // thirds are found by comparison, and a power-of-two head size (the usual case) is a shift
    const int D = e.H * e.hd;
    const int part = (n >= D) + (n >= 2 * D), c = n - part * D;  // 0 = K, 1 = V, 2 = Q
    half4_t o;
    if (part == 2) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)(t[i] * e.qscale);
      *reinterpret_cast<half4_t*>(e.q_out + m * D + c) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (half_t)t[i];
      const int h = e.hd_shift >= 0 ? c >> e.hd_shift : c / e.hd, d = c - h * e.hd;
      const int mi = (int)m;
      const int b = e.T == 1 ? mi : mi / e.T, tt = mi - b * e.T;
      const int s0 = e.len_dev ? e.len_dev[b] : e.S0;  // per-row lengths: T == 1, b = row
      if (s0 >= 0 && s0 + tt < e.S_cap) {
        half_t* dst = (part == 0 ? e.Kc : e.Vc) +
                      (((int64_t)b * e.H + h) * e.S_cap + s0 + tt) * e.hd + d;
        *reinterpret_cast<half4_t*>(dst) = o;
      }
    }
  }
}

__device__ __forceinline__ half8_t zero8() { return half8_t{0, 0, 0, 0, 0, 0, 0, 0}; }

// 8 packed int8 weights (two dwords) times an fp16 per-row scale -> 8 fp16, each round(q * scale).
// The packed layout stores every byte biased to unsigned (u = q + 128, done once by the pack
// kernel).  u is dropped into the mantissa of fp16 1024.0 (0x6400 | u is exactly 1024 + u) and
// 1152 is subtracted: q exactly, in packed fp16 arithmetic.  The packed multiply then rounds
// the exact product q * scale once, as the fp32 route would.
__device__ __forceinline__ half8_t dequant8(uint32_t lo, uint32_t hi, half_t scale) {
  const half2_t bias = {(half_t)1152.0f, (half_t)1152.0f};
  const half2_t sc = {scale, scale};
  half8_t r;
  const uint32_t w[2] = {lo, hi};
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t p0 = __builtin_amdgcn_perm(0x64646464u, w[j], 0x04010400u);  // bytes 0, 1
    const uint32_t p1 = __builtin_amdgcn_perm(0x64646464u, w[j], 0x04030402u);  // bytes 2, 3
    const half2_t h0 = (__builtin_bit_cast(half2_t, p0) - bias) * sc;
    const half2_t h1 = (__builtin_bit_cast(half2_t, p1) - bias) * sc;
    r[4 * j + 0] = h0[0];
    r[4 * j + 1] = h0[1];
    r[4 * j + 2] = h1[0];
    r[4 * j + 3] = h1[1];
  }
  return r;
}

// ---- weight packing ---------------------------------------------------------------------
// fp16: block (tile t = n/16, step ks = k/32) at halves ((t * K/32 + ks) * 512); inside the block
// lane l = 16*((k%32)/8) + n%16 owns halves l*8 .. l*8+7 = W[n][8*(k/8) .. +7].
// int8: block (t, ks8 = k/64) at bytes ((t * K/64 + ks8) * 1024); lane l = 16*g + r owns 16 bytes:
// bytes 0..7 = W[16t+r][64*ks8 + 8g .. +7] and bytes 8..15 = W[16t+r][64*ks8 + 32 + 8g .. +7],
// i.e. the A fragments of the two 32-wide steps the block covers; every byte is stored as
// q + 128.
__global__ __launch_bounds__(256) void pack_f16_kernel(const half_t* __restrict__ src,
                                                       half_t* __restrict__ dst, int N, int K,
                                                       bool unpack) {
  const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece
  const int nks = K >> 5;
  if (piece >= (int64_t)N * K / 8) return;
  const int lane = (int)(piece & 63);
  const int64_t blk = piece >> 6;
  const int ks = (int)(blk % nks), t = (int)(blk / nks);
  const int64_t rm = ((int64_t)t * 16 + (lane & 15)) * K + ks * 32 + (lane >> 4) * 8;
  if (unpack)
    *reinterpret_cast<half8_t*>(dst + rm) = *reinterpret_cast<const half8_t*>(src + piece * 8);
  else
    *reinterpret_cast<half8_t*>(dst + piece * 8) = *reinterpret_cast<const half8_t*>(src + rm);
}

__global__ __launch_bounds__(256) void pack_i8_kernel(const int8_t* __restrict__ src,
                                                      int8_t* __restrict__ dst, int N, int K,
                                                      bool unpack) {
  const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 8-byte piece
  const int nks8 = K >> 6;
  if (piece >= (int64_t)N * K / 8) return;
  const int half = (int)(piece & 1), lane = (int)((piece >> 1) & 63);
  const int64_t blk = piece >> 7;
  const int ks8 = (int)(blk % nks8), t = (int)(blk / nks8);
  const int64_t rm = ((int64_t)t * 16 + (lane & 15)) * K + ks8 * 64 + half * 32 + (lane >> 4) * 8;
  // packed bytes are q + 128 (the sign bit flipped): the kernels expand them without a
  // sign fix-up
  uint2 v = *reinterpret_cast<const uint2*>(unpack ? src + piece * 8 : src + rm);
  v.x ^= 0x80808080u;
  v.y ^= 0x80808080u;
  *reinterpret_cast<uint2*>(unpack ? dst + rm : dst + piece * 8) = v;
}

// packed int8 -> packed fp16, each element round(q * scale): int8 block (t, ks8) becomes the fp16
// blocks (t, 2 ks8) and (t, 2 ks8 + 1), and a lane's bytes 0..7 / 8..15 become its 8 halves in
// the first / second of them (the lane index is the same in both layouts).  One thread per lane
// and int8 block.
__global__ __launch_bounds__(256) void expand_w8_kernel(const uint8_t* __restrict__ Wq,
                                                        const half_t* __restrict__ scales,
                                                        half_t* __restrict__ dst, int N, int K) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= (int64_t)N * K / 16) return;
  const int lane = (int)(id & 63);
  const int64_t blk = id >> 6;
  const int nks8 = K >> 6;
  const int t = (int)(blk / nks8);
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(Wq) + id);
  const half_t sc = scales[t * 16 + (lane & 15)];
  half8_t* out = reinterpret_cast<half8_t*>(dst) + (blk * 2) * 64 + lane;
  out[0] = dequant8(v[0], v[1], sc);
  out[64] = dequant8(v[2], v[3], sc);
}

// ---- stream kernel (M <= 64) --------------------------------------------------------------
// MFMA fragments: lane l supplies 8 consecutive K elements (offset 8*(l>>4)) of row (l&15) of
// its operand; A rows are output features n, B rows are activation rows m.  The accumulator
// of lane l holds m = l&15 and n = 4*(l>>4) .. +3.
constexpr int ST_KG = 8;  // waves per workgroup = interleaved K lanes
constexpr int ST_NT = 4;  // weight tiles sharing one activation fragment (<= 32 rows)
constexpr int ST_RN = 4;  // tiles reduced across the waves per pass through LDS

// XR: the activations are row-major ([rows, K], fragments gathered 16 bytes per lane) instead
// of packed; the kernel then handles rows m_off .. m_off + M - 1 of a taller matrix (the ragged
// bottom of a prefill-sized product) and the epilogue sees the global row numbers.
// With more than 32 activation rows the activation fragments (re-read from L2 once per tile
// group) outweigh the weights in cache-fill traffic, so the fp16 kernel lets twice as many
// tiles share each fragment and buffers fewer K steps to stay inside the register file (the
// int8 kernel, whose stage also holds the raw bytes of two K steps, would spill).
template <int MB, bool W8, int MODE, bool XR = false, int KG = ST_KG,
          int NT = (MB <= 2 || W8 ? ST_NT : 2 * ST_NT), int U = (MB <= 2 ? 4 : (NT > ST_NT ? 1 : 2))>
__global__ __launch_bounds__(KG * 64) void linear_stream_kernel(
    const half_t* __restrict__ xp, const void* __restrict__ Wp, const half_t* __restrict__ scales,
    float* __restrict__ part, int M, int N, int K, int tiles_per_wg, int ks_per_split,
    Epilogue epi, int64_t m_off) {
  // U = K steps (32 wide) buffered per stage; an int8 block covers two steps
  constexpr int UA = W8 ? U / 2 : U;  // weight loads per stage and tile
  constexpr int RN = NT < ST_RN ? NT : ST_RN;  // NT is a multiple of RN
  __shared__ float4_t red[KG][RN * MB][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ntiles = N >> 4;
  const int nks = K >> 5;  // 32-wide steps in a row
  const int tile_begin = blockIdx.x * tiles_per_wg;
  const int tile_end = min(ntiles, tile_begin + tiles_per_wg);
  const int ks_begin = blockIdx.y * ks_per_split;
  const int ks_end = min(nks, ks_begin + ks_per_split);
  if (tile_begin >= tile_end || ks_begin >= ks_end) return;
  const int ngroups = (tile_end - tile_begin + NT - 1) / NT;
  const int nstages = (ks_end - ks_begin + KG * U - 1) / (KG * U);
  const int total = ngroups * nstages;

  struct Stage {
    half8_t a[UA][NT];  // fp16: one A fragment; int8: 16 raw bytes = two A fragments
    half8_t b[U][MB];
  };
  Stage s0, s1;
  // Loads are unconditional so that the hardware counters can keep two stages in flight (a
  // load inside a branch makes the compiler wait for every outstanding load before the MFMAs).
  // Steps and tiles past the end read a clamped, valid address: a surplus tile is dropped in
  // finish(), a surplus step gets its activation fragment zeroed in mma().
  auto load = [&](Stage& s, int idx) {
    const int grp = idx / nstages, st = idx - grp * nstages;
    const int t0 = tile_begin + grp * NT;
#pragma unroll
    for (int u = 0; u < UA; ++u) {
      // first 32-wide step covered by this load (wave-uniform)
      const int ks = W8 ? ks_begin + 2 * (wave + KG * (st * UA + u))
                        : ks_begin + wave + KG * (st * U + u);
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int t = min(t0 + j, tile_end - 1);
        const int ksc = min(ks, ks_end - (W8 ? 2 : 1));
        const int64_t blk = W8 ? (int64_t)t * (nks >> 1) + (ksc >> 1) : (int64_t)t * nks + ksc;
        s.a[u][j] = __builtin_nontemporal_load(
            reinterpret_cast<const half8_t*>((const half_t*)Wp + blk * 512 + lane * 8));
      }
#pragma unroll
      for (int h = 0; h < (W8 ? 2 : 1); ++h) {
        const int kk = min(ks + h, ks_end - 1);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          if (XR) {
            const int64_t m = m_off + min(mb * 16 + (lane & 15), M - 1);
            s.b[W8 ? 2 * u + h : u][mb] = *reinterpret_cast<const half8_t*>(
                xp + m * K + kk * 32 + (lane >> 4) * 8);
          } else {
            s.b[W8 ? 2 * u + h : u][mb] = *reinterpret_cast<const half8_t*>(
                xp + (((int64_t)kk * MB + mb) * 64 + lane) * 8);
          }
        }
      }
    }
  };
  // slot e = threadIdx.x + it * KG * 64 of a reduction pass of finish(); it always maps to the
  // same activation row, whatever the pass (MODE_SELECT keeps one running state per slot)
  constexpr int SEL_IT = (RN * MB * 64 + KG * 64 - 1) / (KG * 64);
  SelectState sel[MODE == MODE_SELECT ? SEL_IT : 1];
  float4_t acc[NT][MB];
  auto clear = [&]() {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[j][mb] = float4_t{0.f, 0.f, 0.f, 0.f};
  };
  auto mma = [&](Stage& s, int idx) {
    const int grp = idx / nstages, st = idx - grp * nstages;
    half_t sc[NT];
    if (W8) {
      const int t0 = tile_begin + grp * NT;
#pragma unroll
      for (int j = 0; j < NT; ++j)
        sc[j] = scales[min(t0 + j, tile_end - 1) * 16 + (lane & 15)];
    }
    // zero the activation fragments of steps past the end of this K range
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ks = W8 ? ks_begin + 2 * (wave + KG * (st * UA + u / 2)) + (u & 1)
                        : ks_begin + wave + KG * (st * U + u);
      if (ks >= ks_end) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) s.b[u][mb] = zero8();
      }
    }
    const int tiles_left = tile_end - (tile_begin + grp * NT);  // real tiles in this group
#pragma unroll
    for (int u = 0; u < UA; ++u)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if (NT > ST_NT && j >= tiles_left) continue;  // wave-uniform: no MFMAs for surplus tiles
        if (!W8) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(s.a[u][j], s.b[u][mb], acc[j][mb],
                                                                0, 0, 0);
        } else {
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          const u4 raw = __builtin_bit_cast(u4, s.a[u][j]);
          const half8_t f0 = dequant8(raw[0], raw[1], sc[j]);
          const half8_t f1 = dequant8(raw[2], raw[3], sc[j]);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            acc[j][mb] =
                __builtin_amdgcn_mfma_f32_16x16x32_f16(f0, s.b[2 * u][mb], acc[j][mb], 0, 0, 0);
            acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f1, s.b[2 * u + 1][mb],
                                                                acc[j][mb], 0, 0, 0);
          }
        }
      }
  };
  auto finish = [&](int idx) {  // after the last stage of a tile group
    const int grp = idx / nstages;
    const int t0 = tile_begin + grp * NT;
#pragma unroll
    for (int p = 0; p < NT / RN; ++p) {  // RN tiles per pass through the LDS buffer
#pragma unroll
      for (int jj = 0; jj < RN; ++jj)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[wave][jj * MB + mb][lane] = acc[p * RN + jj][mb];
      __syncthreads();
#pragma unroll
      for (int it = 0; it < SEL_IT; ++it) {
        const int e = threadIdx.x + it * KG * 64;
        if (e >= RN * MB * 64) break;
        const int jm = e >> 6, l = e & 63;
        const int jj = jm / MB, mb = jm - jj * MB;
        const int j = p * RN + jj;
        float4_t sum = red[0][jm][l];
#pragma unroll
        for (int w = 1; w < KG; ++w) sum += red[w][jm][l];
        const int m = mb * 16 + (l & 15);
        const int n = (t0 + j) * 16 + ((l >> 4) << 2);
        if (m < M && t0 + j < tile_end) {
          if (part)
            *reinterpret_cast<float4_t*>(part + ((int64_t)blockIdx.y * M + m) * N + n) = sum;
          else if (MODE == MODE_SELECT)
            select_update4(sel[it], epi, m, n, sum);
          else
            epilogue4<MODE == MODE_SELECT ? MODE_PLAIN : MODE>(epi, m_off + m, n, sum);
        }
      }
      __syncthreads();
    }
    clear();
  };
  clear();
  load(s0, 0);
  int idx = 0;
  for (; idx + 2 < total; idx += 2) {  // steady state: every load is of a real stage
    load(s1, idx + 1);
    mma(s0, idx);
    if ((idx + 1) % nstages == 0) finish(idx);
    load(s0, idx + 2);
    mma(s1, idx + 1);
    if ((idx + 2) % nstages == 0) finish(idx + 1);
  }
  if (idx + 1 < total) {  // two stages left
    load(s1, idx + 1);
    mma(s0, idx);
    if ((idx + 1) % nstages == 0) finish(idx);
    mma(s1, idx + 1);
    finish(idx + 1);
  } else {  // one stage left
    mma(s0, idx);
    finish(idx);
  }
  if (MODE == MODE_SELECT) {
    // The 16 threads that hold one row (4 lane groups x RN tile slots of one row block) merge
    // their states: lanes through shuffles, tile slots through LDS; one partial per row and
    // workgroup goes to memory for the combine kernel.
    SelectPartial* sp = reinterpret_cast<SelectPartial*>(&red[0][0][0]);  // [RN * MB * 16]
#pragma unroll
    for (int it = 0; it < SEL_IT; ++it) {
      const int e = threadIdx.x + it * KG * 64;
      SelectState st = sel[it];
#pragma unroll
      for (int o = 16; o <= 32; o <<= 1)
        select_merge(st, __shfl_xor(st.m, o, MSA_WAVE), __shfl_xor(st.s, o, MSA_WAVE),
                     __shfl_xor(st.best, o, MSA_WAVE), __shfl_xor(st.bidx, o, MSA_WAVE),
                     (bool)__shfl_xor((int)st.nan, o, MSA_WAVE));
      if (e < RN * MB * 64 && (e & 63) < 16) {
        SelectPartial p;
        p.m = st.m, p.s = st.s, p.best = st.best, p.bidx = st.bidx, p.nan = st.nan ? 1.f : 0.f;
        sp[(e >> 6) * 16 + (e & 15)] = p;  // [jm][row in block]
      }
    }
    __syncthreads();
    if (threadIdx.x < MB * 16) {
      const int mb = threadIdx.x >> 4, r = threadIdx.x & 15;
      SelectState st;
      for (int j = 0; j < RN; ++j) {  // jm = j * MB + mb
        const SelectPartial p = sp[(j * MB + mb) * 16 + r];
        select_merge(st, p.m, p.s, p.best, p.bidx, p.nan > 0.f);
      }
      const int m = mb * 16 + r;
      if (m < M) {
        SelectPartial p;
        p.m = st.m, p.s = st.s, p.best = st.best, p.bidx = st.bidx, p.nan = st.nan ? 1.f : 0.f;
        p.pad[0] = p.pad[1] = p.pad[2] = 0.f;
        epi.partials[(int64_t)m * gridDim.x + blockIdx.x] = p;
      }
    }
  }
}

// ---- shared-activation stream kernel (33 .. 64 rows) ------------------------------------------
// With more than 32 activation rows a wave that loads its own activation fragments moves more
// bytes of activations (from L2) than of weights (from HBM) through the L1, and the L1 fill rate
// becomes the limit.  Here the 8 waves form KL K lanes x NG tile lanes: the NG waves of a K lane
// work on different weight tiles over the same K steps and read their activation fragments from
// LDS, which the whole workgroup fills once per stage (SK = KL * U consecutive K steps, one
// contiguous piece of the packed activations).  Weights still go from HBM straight to registers.
// A tile group is NG * NT tiles, dealt round robin to the tile lanes; one barrier per stage;
// activations are fetched two stages ahead and parked in LDS one stage ahead, weights (and int8
// scales) one stage ahead.  The K lanes are summed through LDS in fixed order.
// KL K lanes x NG tile lanes of one wave each (8 waves as 2 x 4, or 12 waves as 4 x 3 for
// workgroups whose tile count is a multiple of 3: nine tiles fill 4 x 3 slots only to three
// quarters, but 3 x 3 exactly).
template <int MB, bool W8, int KL, int NG, int NT, int U>
struct ShareCfg {
  static constexpr int THREADS = KL * NG * 64;
  static constexpr int SK = KL * U, UA = W8 ? U / 2 : U;
  static constexpr int XH = SK * MB * 512;  // halves of activations per stage
  static constexpr int PIECES = XH / 8;     // 16-byte pieces per stage
  static constexpr int XP = (PIECES + THREADS - 1) / THREADS;  // pieces per thread and stage
  // activations double buffered, then one tile slot's partial sums of the other K lanes; where
  // both do not fit the 160 KB of a compute unit the partial sums take the place of the stage
  // that has just been consumed
  static constexpr int RED_BYTES = (KL - 1) * NG * MB * 1024;
  static constexpr bool RED_ALIAS = 2 * XH * 2 + RED_BYTES > 160 * 1024;
  static constexpr int LDS_BYTES = 2 * XH * 2 + (RED_ALIAS ? 0 : RED_BYTES);
  static_assert(U % 2 == 0, "a stage holds whole int8 blocks");
  static_assert(!RED_ALIAS || RED_BYTES <= XH * 2, "the partial sums must fit one stage");
};

template <int MB, bool W8, int MODE, int KL, int NG, int NT, int U, int PF>
__global__ __launch_bounds__(KL * NG * 64) void linear_share_kernel(
    const half_t* __restrict__ xp, const void* __restrict__ Wp, const half_t* __restrict__ scales,
    float* __restrict__ part, int M, int N, int K, int tiles_per_wg, int ks_per_split,
    Epilogue epi) {
  static_assert(MODE != MODE_SELECT, "selection runs in the plain stream kernel");
  using C = ShareCfg<MB, W8, KL, NG, NT, U>;
  constexpr int SK = C::SK, UA = C::UA, XH = C::XH, XP = C::XP, THREADS = C::THREADS;
  constexpr int PIECES = C::PIECES;
  extern __shared__ __attribute__((aligned(16))) half_t lx_share[];  // [2][XH], then red
  float4_t* red_own = reinterpret_cast<float4_t*>(lx_share + 2 * XH);  // [KL-1][NG][MB][64]
  const int lane = threadIdx.x & 63;
  // the wave number as a scalar: everything derived from it stays out of the vector registers
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kl = wave / NG, ng = wave - kl * NG;
  const uint32_t lane_off = (uint32_t)lane * 16u;  // the lane's 16 bytes of a 1 KB fragment
  const int ntiles = N >> 4, nks = K >> 5;
  const int tile_begin = blockIdx.x * tiles_per_wg;
  const int tile_end = min(ntiles, tile_begin + tiles_per_wg);
  const int ks_begin = blockIdx.y * ks_per_split;
  const int ks_end = min(nks, ks_begin + ks_per_split);
  if (tile_begin >= tile_end || ks_begin >= ks_end) return;
  const int ngroups = (tile_end - tile_begin + NG * NT - 1) / (NG * NT);
  const int nstages = (ks_end - ks_begin + SK - 1) / SK;
  const int total = ngroups * nstages;

  // Every load is unconditional (clamped address): K steps past the end are zeroed on their way
  // into LDS, tiles past the end are dropped in finish().
  half8_t xr[XP];
  auto gload_x = [&](int idx) {
    const int kb = ks_begin + (idx % nstages) * SK;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      // Piece p = 64 * f + lane: fragment f is the same for the whole wave, so the address is a
      // scalar base plus the lane's 16 bytes.  A stage need not split evenly over the waves:
      // surplus slots re-read the last fragment.
      const int f = min(wave + (THREADS / 64) * i, PIECES / 64 - 1);
      const int kk = min(kb + f / MB, ks_end - 1);
      const half_t* frag = xp + ((int64_t)kk * MB + f % MB) * 512;
      xr[i] = *reinterpret_cast<const half8_t*>(reinterpret_cast<const char*>(frag) + lane_off);
    }
  };
  auto lstore = [&](int idx) {
    const int kb = ks_begin + (idx % nstages) * SK;
    half_t* l = lx_share + (idx & 1) * XH;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int f = wave + (THREADS / 64) * i;  // wave-uniform, as are the two conditions
      const bool live = kb + f / MB < ks_end;
      if (PIECES % THREADS == 0 || f < PIECES / 64)
        *reinterpret_cast<half8_t*>(l + f * 512 + lane * 8) = live ? xr[i] : zero8();
    }
  };
  struct Wst {
    half8_t a[UA][NT];  // fp16: one A fragment; int8: 16 raw bytes = two A fragments
  };
  uint32_t sc[NT];  // int8: the row's fp16 scale in the low half, one per tile of the group
  auto gload_sc = [&](int grp) {
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int t = min(tile_begin + (grp * NT + j) * NG + ng, tile_end - 1);
      sc[j] = W8 ? reinterpret_cast<const uint16_t*>(scales)[t * 16 + (lane & 15)] : 0u;
    }
  };
  auto gload_w = [&](Wst& w, int idx) {
    const int grp = idx / nstages, st = idx - grp * nstages;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const int t = min(tile_begin + (grp * NT + j) * NG + ng, tile_end - 1);
#pragma unroll
      for (int u = 0; u < UA; ++u) {
        const int ks = ks_begin + st * SK + kl * U + (W8 ? 2 * u : u);
        const int ksc = min(ks, ks_end - (W8 ? 2 : 1));
        const int64_t blk = W8 ? (int64_t)t * (nks >> 1) + (ksc >> 1) : (int64_t)t * nks + ksc;
        const half_t* block = (const half_t*)Wp + blk * 512;  // wave-uniform
        w.a[u][j] = __builtin_nontemporal_load(
            reinterpret_cast<const half8_t*>(reinterpret_cast<const char*>(block) + lane_off));
      }
    }
  };

  float4_t acc[NT][MB];
  auto clear = [&]() {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[j][mb] = float4_t{0.f, 0.f, 0.f, 0.f};
  };
  auto compute = [&](const Wst& w, int idx) {
    const half_t* l = lx_share + (idx & 1) * XH + kl * U * MB * 512 + lane * 8;
    constexpr int F = U * MB;  // fragment f = K step f / MB, row block f % MB
    constexpr int PD = KL * NG > 8 ? 2 : 4;  // LDS fragment reads in flight (registers are
                                             // scarcer at three waves per SIMD)
    half8_t bx[PD];
#pragma unroll
    for (int p = 0; p < PD; ++p) bx[p] = *reinterpret_cast<const half8_t*>(l + p * 512);
    // the A fragments of K step u (one set only where registers are scarce: the other waves of
    // the SIMD then cover the expansion)
    constexpr int AB = PF > 2 ? 1 : 2;
    half8_t a[AB][NT];
    auto expand = [&](int u) {
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        if (W8) {
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          const u4 raw = __builtin_bit_cast(u4, w.a[u / 2][j]);
          const half_t scj = __builtin_bit_cast(half2_t, sc[j])[0];
          a[u % AB][j] = (u & 1) ? dequant8(raw[2], raw[3], scj) : dequant8(raw[0], raw[1], scj);
        } else {
          a[u % AB][j] = w.a[W8 ? 0 : u][j];
        }
      }
    };
    // the stage's LDS stores and global loads go out first, then LDS reads and MFMAs alternate
    __builtin_amdgcn_sched_group_barrier(0x200, XP, 0);
    __builtin_amdgcn_sched_group_barrier(0x020, XP, 0);  // activations first: needed first
    __builtin_amdgcn_sched_group_barrier(0x020, UA * NT, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, PD, 0);
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const int u = f / MB, mb = f % MB;
      if (mb == 0) expand(u);
      const half8_t cur = bx[f % PD];
#pragma unroll
      for (int j = 0; j < NT; ++j)
        acc[j][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[u % AB][j], cur, acc[j][mb], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, NT, 0);
      if (f + PD < F) {
        bx[f % PD] = *reinterpret_cast<const half8_t*>(l + (f + PD) * 512);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };
  auto finish = [&](int idx) {  // after the last stage of a tile group
    const int grp = idx / nstages;
    float4_t* red = red_own;
    if constexpr (C::RED_ALIAS) {  // the stage just consumed, once every wave is done reading it
      red = reinterpret_cast<float4_t*>(lx_share + (idx & 1) * XH);
      __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < NT; ++j) {  // one tile slot per round through the reduction buffer
      if (kl > 0) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          red[(((kl - 1) * NG + ng) * MB + mb) * 64 + lane] = acc[j][mb];
      }
      __syncthreads();
      const int t = tile_begin + (grp * NT + j) * NG + ng;
      if (kl == 0 && t < tile_end) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          float4_t sum = acc[j][mb];
#pragma unroll
          for (int k = 1; k < KL; ++k) sum += red[(((k - 1) * NG + ng) * MB + mb) * 64 + lane];
          const int m = mb * 16 + (lane & 15);
          const int n = t * 16 + ((lane >> 4) << 2);
          if (m >= M) continue;
          if (part)
            *reinterpret_cast<float4_t*>(part + ((int64_t)blockIdx.y * M + m) * N + n) = sum;
          else
            epilogue4<MODE>(epi, m, n, sum);
        }
      }
      if (j + 1 < NT) __syncthreads();  // the buffer is rewritten by the next slot
    }
    clear();
    if (W8 && grp + 1 < ngroups) gload_sc(grp + 1);
  };

  // PF - 1 weight stages in flight beyond the one being consumed
  Wst w[PF];
  clear();
  if (W8) gload_sc(0);
  // same issue order as in the loop (activations of the next stage, then weights), so that the
  // wait before the loop's first LDS store does not cover the weight loads
  gload_x(0);
  lstore(0);
  gload_x(1);
#pragma unroll
  for (int st = 0; st < PF - 1; ++st) gload_w(w[st], st);
  __syncthreads();
  // Stages are taken PF at a time; surplus stages at the end work on clamped addresses into
  // accumulators that are never stored.
  for (int idx = 0; idx < total; idx += PF) {
#pragma unroll
    for (int st = 0; st < PF; ++st) {
      const int i = idx + st;
      lstore(i + 1);  // fetched during stage i - 1
      gload_x(i + 2);
      gload_w(w[(st + PF - 1) % PF], i + PF - 1);
      compute(w[st], i);
      if (i < total && (i + 1) % nstages == 0) finish(i);
      __syncthreads();
    }
  }
}

// sums split-K partials part[s][m][n] in slice order and applies the epilogue
template <int MODE>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int S,
                                                            int M, int N, Epilogue epi) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one float4 of one row
  const int nq = N >> 2;
  if (idx >= (int64_t)M * nq) return;
  const int m = (int)(idx / nq), n = (int)(idx % nq) << 2;
  float4_t s = *reinterpret_cast<const float4_t*>(part + (int64_t)m * N + n);
  for (int i = 1; i < S; ++i)
    s += *reinterpret_cast<const float4_t*>(part + ((int64_t)i * M + m) * N + n);
  epilogue4<MODE>(epi, m, n, s);
}

// ---- tiled kernel ---------------------------------------------------------------------
constexpr int TL_BM = 128, TL_BN = 128, TL_BK = 32, TL_LD = TL_BK + 8, TL_THREADS = 256;

template <bool W8, int MODE>
__global__ __launch_bounds__(TL_THREADS) void linear_tiled_kernel(
    const half_t* __restrict__ x, const void* __restrict__ Wp, const half_t* __restrict__ scales,
    int64_t M, int N, int K, Epilogue epi) {
  __shared__ __attribute__((aligned(16))) half_t lx[2][TL_BM * TL_LD];
  __shared__ __attribute__((aligned(16))) half_t lw[2][TL_BN * TL_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int li = lane & 31, lg = lane >> 5;
  const int64_t m0 = (int64_t)blockIdx.y * TL_BM;
  const int n0 = blockIdx.x * TL_BN;
  const int nkt = K / TL_BK;
  const int nks = K >> 5;

  // staging: each thread moves two 16-byte pieces of each operand tile.  x: piece c covers row
  // c/4, columns 8*(c%4); W: piece c is lane c%64 of the packed block of row tile c/64.
  int xrow[2], xcol[2], wrow[2], wcol[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + TL_THREADS * i;
    xrow[i] = c >> 2;
    xcol[i] = (c & 3) << 3;
    wrow[i] = (c >> 6) * 16 + (c & 15);
    wcol[i] = ((c >> 4) & 3) << 3;
  }
  half8_t rx[2], rw[2];

  auto load_tile = [&](int kt) {
    const int k0 = kt * TL_BK;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int64_t m = m0 + xrow[i];
      if (m < M)
        rx[i] = *reinterpret_cast<const half8_t*>(x + m * K + k0 + xcol[i]);
      else
        rx[i] = zero8();
      const int n = n0 + wrow[i];
      if (n < N) {
        const int c = tid + TL_THREADS * i;
        if (!W8) {
          rw[i] = *reinterpret_cast<const half8_t*>((const half_t*)Wp +
                                                    ((int64_t)(n >> 4) * nks + kt) * 512 +
                                                    (c & 63) * 8);
        } else {
          const uint2 w = *reinterpret_cast<const uint2*>(
              (const int8_t*)Wp + ((int64_t)(n >> 4) * (nks >> 1) + (kt >> 1)) * 1024 +
              (c & 63) * 16 + (kt & 1) * 8);
          rw[i] = dequant8(w.x, w.y, scales[n]);
        }
      } else {
        rw[i] = zero8();
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<half8_t*>(&lx[buf][xrow[i] * TL_LD + xcol[i]]) = rx[i];
      *reinterpret_cast<half8_t*>(&lw[buf][wrow[i] * TL_LD + wcol[i]]) = rw[i];
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

// ---- large tiled kernel -------------------------------------------------------------------
// 256 x 256 x 64 per workgroup of 8 waves on v_mfma_f32_16x16x32_f16; every wave owns 32 output
// features (two weight tiles) for all 256 activation rows.  Weight fragments come straight from
// the packed layout in global memory into registers (one KB per wave instruction, no LDS round
// trip, no two waves read the same weights); only the row-major activations are staged through
// LDS, double buffered, one barrier per 64-wide K stage.  A staged row is 128 bytes, unpadded, and
// its eight 16-byte chunks are stored XOR-swizzled by (row / 2) % 8: this part's LDS serves 256
// bytes per clock only when the 16 lanes it takes together hit 16 different 16-byte bank groups,
// which rows padded to 144 bytes do not (measured: 128 bytes per clock, i.e. the fragment reads of a
// stage alone took as long as its MFMAs).  The stage is software pipelined by
// hand: activations are fetched two stages ahead and parked in LDS one stage ahead, weights
// are fetched one stage ahead, LDS fragment reads run TB_PD fragments ahead of the MFMAs, and
// sched_group_barrier pins that order.  The main loop is branch free: rows and tiles past the
// edge read clamped addresses and are dropped in the epilogue.  Needs K % 128 == 0.
constexpr int TB_BM = 256, TB_BN = 256, TB_BK = 64, TB_LD = TB_BK, TB_THREADS = 512;
constexpr int TB_MF = TB_BM / 16;       // activation fragments per wave and 32-wide step
constexpr int TB_NT = TB_BN / 8 / 16;   // weight tiles per wave
constexpr int TB_PD = 4;                // LDS fragment reads in flight
constexpr int TB_LDS_BYTES = 2 * TB_BM * TB_LD * (int)sizeof(half_t);

template <bool W8>
struct BigW {  // the weight fragments of one 64-wide stage; int8: the raw 16 bytes per tile
  half8_t f[W8 ? 1 : 2][TB_NT];
};

template <bool W8, int MODE>
__global__ __launch_bounds__(TB_THREADS) void linear_tiled_big_kernel(
    const half_t* __restrict__ x, const void* __restrict__ Wp, const half_t* __restrict__ scales,
    int64_t M, int N, int K, Epilogue epi) {
  extern __shared__ __attribute__((aligned(16))) half_t lx_big[];  // [2][TB_BM * TB_LD]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.y * TB_BM;
  const int n0 = blockIdx.x * TB_BN + wave * (TB_NT * 16);
  const int nkt = K / TB_BK;
  const int ntiles = N / 16;

  // activation staging: piece c = row c/8, 16-byte chunk c%8 (8 lanes cover one 128-byte line)
  const half_t* xsrc[4];
  int xdst[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + TB_THREADS * i;
    const int row = c >> 3, ch = c & 7;
    const int64_t m = min(m0 + row, M - 1);
    xsrc[i] = x + m * K + ch * 8;
    xdst[i] = row * TB_LD + ((ch ^ ((row >> 1) & 7)) * 8);
  }
  const char* wsrc[TB_NT];
  half_t wscale[TB_NT];
#pragma unroll
  for (int j = 0; j < TB_NT; ++j) {
    const int t = min(n0 / 16 + j, ntiles - 1);
    // a tile's K sweep is K * 16 elements: K * 32 bytes in fp16, K * 16 bytes in int8
    wsrc[j] = (const char*)Wp + (int64_t)t * K * (W8 ? 16 : 32) + lane * 16;
    wscale[j] = W8 ? scales[t * 16 + lr] : (half_t)0.f;
  }

  auto gload_x = [&](half8_t(&xr)[4], int kt) {
    kt = min(kt, nkt - 1);
#pragma unroll
    for (int i = 0; i < 4; ++i) xr[i] = *reinterpret_cast<const half8_t*>(xsrc[i] + kt * TB_BK);
  };
  auto gload_w = [&](BigW<W8>& w, int kt) {
    kt = min(kt, nkt - 1);
#pragma unroll
    for (int j = 0; j < TB_NT; ++j) {
      if (W8) {
        w.f[0][j] = *reinterpret_cast<const half8_t*>(wsrc[j] + (int64_t)kt * 1024);
      } else {
        w.f[0][j] = *reinterpret_cast<const half8_t*>(wsrc[j] + (int64_t)kt * 2048);
        w.f[W8 ? 0 : 1][j] = *reinterpret_cast<const half8_t*>(wsrc[j] + (int64_t)kt * 2048 + 1024);
      }
    }
  };
  auto lstore = [&](const half8_t(&xr)[4], int buf) {
    half_t* l = lx_big + buf * (TB_BM * TB_LD);
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<half8_t*>(l + xdst[i]) = xr[i];
  };

  float4_t acc[TB_MF][TB_NT];
#pragma unroll
  for (int a = 0; a < TB_MF; ++a)
#pragma unroll
    for (int b = 0; b < TB_NT; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

  auto compute = [&](const BigW<W8>& w, int buf) {
    // fragment f = 32-wide step f / TB_MF, row block f % TB_MF: chunk 4 * step + lg of row
    // 16 * block + lr, whose swizzle is (lr / 2) % 8 for every block
    const half_t* lb = lx_big + buf * (TB_BM * TB_LD) + lr * TB_LD;
    const int sw = (lr >> 1) & 7;
    const half_t* l0 = lb + ((lg ^ sw) * 8);
    const half_t* l1 = lb + ((lg ^ sw ^ 4) * 8);
    auto frag = [&](int f) {
      return *reinterpret_cast<const half8_t*>((f / TB_MF ? l1 : l0) + (f % TB_MF) * 16 * TB_LD);
    };
    constexpr int F = 2 * TB_MF;
    half8_t a[2][TB_NT];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int j = 0; j < TB_NT; ++j) {
        if (W8) {
          const uint4 q = __builtin_bit_cast(uint4, w.f[0][j]);
          a[ks][j] = ks == 0 ? dequant8(q.x, q.y, wscale[j]) : dequant8(q.z, q.w, wscale[j]);
        } else {
          a[ks][j] = w.f[W8 ? 0 : ks][j];
        }
      }
    half8_t bx[TB_PD];
#pragma unroll
    for (int p = 0; p < TB_PD; ++p)
      bx[p] = frag(p);
    __builtin_amdgcn_sched_group_barrier(0x200, 4, 0);                         // LDS stores
    __builtin_amdgcn_sched_group_barrier(0x020, 4 + (W8 ? 1 : 2) * TB_NT, 0);  // global loads
    __builtin_amdgcn_sched_group_barrier(0x100, TB_PD, 0);                     // leading LDS reads
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const int ks = f / TB_MF, mf = f % TB_MF;
      const half8_t cur = bx[f % TB_PD];
#pragma unroll
      for (int j = 0; j < TB_NT; ++j)
        acc[mf][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[ks][j], cur, acc[mf][j], 0, 0, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, TB_NT, 0);
      if (f + TB_PD < F) {
        bx[f % TB_PD] = frag(f + TB_PD);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };

  half8_t xr[4];
  BigW<W8> w0, w1;
  gload_x(xr, 0);
  gload_w(w0, 0);
  lstore(xr, 0);
  gload_x(xr, 1);
  __syncthreads();
  for (int kt = 0; kt < nkt; kt += 2) {
    lstore(xr, 1);  // stage kt + 1, fetched during stage kt - 1
    gload_x(xr, kt + 2);
    gload_w(w1, kt + 1);
    compute(w0, 0);
    __syncthreads();
    lstore(xr, 0);
    gload_x(xr, kt + 3);
    gload_w(w0, kt + 2);
    compute(w1, 1);
    __syncthreads();
  }

  // D of the 16x16 MFMA: lane holds activation row (lane & 15) and the 4 consecutive features
  // 4 * (lane >> 4) .. + 3 of the weight tile
#pragma unroll
  for (int mf = 0; mf < TB_MF; ++mf) {
    const int64_t m = m0 + mf * 16 + lr;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TB_NT; ++j) {
      const int n = n0 + j * 16;
      if (n >= N) continue;
      epilogue4<MODE>(epi, m, n + lg * 4, acc[mf][j]);
    }
  }
}

// ---- large tiled kernel, fp16 weights: four waves of 128 x 128 ---------------------------------
// 256 x 256 per workgroup of 4 waves (2 x 2), one wave per SIMD, each wave 128 rows x 128 features
// on v_mfma_f32_16x16x32_f16: 64 accumulator tiles = 256 registers, kept in the AGPR bank.  hipcc
// copies such accumulators in and out of the bank around every MFMA, so the MFMAs are issued from
// inline assembly with the accumulator tied in place ("+a").  Both operands go global -> LDS
// directly (global_load_lds_dwordx4: LDS address = M0 + instruction offset + 16 * lane, global
// address = scalar base + lane offset + the same instruction offset), so no load ever targets a
// register and the only hand-placed waits are the vmcnt before each barrier:
//   * activations in 64-wide stages (whole 128-byte lines), rows unpadded with their eight 16-byte
//     chunks XOR-swizzled by (row / 2) % 8, ring of 3 x 32 KB;
//   * weights in 32-wide steps, the packed 16 x 32 blocks as they lie in memory (lane order, so the
//     fragment reads are linear), ring of 4 x 16 KB.
// A group of loads (the 8 of a wave's share of a stage, the 4 of its share of a step) shares one
// M0 and one lane offset; the instruction offset picks the 1 KB piece, and the scalar bases, which
// are loop invariant, are moved back by it.
// One barrier per 32-wide step.  Behind the barrier of step t the weights of step t+1 (and, every
// other step, the activations of the next stage) are complete and the buffers of step t are free:
// the loads of step t+4 / stage S+2 are issued there, one between every few MFMAs, and the 16
// fragments of step t+1 are read under the 64 MFMAs of step t (one ds_read_b128 per 4 MFMAs, a
// quarter of the LDS traffic per MFMA of the 8-wave kernel above).
// Epilogue through LDS: a lane holds 4 features of 16 different rows per tile, which as stores are
// 32-byte pieces; the rounded tile rows are parked in LDS and read back as 16 bytes per lane, whole
// 256-byte row pieces per 16 lanes.
// Workgroup -> tile: consecutive workgroups land on consecutive XCDs; where the default order would
// give an XCD a long thin strip of a round's tiles, the 256 tiles of a round are regrouped so that
// every XCD's L2 serves a compact a x b block (rm_a, rm_b, rm_r from the host).
// Three widths of the workgroup's tile, by the number WF of 16-feature weight fragments per wave:
// 8 -> 256 x 256 (as described), 4 -> 256 x 128, 2 -> 256 x 64 (fewer accumulators, weight loads and
// MFMAs per step; the same activation stages).  The two wider forms need M >= 256: a ragged last
// row tile is moved up to end at M and stores only the rows no other tile owns.  The narrowest
// form repeats the last row in its loads instead and drops the rows past it, so it also serves
// fewer than 256 rows.  All need K % 64 == 0, K >= 128.
constexpr int TQ_BM = 256, TQ_THREADS = 256;
constexpr int TQ_RX = 3, TQ_RW = 4;
constexpr int TQ_XBYTES = TQ_BM * 64 * 2;       // one 64-wide stage of activations
constexpr int TQ_WOFF = TQ_RX * TQ_XBYTES;
constexpr int tq_bn(int WF) { return 32 * WF; }
constexpr int tq_wbytes(int WF) { return 2 * WF * 1024; }  // one 32-wide step of weights
constexpr int tq_lds_bytes(int WF) {  // 160 / 128 / 112 KB
  return TQ_RX * TQ_XBYTES + TQ_RW * tq_wbytes(WF);
}
typedef __attribute__((address_space(3))) void tq_lds_void;

#define TQ_MFMA(ACC, A, B) \
  asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(ACC) : "v"(A), "v"(B))

template <int... I, class F>
__device__ __forceinline__ void tq_static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void tq_static_for(F&& f) {
  tq_static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// 8 consecutive output columns n..n+7 of row m; v holds the accumulators rounded to fp16, b the
// bias and r the residual values of those columns (read only where the epilogue has them)
// (QKV mode: qb, qt = the row's batch row and position, m = qb * T + qt)
template <int MODE>
__device__ __forceinline__ void epilogue8(const Epilogue& e, int64_t m, int n, half8_t v,
                                          half8_t b, half8_t r, int qb, int qt) {
  float t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = (float)v[i];
  if (e.bias) {
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = round_h(t[i] + (float)b[i]);
  }
  half8_t o;
  if (MODE == MODE_PLAIN) {
    if (e.flags & MSA_EPI_RELU) {
#pragma unroll
      for (int i = 0; i < 8; ++i) t[i] = fmaxf(t[i], 0.f);
    }
    if (e.residual) {
#pragma unroll
      for (int i = 0; i < 8; ++i) t[i] = round_h(t[i] + (float)r[i]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = (half_t)t[i];
    if (e.out_mb > 0)
      *reinterpret_cast<half8_t*>(e.y + packed_act_offset((int)m, n, e.out_mb)) = o;
    else
      *reinterpret_cast<half8_t*>(e.y + m * e.N + n) = o;
  } else {
    const int D = e.H * e.hd;
    const int part = (n >= D) + (n >= 2 * D), c = n - part * D;  // 0 = K, 1 = V, 2 = Q
    if (part == 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = (half_t)(t[i] * e.qscale);
      *reinterpret_cast<half8_t*>(e.q_out + m * D + c) = o;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] = (half_t)t[i];
      const int h = e.hd_shift >= 0 ? c >> e.hd_shift : c / e.hd, d = c - h * e.hd;
      const int s0 = e.len_dev ? e.len_dev[qb] : e.S0;
      if (s0 >= 0 && s0 + qt < e.S_cap) {
        half_t* dst = (part == 0 ? e.Kc : e.Vc) +
                      (((int64_t)qb * e.H + h) * e.S_cap + s0 + qt) * e.hd + d;
        *reinterpret_cast<half8_t*>(dst) = o;
      }
    }
  }
}

// PART: split-K.  Workgroup (bx, by, z) sums over the K range of ``part_stages`` 64-wide stages
// that starts at stage z * part_stages and stores its fp32 sums, with no epilogue, as slice z of
// ``part`` ([gridDim.z][M][N]); a later launch adds the slices in slice order.
template <int MODE, int WF, bool PART = false>
__global__ __launch_bounds__(TQ_THREADS) void linear_quad_kernel(
    const half_t* __restrict__ x, const void* __restrict__ Wp, int64_t M, int N, int K,
    int rm_a, int rm_b, int rm_r, Epilogue epi, float* __restrict__ part, int part_stages) {
  extern __shared__ __attribute__((aligned(16))) char tq_lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int TQ_BN = tq_bn(WF), TQ_WBYTES = tq_wbytes(WF);
  constexpr int WL = WF / 2;  // weight load instructions per wave and step
  int bx = blockIdx.x, by = blockIdx.y;
  if (rm_a > 0) {
    const int ncol = gridDim.x, L = by * ncol + bx, round = L >> 8, i = L & 255;
    if ((round + 1) * rm_r <= (int)gridDim.y) {  // a full round of 256 tiles
      const int xcd = i & 7, k = i >> 3, gx = ncol / rm_a;
      bx = (xcd % gx) * rm_a + k % rm_a;
      by = round * rm_r + (xcd / gx) * rm_b + k / rm_a;
    }
  }
  // The narrowest form (WF = 2) also serves fewer than 256 rows: it does not move a ragged tile up
  // but repeats the last row in its loads and drops the rows past it in the epilogue.  So does
  // the split-K form of WF = 4 (decode batches of 129 .. 255 rows cut K eight ways over it).
  constexpr bool CLAMP = WF == 2 || (WF == 4 && PART);
  const int64_t m_own = (int64_t)by * TQ_BM;  // first row this tile owns
  const int64_t m0 = !CLAMP && m_own + TQ_BM > M ? M - TQ_BM : m_own;
  const int n0 = bx * TQ_BN;
  // the stages this workgroup sums over: all of K, or its slice (the operand bases below move
  // to the slice's first stage, so that stage and step numbers count from 0 either way)
  const int st_first = PART ? (int)blockIdx.z * part_stages : 0;
  const int nst = PART ? part_stages : K / 64, nks = 2 * nst;
  const int ntiles = N / 16;

  // direct loads.  Activations, per stage: instruction i (0..7) of the wave fills rows
  // 64 * wave + 8 * i .. + 7 (lane l: row l / 8, chunk position l % 8, which must hold chunk
  // (l % 8) ^ ((row / 2) % 8) = (l % 8) ^ (4 * (i % 2) + l / 16)), with M0 at the wave's piece
  // + 4 KB and instruction offset 1024 * (i - 4).  Weights, per step: the wave copies the blocks
  // of tiles 4 * wave .. 4 * wave + 3, instruction offset 1024 * j.
  const char* xb[8];
  const char* wb[WL];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int64_t r = m0 + wave * 64 + i * 8;
    xb[i] = (const char*)(x + (CLAMP ? min(r, M - 1) : r) * K + (int64_t)st_first * 64) -
            (i - 4) * 1024;
  }
#pragma unroll
  for (int j = 0; j < WL; ++j) {
    const int tt = min(n0 / 16 + wave * WL + j, ntiles - 1);
    wb[j] = (const char*)Wp + (int64_t)tt * K * 32 + (int64_t)st_first * 2048 - j * 1024;
  }
  const uint32_t xrow = (uint32_t)(lane >> 3) * (uint32_t)K * 2;
  const uint32_t xlane0 = xrow + (((lane & 7) ^ (lane >> 4)) * 16);
  const uint32_t xlane1 = xrow + (((lane & 7) ^ (4 + (lane >> 4))) * 16);
  const uint32_t wlane = lane * 16;
  // CLAMP: per instruction, the lane's row offset from the (clamped) scalar base row
  uint32_t xl[CLAMP ? 8 : 1];
  if (CLAMP) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t r = m0 + wave * 64 + i * 8;
      const int64_t d = min(r + (lane >> 3), M - 1) - min(r, M - 1);
      xl[i] = (uint32_t)d * (uint32_t)K * 2 + ((i & 1 ? xlane1 : xlane0) - xrow);
    }
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(tq_lds_void*)tq_lds;
  // Lane offsets and LDS base of the group being issued.  The LDS base travels in M0, which every
  // load names as an explicit register operand: the compiler then knows that M0 is live between
  // the loads of a group (ordinary code - fragment reads, MFMAs - runs between them) and writes
  // it once per group.
  uint32_t xv0 = 0, xv1 = 0, wv = 0, xst = 0, xm0 = 0, wm0 = 0;
  auto set_x = [&](int slot, int st) {
    st = min(st, nst - 1);
    xst = st * 128;
    xv0 = xlane0 + st * 128;
    xv1 = xlane1 + st * 128;
    xm0 = lds0 + slot * TQ_XBYTES + wave * (64 * 128) + 4096;
  };
  auto set_w = [&](int slot, int ks) {
    ks = min(ks, nks - 1);
    wv = wlane + ks * 1024;
    wm0 = lds0 + TQ_WOFF + slot * TQ_WBYTES + wave * (WL * 1024);
  };
  auto issue_x = [&](auto ic) {
    constexpr int i = decltype(ic)::value;
    const uint32_t vo = CLAMP ? xl[CLAMP ? i : 0] + xst : (i & 1 ? xv1 : xv0);
    const char* sb = xb[i];
    const uint32_t base = xm0;
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(vo), "s"(sb),
                 "n"((i - 4) * 1024), "{m0}"(base)
                 : "memory");
  };
  auto issue_w = [&](auto jc) {
    constexpr int j = decltype(jc)::value;
    const uint32_t vo = wv;
    const char* sb = wb[j];
    const uint32_t base = wm0;
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(vo), "s"(sb), "n"(j * 1024),
                 "{m0}"(base)
                 : "memory");
  };
  auto group_x = [&](int slot, int st) {
    set_x(slot, st);
    tq_static_for<8>([&](auto ic) { issue_x(ic); });
  };
  auto group_w = [&](int slot, int ks) {
    set_w(slot, ks);
    tq_static_for<WL>([&](auto jc) { issue_w(jc); });
  };

  // fragment reads.  Activation fragment i of half h of a stage: row 128 * wm + 16 * i + lr, chunk
  // 4 * h + lg at position (4 * h + lg) ^ ((lr / 2) % 8); weight fragment j: tile 8 * wn + j.
  const int sw = (lr >> 1) & 7;
  const uint32_t xoff0 = (uint32_t)(wm * 128 + lr) * 128 + ((lg ^ sw) * 16);
  const uint32_t xoff1 = (uint32_t)(wm * 128 + lr) * 128 + ((lg ^ sw ^ 4) * 16);
  const uint32_t woff = TQ_WOFF + (uint32_t)(wn * WF) * 1024 + lane * 16;
  auto xfrag = [&](int slot, int h, int i) {
    return *reinterpret_cast<const half8_t*>(tq_lds + slot * TQ_XBYTES + (h ? xoff1 : xoff0) +
                                             i * (16 * 128));
  };
  auto wfrag = [&](int slot, int j) {
    return *reinterpret_cast<const half8_t*>(tq_lds + slot * TQ_WBYTES + woff + j * 1024);
  };

  float4_t acc[8][WF];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < WF; ++j) {
      acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
      asm volatile("" : "+a"(acc[i][j]));
    }

  // prologue: activation stages 0 and 1, weight steps 0..3 requested; stages 0, 1 and steps 0, 1
  // landed
  half8_t xf[2][8], wf[2][WF];
  group_x(0, 0);
  group_w(0, 0);
  group_x(1, 1);
  group_w(1, 1);
  group_w(2, 2);
  group_w(3, 3);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * WL) : "memory");
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) xf[0][i] = xfrag(0, 0, i);
#pragma unroll
  for (int j = 0; j < WF; ++j) wf[0][j] = wfrag(0, j);

  // step t = 2 S + H; xs, ws: ring slots of stage S and step t.  An even step issues 8 + WL loads
  // (stage S + 2, then step t + 4), an odd one WL (step t + 4).  Loads complete in order; the
  // weights of step t + 1 were requested in step t - 3, and the 8 + 2 WL loads of steps t - 2 and
  // t - 1 may still be outstanding at the barrier.  The activations an odd step starts to read
  // (stage S + 1) were requested in step t - 3 as well, ahead of that step's weights.
  // The 8 x WF MFMAs of a step carry, one each: the 8 + WF fragment reads of step t + 1 and the
  // loads (even steps: activations under rows 0..3, weights under rows 4..7).
  auto step = [&](int t, int xs, int ws, auto hc) {
    constexpr int H = decltype(hc)::value;
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(8 + 2 * WL) : "memory");
    __syncthreads();
    const int S = t >> 1;
    const int xfree = xs == 0 ? TQ_RX - 1 : xs - 1;  // slot of stage S - 1 = slot of stage S + 2
    const int xnext = xs == TQ_RX - 1 ? 0 : xs + 1;  // slot of stage S + 1
    const int wnext = ws == TQ_RW - 1 ? 0 : ws + 1;  // slot of step t + 1
    tq_static_for<8>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      tq_static_for<WF>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        TQ_MFMA(acc[i][j], wf[H][j], xf[H][i]);
        if (j == 1) xf[H ^ 1][i] = H == 0 ? xfrag(xs, 1, i) : xfrag(xnext, 0, i);
        if constexpr (WF == 8) {
          if (j == 5) wf[H ^ 1][i % WF] = wfrag(wnext, i % WF);
        } else if constexpr (WF == 4) {
          if constexpr (j == 3 && (i & 1)) wf[H ^ 1][(i >> 1) % WF] = wfrag(wnext, (i >> 1) % WF);
        } else {
          if constexpr (j == 0 && (i == 1 || i == 5)) wf[H ^ 1][(i >> 2) % WF] = wfrag(wnext, (i >> 2) % WF);
        }
        if constexpr (H == 0) {
          if (i == 0 && j == 0) set_x(xfree, S + 2);
          if constexpr (i < 4 && j == WF / 2 - 1) issue_x(std::integral_constant<int, (i & 3) * 2>{});
          if constexpr (i < 4 && j == WF - 1) issue_x(std::integral_constant<int, (i & 3) * 2 + 1>{});
          if (i == 4 && j == 0) set_w(ws, t + TQ_RW);
          if constexpr (WF == 8) {
            if constexpr (i >= 4 && j == 3) issue_w(std::integral_constant<int, (i & 3) % WL>{});
          } else if constexpr (WF == 4) {
            if constexpr ((i == 4 || i == 6) && j == 2)
              issue_w(std::integral_constant<int, ((i >> 1) & 1) % WL>{});
          } else {
            if constexpr (i == 4 && j == 1) issue_w(std::integral_constant<int, 0>{});
          }
        } else {
          if (i == 0 && j == 0) set_w(ws, t + TQ_RW);
          if constexpr (WF == 8) {
            if constexpr (j == 3 && (i & 1)) issue_w(std::integral_constant<int, (i >> 1) % WL>{});
          } else if constexpr (WF == 4) {
            if constexpr ((i == 2 || i == 6) && j == 2)
              issue_w(std::integral_constant<int, ((i >> 2) & 1) % WL>{});
          } else {
            if constexpr (i == 2 && j == 1) issue_w(std::integral_constant<int, 0>{});
          }
        }
      });
    });
  };
  int xs = 0, ws = 0;
  for (int t = 0; t < nks; t += 2) {
    step(t, xs, ws, std::integral_constant<int, 0>{});
    ws = ws == TQ_RW - 1 ? 0 : ws + 1;
    step(t + 1, xs, ws, std::integral_constant<int, 1>{});
    ws = ws == TQ_RW - 1 ? 0 : ws + 1;
    xs = xs == TQ_RX - 1 ? 0 : xs + 1;
  }
  // no direct load may still be in flight when the rings are reused below (or when the workgroup's
  // LDS is released); the last MFMAs must have written their accumulators before these are read
  // (the compiler does not see MFMAs inside the asm)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  // ties every accumulator to this point: none of their reads may be scheduled above the wait
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < WF; ++j) asm volatile("" : "+a"(acc[i][j]));
  __syncthreads();  // every wave is done with the operand rings

  if constexpr (PART) {
    // the sums as the lanes hold them: D tile (i, j) = activation row 16 * i + lr of the wave's
    // 128, features 16 * j + 4 * lg .. + 3 of the wave's 16 WF (16 bytes per lane, 64 per row)
    float* slice = part + (int64_t)blockIdx.z * M * N;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t m = m0 + wm * 128 + i * 16 + lr;
#pragma unroll
      for (int j = 0; j < WF; ++j) {
        const int n = n0 + wn * (16 * WF) + 16 * j + 4 * lg;
        if (m >= m_own && m < M && n < N)
          *reinterpret_cast<float4_t*>(slice + m * N + n) = acc[i][j];
      }
    }
    return;
  }

  // D tile (i, j): the lane holds activation row 16 * i + lr of the wave's 128 and the 4 features
  // 16 * j + 4 * lg ...  Per i the wave's 16 rows x 16 WF features (4 or 2 KB, two buffers per wave)
  // are written as the lanes hold them (16-byte chunk 2 j + lg / 2 of the row, swizzled by the row)
  // and read back 16 bytes per lane, whole rows per 16 (8) lanes.
  // The lane's column group is the same in every iteration, so the bias is read once; the residual
  // rows are requested four iterations ahead (the fragment registers are free now), so that their
  // latency is paid once per workgroup and not once per iteration.
  char* mine = tq_lds + wave * 8192;
  constexpr int ECH = 2 * WF;        // 16-byte chunks of a staged row (16 WF features)
  constexpr int ERB = 16 * ECH;      // bytes of a staged row
  constexpr int ERPI = 64 / ECH;     // rows a 64-lane read covers
  constexpr int ENR = 16 / ERPI;     // reads per 16 rows
  const int ec = lane % ECH, erow = lane / ECH;
  const int en = n0 + wn * (16 * WF) + ec * 8;
  const bool col_ok = en < N;
  half8_t bias8 = zero8();
  if (epi.bias && col_ok) bias8 = *reinterpret_cast<const half8_t*>(epi.bias + en);
  constexpr int TQ_RES_AHEAD = 4;
  half8_t res8[TQ_RES_AHEAD][ENR];
  auto load_res = [&](int i, half8_t(&dst)[ENR]) {
    if (MODE != MODE_PLAIN || !epi.residual) return;
#pragma unroll
    for (int r = 0; r < ENR; ++r) {
      const int64_t m = m0 + wm * 128 + i * 16 + ERPI * r + erow;
      if (col_ok && m >= m_own && m < M)
        dst[r] = *reinterpret_cast<const half8_t*>(epi.residual + m * epi.N + en);
    }
  };
#pragma unroll
  for (int i = 0; i < TQ_RES_AHEAD; ++i) load_res(i, res8[i]);
  // QKV mode: the lane's rows come ERPI apart, so (batch row, position) of a row follow from the
  // previous row's without a division
  int qb = 0, qt = 0;
  if (MODE == MODE_QKV) {
    const int mf = (int)(m0 + wm * 128 + erow);
    qb = epi.T == 1 ? mf : mf / epi.T;
    qt = mf - qb * epi.T;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    char* buf = mine + (i & 1) * 4096;
#pragma unroll
    for (int j = 0; j < WF; ++j) {
      half4_t o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (half_t)(acc[i][j][e]);
      const int c = (2 * j + (lg >> 1)) ^ (lr & (ECH - 1));
      *reinterpret_cast<half4_t*>(buf + lr * ERB + c * 16 + (lg & 1) * 8) = o;
    }
#pragma unroll
    for (int r = 0; r < ENR; ++r) {
      const int row = ERPI * r + erow;
      const half8_t v = *reinterpret_cast<const half8_t*>(buf + row * ERB +
                                                          ((ec ^ (row & (ECH - 1))) * 16));
      const int64_t m = m0 + wm * 128 + i * 16 + row;
      if (col_ok && m >= m_own && m < M)
        epilogue8<MODE>(epi, m, en, v, bias8, res8[i % TQ_RES_AHEAD][r], qb, qt);
      if (MODE == MODE_QKV) {
        qt += ERPI;
        while (qt >= epi.T) qt -= epi.T, ++qb;
      }
    }
    if (i + TQ_RES_AHEAD < 8) load_res(i + TQ_RES_AHEAD, res8[i % TQ_RES_AHEAD]);
  }
}

// ---- host side ------------------------------------------------------------------------------
// Per-device facts are kept per device: a process may drive several GPUs, from several threads.
constexpr int MAX_DEVICES = 64;
int current_device() {
  int dev = 0;
  return hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < MAX_DEVICES ? dev : -1;
}

std::atomic<int> g_num_cus[MAX_DEVICES];
int num_cus() {  // compute units of the current device
  const int dev = current_device();
  int n = dev >= 0 ? g_num_cus[dev].load(std::memory_order_relaxed) : 0;
  if (n == 0) {
    if (dev < 0 ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n <= 0)
      n = 256;
    if (dev >= 0) g_num_cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Raises a kernel's dynamic LDS limit once per device (one mask per kernel instantiation; a
// second thread that gets here at the same time only repeats the call).
bool allow_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done) {
  const int dev = current_device();
  const uint64_t bit = dev >= 0 ? 1ull << dev : 0;
  if (bit && (done.load(std::memory_order_acquire) & bit)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess)
    return false;
  if (bit) done.fetch_or(bit, std::memory_order_release);
  return true;
}

template <int MB, bool W8, int MODE, bool XR = false>
void launch_stream_mb(const void* xp, const void* W, const void* scales, float* part, int S, int M,
                      int N, int K, const Epilogue& epi, hipStream_t s, int64_t m_off = 0) {
  const int ntiles = N / 16, nks = K / 32;
  int G = num_cus() / S;
  if (G < 1) G = 1;
  const int tiles_per_wg = (ntiles + G - 1) / G;
  const int gx = (ntiles + tiles_per_wg - 1) / tiles_per_wg;
  int ks_per_split = (nks + S - 1) / S;
  if (W8) ks_per_split = (ks_per_split + 1) & ~1;  // int8 blocks cover two steps
  // Up to 32 packed rows: groups of 3 tiles instead of 4 when that needs no more groups (no
  // more sweeps over the activations) and leaves fewer empty tile slots, e.g. 3 tiles per
  // workgroup for qkv_proj at d_model 4096.
  if (MB <= 2 && !XR && (tiles_per_wg + 2) / 3 == (tiles_per_wg + 3) / 4 &&
      (tiles_per_wg + 2) / 3 * 3 < (tiles_per_wg + 3) / 4 * 4) {
    hipLaunchKernelGGL((linear_stream_kernel<(MB <= 2 ? MB : 1), W8, MODE, false, ST_KG, 3>),
                       dim3(gx, S), dim3(ST_KG * 64), 0, s, (const half_t*)xp, W,
                       (const half_t*)scales, part, M, N, K, tiles_per_wg, ks_per_split, epi,
                       m_off);
    return;
  }
  // The ragged bottom rows of a prefill-sized product (row-major activations, 33 .. 64 rows, fp16):
  // the workgroup's few tiles would leave most of the 8 tile slots per activation fragment empty
  // (their clamped loads still run), so groups of 4 are used when the tiles fit them.
  if constexpr (XR && !W8 && MB > 2) {
    if (tiles_per_wg <= ST_NT) {
      hipLaunchKernelGGL((linear_stream_kernel<MB, W8, MODE, XR, ST_KG, ST_NT>), dim3(gx, S),
                         dim3(ST_KG * 64), 0, s, (const half_t*)xp, W, (const half_t*)scales, part,
                         M, N, K, tiles_per_wg, ks_per_split, epi, m_off);
      return;
    }
  }
  hipLaunchKernelGGL((linear_stream_kernel<MB, W8, MODE, XR>), dim3(gx, S), dim3(ST_KG * 64), 0,
                     s, (const half_t*)xp, W, (const half_t*)scales, part, M, N, K, tiles_per_wg,
                     ks_per_split, epi, m_off);
}

constexpr int SH_GROUP = 12;  // most tiles per pass of the shared-activation kernel (4 lanes x 3)
constexpr int SH_GROUP_W8 = 18;  // int8 only: 6 lanes x 3

// The shared-activation kernel sweeps K once per pass of SH_GROUP tiles: it is used when the
// workgroup's tiles fill their passes to at least three quarters.
bool share_fits(int N, int S, bool w8) {
  int G = num_cus() / S;
  if (G < 1) G = 1;
  const int tpw = (N / 16 + G - 1) / G;
  if (tpw <= SH_GROUP) return true;  // one pass, with the tile count per wave chosen to fit
  if (w8 && tpw <= SH_GROUP_W8 && 4 * tpw >= 3 * SH_GROUP_W8) return true;  // one pass of 18
  const int passes = (tpw + SH_GROUP - 1) / SH_GROUP;
  return 4 * tpw >= 3 * passes * SH_GROUP;
}

template <int MB, bool W8, int MODE, int KL, int NG, int NT, int U, int PF = 2>
void launch_share_cfg(const void* xp, const void* W, const void* scales, float* part, int S, int M,
                      int N, int K, int tiles_per_wg, int gx, int ks_per_split, const Epilogue& epi,
                      hipStream_t s) {
  using C = ShareCfg<MB, W8, KL, NG, NT, U>;
  static std::atomic<uint64_t> lds_allowed{0};  // one mask per instantiation
  if (!allow_lds((const void*)linear_share_kernel<MB, W8, MODE, KL, NG, NT, U, PF>, C::LDS_BYTES,
                 lds_allowed))
    return;  // the caller's launch check reports the error
  hipLaunchKernelGGL((linear_share_kernel<MB, W8, MODE, KL, NG, NT, U, PF>), dim3(gx, S),
                     dim3(C::THREADS), C::LDS_BYTES, s, (const half_t*)xp, W,
                     (const half_t*)scales, part, M, N, K, tiles_per_wg, ks_per_split, epi);
}

// 33 .. 64 packed rows, no selection: the shared-activation kernel
template <int MB, bool W8, int MODE>
void launch_share(const void* xp, const void* W, const void* scales, float* part, int S, int M,
                  int N, int K, const Epilogue& epi, hipStream_t s) {
  const int ntiles = N / 16, nks = K / 32;
  int G = num_cus() / S;
  if (G < 1) G = 1;
  const int tiles_per_wg = (ntiles + G - 1) / G;
  const int gx = (ntiles + tiles_per_wg - 1) / tiles_per_wg;
  int ks_per_split = (nks + S - 1) / S;
  if (W8) ks_per_split = (ks_per_split + 1) & ~1;  // int8 blocks cover two steps
  // the wave grid and tiles per wave whose slots the workgroup's tiles fill best in one pass
  if constexpr (W8) {
    if (tiles_per_wg == 5 || tiles_per_wg == 6)
      return launch_share_cfg<MB, W8, MODE, 4, 3, 2, 2, 2>(xp, W, scales, part, S, M, N, K,
                                                        tiles_per_wg, gx, ks_per_split, epi, s);
    if (tiles_per_wg == 9)
      return launch_share_cfg<MB, W8, MODE, 4, 3, 3, 2, 2>(xp, W, scales, part, S, M, N, K,
                                                        tiles_per_wg, gx, ks_per_split, epi, s);
    if (tiles_per_wg > 12 && tiles_per_wg <= 18)
      return launch_share_cfg<MB, W8, MODE, 2, 6, 3, 2, 3>(xp, W, scales, part, S, M, N, K,
                                                        tiles_per_wg, gx, ks_per_split, epi, s);
  }
  if (tiles_per_wg <= 4)
    launch_share_cfg<MB, W8, MODE, 2, 4, 1, 8>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                               ks_per_split, epi, s);
  else if (tiles_per_wg <= 8)
    launch_share_cfg<MB, W8, MODE, 2, 4, 2, 4>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                               ks_per_split, epi, s);
  else
    launch_share_cfg<MB, W8, MODE, 2, 4, 3, 4>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                               ks_per_split, epi, s);
}

// 65 .. 128 packed rows (eight row blocks): the shared-activation kernel as 2 K lanes x 4 tile
// lanes with stages of four K steps (32 KB of activations per stage; two stages and the
// reduction buffer make 96 KB of LDS).  With so many rows per weight fragment the tiles of a
// workgroup are few per wave, so more weight stages are kept in flight instead (PF).  Measured
// at 128 x 12288 x 4096 (38.6 us as built): four K lanes x two tile lanes x two tiles 45.8 us,
// stages of eight K steps 43.0, six weight stages in flight instead of four 44.3.
template <bool W8, int MODE>
void launch_wide(const void* xp, const void* W, const void* scales, float* part, int S, int M,
                 int N, int K, const Epilogue& epi, hipStream_t s) {
  const int ntiles = N / 16, nks = K / 32;
  int G = num_cus() / S;
  if (G < 1) G = 1;
  const int tiles_per_wg = (ntiles + G - 1) / G;
  const int gx = (ntiles + tiles_per_wg - 1) / tiles_per_wg;
  int ks_per_split = (nks + S - 1) / S;
  if (W8) ks_per_split = (ks_per_split + 1) & ~1;  // int8 blocks cover two steps
  if (tiles_per_wg <= 4)
    launch_share_cfg<8, W8, MODE, 2, 4, 1, 2, 4>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                                 ks_per_split, epi, s);
  else if (tiles_per_wg <= 8)
    launch_share_cfg<8, W8, MODE, 2, 4, 2, 2, 3>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                                 ks_per_split, epi, s);
  else
    launch_share_cfg<8, W8, MODE, 2, 4, 3, 2, 2>(xp, W, scales, part, S, M, N, K, tiles_per_wg, gx,
                                                 ks_per_split, epi, s);
}

template <bool W8, int MODE, bool XR = false>
void launch_stream(const void* xp, const void* W, const void* scales, float* part, int S, int M,
                   int N, int K, const Epilogue& epi, hipStream_t s, int64_t m_off = 0) {
  if constexpr (!XR && MODE != MODE_SELECT) {
    if (M > 64) return launch_wide<W8, MODE>(xp, W, scales, part, S, M, N, K, epi, s);
  }
  if (!XR && MODE != MODE_SELECT && M > 32 && share_fits(N, S, W8)) {
    constexpr int PM = MODE == MODE_SELECT ? MODE_PLAIN : MODE;
    if (M > 48)
      launch_share<4, W8, PM>(xp, W, scales, part, S, M, N, K, epi, s);
    else
      launch_share<3, W8, PM>(xp, W, scales, part, S, M, N, K, epi, s);
    return;
  }
  switch ((M + 15) / 16) {
    case 1:
      launch_stream_mb<1, W8, MODE, XR>(xp, W, scales, part, S, M, N, K, epi, s, m_off);
      break;
    case 2:
      launch_stream_mb<2, W8, MODE, XR>(xp, W, scales, part, S, M, N, K, epi, s, m_off);
      break;
    case 3:
      launch_stream_mb<3, W8, MODE, XR>(xp, W, scales, part, S, M, N, K, epi, s, m_off);
      break;
    default:
      launch_stream_mb<4, W8, MODE, XR>(xp, W, scales, part, S, M, N, K, epi, s, m_off);
      break;
  }
}

// One launch of the four-wave kernel (WF = 8: 256 x 256 tiles, WF = 4: 256 x 128) on rows
// 0 .. M_main - 1 (a ragged last row tile is moved up) plus the streaming kernel on the rows from
// M_main on (at most 128).
template <int MODE, int WF>
void launch_quad(const void* x, const void* W, const void* scales, int64_t M, int64_t M_main, int N,
                 int K, const Epilogue& epi, hipStream_t s) {
  static std::atomic<uint64_t> lds_allowed_q{0};
  if (!allow_lds((const void*)linear_quad_kernel<MODE, WF>, tq_lds_bytes(WF), lds_allowed_q)) return;
  const int ncol = (N + tq_bn(WF) - 1) / tq_bn(WF);
  const int nrow = (int)((M_main + TQ_BM - 1) / TQ_BM);
  // regrouping of a round's 256 tiles: a x b per XCD with a * b = 32, (ncol / a) * (r / b) = 8
  // for r = 256 / ncol rows per round; taken when it beats the default strip (ncol / 8) x r
  int rm_a = 0, rm_b = 0, rm_r = 0;
  if (ncol >= 8 && 256 % ncol == 0) {
    const int r = 256 / ncol;
    int best = ncol / 8 + r;
    for (int a = 1; a <= 32; a *= 2) {
      const int b = 32 / a;
      if (ncol % a || r % b || (ncol / a) * (r / b) != 8) continue;
      if (a + b < best) best = a + b, rm_a = a, rm_b = b, rm_r = r;
    }
  }
  hipLaunchKernelGGL((linear_quad_kernel<MODE, WF>), dim3(ncol, nrow), dim3(TQ_THREADS),
                     tq_lds_bytes(WF), s, (const half_t*)x, W, M_main, N, K, rm_a, rm_b, rm_r, epi,
                     (float*)nullptr, 0);
  for (int64_t m0 = M_main; m0 < M; m0 += 64)
    launch_stream<false, MODE, true>(x, W, scales, nullptr, 1, (int)min((int64_t)64, M - m0), N,
                                     K, epi, s, m0);
}

// Split-K launch of a narrow four-wave form (WF = 2: 256 x 64 tiles, WF = 4: 256 x 128) on
// row-major activations: S slices of K, each a whole number of 64-wide stages (at least two),
// fp32 sums into part[S][M][N].
template <int WF>
void launch_quad_partial_w(const void* x, const void* W, float* part, int64_t M, int N, int K,
                           int S, hipStream_t s) {
  static std::atomic<uint64_t> lds_allowed_p{0};
  auto kernel = linear_quad_kernel<MODE_PLAIN, WF, true>;
  if (!allow_lds((const void*)kernel, tq_lds_bytes(WF), lds_allowed_p)) return;
  const int ncol = (N + tq_bn(WF) - 1) / tq_bn(WF);
  const int nrow = (int)((M + TQ_BM - 1) / TQ_BM);
  Epilogue e{};
  hipLaunchKernelGGL(kernel, dim3(ncol, nrow, S), dim3(TQ_THREADS), tq_lds_bytes(WF), s,
                     (const half_t*)x, W, M, N, K, 0, 0, 0, e, part, K / 64 / S);
}

// 256 x 64 tiles while their S slices fit the chip in one round; an S beyond that means 256 x 128
// tiles.
void launch_quad_partial(const void* x, const void* W, float* part, int64_t M, int N, int K, int S,
                         hipStream_t s) {
  const int64_t tiles2 = ((M + TQ_BM - 1) / TQ_BM) * ((N + tq_bn(2) - 1) / tq_bn(2));
  if (tiles2 * S > num_cus())
    return launch_quad_partial_w<4>(x, W, part, M, N, K, S, s);
  launch_quad_partial_w<2>(x, W, part, M, N, K, S, s);
}

// Slices for a product of M row-major rows whose tiles alone leave most of the chip idle (a
// decode batch of a few hundred rows against d_model output features): the most of 2, 4, 8 that
// keep the 256 x 64 tiles within the chip, the K range of a slice at 512 or more, and whole
// stages.  Where a slice would still span 4096 or more of K, twice the slices over 256 x 128
// tiles measured faster (half the activation bytes per workgroup and weight byte: M = 256,
// N = 4096, K = 16384: 51.8 against 55.4 us; M = 512: 78.0 against 93.6; M = 200, inside a
// decode step: 42.4 against 47.2).
int pick_row_splits(int64_t M, int N, int K) {
  if (M < 1 || N % 16 || K % 64) return 1;
  const int64_t tiles = ((M + TQ_BM - 1) / TQ_BM) * ((N + tq_bn(2) - 1) / tq_bn(2));
  int best = 1;
  for (int S = 2; S <= 8; S *= 2)
    if (tiles * S <= num_cus() && K % (64 * S) == 0 && K / S >= 512) best = S;
  if (best > 1 && best < 8 && M > 128 && K / best >= 4096 && K % (128 * best) == 0) best *= 2;
  return best;
}

template <bool W8, int MODE>
void launch_tiled(const void* x, const void* W, const void* scales, int64_t M, int N, int K,
                  const Epilogue& epi, hipStream_t s) {
  // Up to 64 rows (a short prompt, a small batch held row-major): one sweep of the
  // weight-streaming kernel, which reads its activation fragments from the row-major matrix.
  // No tile kernel comes near it there (64 x 12288 x 4096, fp16: 101 us on 128 x 128 tiles).
  if (M <= 64)
    return launch_stream<W8, MODE, true>(x, W, scales, nullptr, 1, (int)M, N, K, epi, s, 0);
  // int8 weights, up to 256 rows: a sweep per 64 rows.  The int8 tile kernels need thousands of
  // rows to fill the chip (128 x 9216 x 9216: 303 us on 128 x 128 tiles, 51 us per sweep).
  if constexpr (W8) {
    if (M <= 256) {
      for (int64_t m0 = 0; m0 < M; m0 += 64)
        launch_stream<W8, MODE, true>(x, W, scales, nullptr, 1, (int)min((int64_t)64, M - m0), N,
                                      K, epi, s, m0);
      return;
    }
  }
  // the 256 x 256 kernel once it fills the chip; the 128 x 128 one for the shapes in between
  const int64_t big_tiles = ((M + TB_BM - 1) / TB_BM) * ((N + TB_BN - 1) / TB_BN);
  if constexpr (!W8) {
    // Three tile widths, 256, 128 and 64 features (a workgroup of 128 does half the MFMAs of 256 in
    // about 0.8 of the time, one of 64 a quarter in about 0.55), and two ways to take a ragged
    // bottom of at most 128 rows: as one more, moved-up row of tiles, or through the streaming
    // kernel (one sweep over the weights per 64 rows).  The combinations are priced in rounds of
    // workgroups and the cheapest is taken.  The two wider forms go down to 3/8 of a tile per CU:
    // below that a single round of their tiles no longer beats the narrowest form, which is taken
    // down to 1/8 of a tile per CU and also serves 65 .. 255 rows (it repeats the last row instead
    // of moving a tile up); below that the 128 x 128 kernel runs.
    if (K % 64 == 0 && K >= 128 && M > 64) {
      const int64_t cus = num_cus(), rem = M % TQ_BM;
      const int64_t cols[3] = {(N + 255) / 256, (N + 127) / 128, (N + 63) / 64};
      const double factor[3] = {1.0, 0.8, 0.55};
      const double unit = 63.0 * K / 4096;  // us per round of wide tiles
      const double sweep = (double)N * K * 2 / 5e6 + 4;  // us per streaming launch
      double best = 1e30;
      int best_w = -1;
      int64_t best_main = M;
      for (int opt = 0; opt < 6; ++opt) {
        const int w = opt >> 1;
        const bool stream = opt & 1;
        if (w < 2 && M < TQ_BM) continue;
        if (stream && !(w < 2 && rem > 0 && rem <= 128 && M - rem >= TQ_BM)) continue;
        const int64_t m_main = stream ? M - rem : M;
        const int64_t tiles = ((m_main + TQ_BM - 1) / TQ_BM) * cols[w];
        if (tiles * 8 < (w == 2 ? cus : cus * 3)) continue;
        const double cost = (double)((tiles + cus - 1) / cus) * factor[w] * unit +
                            (stream ? (double)((rem + 63) / 64) * sweep : 0.0);
        if (cost < best) best = cost, best_w = w, best_main = m_main;
      }
      if (best_w == 0) return launch_quad<MODE, 8>(x, W, scales, M, best_main, N, K, epi, s);
      if (best_w == 1) return launch_quad<MODE, 4>(x, W, scales, M, best_main, N, K, epi, s);
      if (best_w == 2) return launch_quad<MODE, 2>(x, W, scales, M, best_main, N, K, epi, s);
    }
  }
  if (K % (2 * TB_BK) == 0 && big_tiles >= num_cus()) {
    static std::atomic<uint64_t> lds_allowed{0};  // one mask per instantiation
    if (!allow_lds((const void*)linear_tiled_big_kernel<W8, MODE>, TB_LDS_BYTES, lds_allowed))
      return;  // the launch check below reports the error
    // A ragged bottom block would cost a full extra round of workgroups for a few rows (a
    // prompt of 2^k tokens plus the leading end-of-sentence token always has one): up to 128
    // leftover rows go through the weight-streaming kernel instead, 64 rows at a time.
    int64_t M_main = M;
    const int64_t rem = M % TB_BM;
    if (rem > 0 && rem <= 128 && M > rem) M_main = M - rem;
    const dim3 grid((N + TB_BN - 1) / TB_BN, (unsigned)((M_main + TB_BM - 1) / TB_BM));
    hipLaunchKernelGGL((linear_tiled_big_kernel<W8, MODE>), grid, dim3(TB_THREADS), TB_LDS_BYTES,
                       s, (const half_t*)x, W, (const half_t*)scales, M_main, N, K, epi);
    for (int64_t m0 = M_main; m0 < M; m0 += 64)
      launch_stream<W8, MODE, true>(x, W, scales, nullptr, 1, (int)min((int64_t)64, M - m0), N, K,
                                    epi, s, m0);
    return;
  }
  const dim3 grid((N + TL_BN - 1) / TL_BN, (unsigned)((M + TL_BM - 1) / TL_BM));
  hipLaunchKernelGGL((linear_tiled_kernel<W8, MODE>), grid, dim3(TL_THREADS), 0, s,
                     (const half_t*)x, W, (const half_t*)scales, M, N, K, epi);
}

int check_linear_args(const char* name, const void* x, const void* W, const void* y, int64_t M,
                      int N, int K, bool w8, unsigned flags, unsigned allowed) {
  MSA_REQUIRE(x && W && y, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(M >= 0 && M < (1ll << 31) && N > 0 && K > 0, MSA_ERR_INVALID_ARG,
              "%s: bad shape M=%lld N=%d K=%d", name, (long long)M, N, K);
  MSA_REQUIRE(K % (w8 ? 64 : 32) == 0 && N % 16 == 0, MSA_ERR_INVALID_ARG,
              "%s: K=%d must be a multiple of %d and N=%d a multiple of 16", name, K, w8 ? 64 : 32,
              N);
  MSA_REQUIRE((M + TL_BM - 1) / TL_BM <= 65535, MSA_ERR_INVALID_ARG, "%s: M=%lld too large", name,
              (long long)M);
  MSA_REQUIRE((flags & ~allowed) == 0, MSA_ERR_INVALID_ARG, "%s: unsupported flags 0x%x", name,
              flags);
  MSA_REQUIRE(!(flags & (MSA_IN_PACKED | MSA_OUT_PACKED)) || M <= MSA_PACKED_MAX_ROWS,
              MSA_ERR_INVALID_ARG, "%s: packed activations exist only for M <= %d (M=%lld)", name,
              MSA_PACKED_MAX_ROWS, (long long)M);
  return MSA_OK;
}

template <bool W8>
int linear_entry(const char* name, const void* x, const void* W, const void* scales,
                 const void* bias, const void* residual, void* y, int64_t M, int N, int K,
                 unsigned flags, void* stream) {
  int rc = check_linear_args(name, x, W, y, M, N, K, W8, flags,
                             MSA_EPI_RELU | MSA_IN_PACKED | MSA_OUT_PACKED);
  if (rc) return rc;
  MSA_REQUIRE(!W8 || scales, MSA_ERR_INVALID_ARG, "%s: null scales", name);
  MSA_REQUIRE(!((flags & MSA_OUT_PACKED) && residual && residual == y), MSA_ERR_INVALID_ARG,
              "%s: a packed output cannot alias the row-major residual", name);
  if (M == 0) return MSA_OK;
  Epilogue e{};
  e.bias = (const half_t*)bias;
  e.residual = (const half_t*)residual;
  e.y = (half_t*)y;
  e.N = N;
  e.flags = flags & MSA_EPI_RELU;
  e.out_mb = (flags & MSA_OUT_PACKED) ? packed_row_blocks(M) : 0;
  if (flags & MSA_IN_PACKED)
    launch_stream<W8, MODE_PLAIN>(x, W, scales, nullptr, 1, (int)M, N, K, e, (hipStream_t)stream);
  else
    launch_tiled<W8, MODE_PLAIN>(x, W, scales, M, N, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

template <bool W8>
int partial_entry(const char* name, const void* x, const void* W, const void* scales, float* part,
                  int64_t M, int N, int K, int S, unsigned flags, void* stream) {
  int rc = check_linear_args(name, x, W, part, M, N, K, W8, flags, MSA_IN_PACKED);
  if (rc) return rc;
  MSA_REQUIRE(!W8 || scales, MSA_ERR_INVALID_ARG, "%s: null scales", name);
  if (!(flags & MSA_IN_PACKED)) {
    // row-major activations: the MFMA tile kernel over S equal K ranges
    MSA_REQUIRE(!W8, MSA_ERR_INVALID_ARG,
                "%s: partial sums of row-major activations exist for fp16 weights only (expand "
                "the int8 matrix with msa_expand_weight_w8_f16 first)", name);
    MSA_REQUIRE(M >= 1, MSA_ERR_INVALID_ARG, "%s: M=%lld", name, (long long)M);
    MSA_REQUIRE(S >= 1 && K % (64 * S) == 0 && K / S >= 128, MSA_ERR_INVALID_ARG,
                "%s: row-major activations need K=%d cut by S=%d into ranges that are multiples "
                "of 64 and at least 128", name, K, S);
    launch_quad_partial(x, W, part, M, N, K, S, (hipStream_t)stream);
    MSA_CHECK_LAUNCH(name);
    return MSA_OK;
  }
  MSA_REQUIRE(M >= 1 && M <= MSA_PACKED_MAX_ROWS, MSA_ERR_INVALID_ARG,
              "%s: packed activations need 1 <= M <= %d (M=%lld)", name, MSA_PACKED_MAX_ROWS,
              (long long)M);
  MSA_REQUIRE(S >= 1 && S <= K / (W8 ? 64 : 32), MSA_ERR_INVALID_ARG,
              "%s: S=%d outside 1..%d", name, S, K / (W8 ? 64 : 32));
  {
    // the ranges are ceil(steps / S) 32-wide steps each (an even count for int8): every one of
    // the S slices must get at least one step, or it would stay unwritten
    const int nks = K / 32;
    int per = (nks + S - 1) / S;
    if (W8) per = (per + 1) & ~1;
    MSA_REQUIRE((int64_t)(S - 1) * per < nks, MSA_ERR_INVALID_ARG,
                "%s: S=%d leaves a K range empty (K=%d is cut into ranges of %d elements)", name, S,
                K, per * 32);
  }
  Epilogue e{};
  launch_stream<W8, MODE_PLAIN>(x, W, scales, part, S, (int)M, N, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

template <bool W8>
int qkv_entry(const char* name, const void* x, const void* W, const void* scales, const void* bqkv,
              void* q_out, void* Kc, void* Vc, int B, int T, int H, int hd, int S0, int S_cap,
              int K, unsigned flags, const int32_t* len_dev, void* stream) {
  MSA_REQUIRE(!len_dev || T == 1, MSA_ERR_INVALID_ARG, "%s: a device-side length needs T == 1",
              name);
  MSA_REQUIRE(q_out && Kc && Vc, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(B > 0 && T > 0 && H > 0 && hd > 0 && hd % 8 == 0 && S0 >= 0, MSA_ERR_INVALID_ARG,
              "%s: bad shape B=%d T=%d H=%d hd=%d S0=%d", name, B, T, H, hd, S0);
  MSA_REQUIRE((int64_t)S0 + T <= S_cap, MSA_ERR_CAPACITY,
              "%s: S0 + T = %d exceeds the cache capacity %d", name, S0 + T, S_cap);
  const int64_t M = (int64_t)B * T;
  const int N = 3 * H * hd;
  int rc = check_linear_args(name, x, W, q_out, M, N, K, W8, flags, MSA_IN_PACKED);
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
  e.hd_shift = (hd & (hd - 1)) == 0 ? __builtin_ctz((unsigned)hd) : -1;
  e.S0 = S0;
  e.len_dev = len_dev;
  e.S_cap = S_cap;
  e.qscale = (float)pow((double)hd, -0.5);  // the reference's head_dim ** -0.5, cast to fp32
  if (flags & MSA_IN_PACKED)
    launch_stream<W8, MODE_QKV>(x, W, scales, nullptr, 1, (int)M, N, K, e, (hipStream_t)stream);
  else
    launch_tiled<W8, MODE_QKV>(x, W, scales, M, N, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

int pack_entry(const char* name, const void* src, void* dst, int N, int K, bool i8, bool unpack,
               void* stream) {
  MSA_REQUIRE(src && dst && src != dst, MSA_ERR_INVALID_ARG, "%s: null or aliased pointers", name);
  MSA_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % (i8 ? 64 : 32) == 0, MSA_ERR_INVALID_ARG,
              "%s: N=%d must be a multiple of 16 and K=%d of %d", name, N, K, i8 ? 64 : 32);
  const int64_t pieces = (int64_t)N * K / 8;
  const dim3 grid((unsigned)((pieces + 255) / 256));
  if (i8)
    hipLaunchKernelGGL(pack_i8_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const int8_t*)src,
                       (int8_t*)dst, N, K, unpack);
  else
    hipLaunchKernelGGL(pack_f16_kernel, grid, dim3(256), 0, (hipStream_t)stream,
                       (const half_t*)src, (half_t*)dst, N, K, unpack);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}

}  // namespace

extern "C" int msa_pack_weight_f16(const void* src, void* dst, int N, int K, void* stream) {
  return pack_entry("msa_pack_weight_f16", src, dst, N, K, false, false, stream);
}
extern "C" int msa_unpack_weight_f16(const void* src, void* dst, int N, int K, void* stream) {
  return pack_entry("msa_unpack_weight_f16", src, dst, N, K, false, true, stream);
}
extern "C" int msa_pack_weight_i8(const int8_t* src, int8_t* dst, int N, int K, void* stream) {
  return pack_entry("msa_pack_weight_i8", src, dst, N, K, true, false, stream);
}
extern "C" int msa_unpack_weight_i8(const int8_t* src, int8_t* dst, int N, int K, void* stream) {
  return pack_entry("msa_unpack_weight_i8", src, dst, N, K, true, true, stream);
}

extern "C" int msa_expand_weight_w8_f16(const int8_t* Wq, const void* scales, void* Wp, int N,
                                        int K, void* stream) {
  MSA_REQUIRE(Wq && scales && Wp && (const void*)Wq != Wp, MSA_ERR_INVALID_ARG,
              "msa_expand_weight_w8_f16: null or aliased pointers");
  MSA_REQUIRE(N > 0 && K > 0 && N % 16 == 0 && K % 64 == 0, MSA_ERR_INVALID_ARG,
              "msa_expand_weight_w8_f16: N=%d must be a multiple of 16 and K=%d of 64", N, K);
  const int64_t n = (int64_t)N * K / 16;
  hipLaunchKernelGGL(expand_w8_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, (const uint8_t*)Wq, (const half_t*)scales, (half_t*)Wp,
                     N, K);
  MSA_CHECK_LAUNCH("msa_expand_weight_w8_f16");
  return MSA_OK;
}

extern "C" int64_t msa_lm_head_select_workspace_bytes(int M) {
  // one partial per row and workgroup; the streaming kernel never launches more workgroups
  // than there are compute units
  return (int64_t)(M > 0 ? M : 0) * num_cus() * (int64_t)sizeof(SelectPartial);
}

namespace {
int lm_head_select_impl(const char* name, const void* x, const void* Ep, void* logits,
                        void* workspace, int M, int V, int K, float temperature,
                        const int32_t* banned_host, int n_banned, const int32_t* stop_host,
                        int n_stop, uint8_t* finished, const uint8_t* row_mode, int force_eos_all,
                        int eos_idx, int64_t* tok, int64_t tok_stride, float* score,
                        int64_t score_stride, const int32_t* len_dev, void* stream) {
  MSA_REQUIRE(x && Ep && workspace && tok && score, MSA_ERR_INVALID_ARG, "%s: null pointer", name);
  MSA_REQUIRE(M >= 1 && M <= 64 && V > 0 && V % 16 == 0 && K > 0 && K % 32 == 0,
              MSA_ERR_INVALID_ARG, "%s: bad shape M=%d V=%d K=%d (1 <= M <= 64, V %% 16, K %% 32)",
              name, M, V, K);
  MSA_REQUIRE(n_banned >= 0 && n_banned <= 16 && (n_banned == 0 || banned_host),
              MSA_ERR_INVALID_ARG, "%s: n_banned=%d (0..16)", name, n_banned);
  MSA_REQUIRE(n_stop >= 0 && n_stop <= 15 && (n_stop == 0 || stop_host), MSA_ERR_INVALID_ARG,
              "%s: n_stop=%d (0..15)", name, n_stop);
  MSA_REQUIRE(eos_idx >= 0 && eos_idx < V, MSA_ERR_INVALID_ARG,
              "%s: eos_idx=%d outside the vocabulary", name, eos_idx);
  MSA_REQUIRE(temperature >= 0.f, MSA_ERR_INVALID_ARG, "%s: temperature < 0", name);
  Epilogue e{};
  e.y = (half_t*)logits;
  e.N = V;
  e.partials = (SelectPartial*)workspace;
  e.finished = finished;
  e.row_mode = row_mode;
  e.early.n = 1 + n_stop;
  e.early.id[0] = eos_idx;
  for (int i = 0; i < n_stop; ++i) e.early.id[1 + i] = stop_host[i];
  e.banned.n = n_banned;
  for (int i = 0; i < n_banned; ++i) e.banned.id[i] = banned_host[i];
  e.temperature = temperature;
  e.scale = temperature > 0.f && temperature != 1.0f;
  e.force_eos_all = force_eos_all;
  e.eos = eos_idx;
  IdList stop{};
  stop.n = n_stop;
  for (int i = 0; i < n_stop; ++i) stop.id[i] = stop_host[i];
  // same decomposition as launch_stream_mb at S = 1: the partial stride is its grid size
  const int ntiles = V / 16;
  const int tiles_per_wg = (ntiles + num_cus() - 1) / num_cus();
  const int gx = (ntiles + tiles_per_wg - 1) / tiles_per_wg;
  launch_stream<false, MODE_SELECT>(x, Ep, nullptr, nullptr, 1, M, V, K, e, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  msa_launch_select_combine((const SelectPartial*)workspace, gx, M, stop, finished, eos_idx, tok,
                            tok_stride, score, score_stride, len_dev, (hipStream_t)stream);
  MSA_CHECK_LAUNCH(name);
  return MSA_OK;
}
}  // namespace

extern "C" int msa_lm_head_greedy_select_f16(
    const void* x, const void* Ep, void* logits, void* workspace, int M, int V, int K,
    float temperature, const int32_t* banned_host, int n_banned, const int32_t* stop_host,
    int n_stop, uint8_t* finished, const uint8_t* row_mode, int force_eos_all, int eos_idx,
    int64_t* tok, int64_t tok_stride, float* score, int64_t score_stride, const int32_t* len_dev,
    void* stream) {
  return lm_head_select_impl("msa_lm_head_greedy_select_f16", x, Ep, logits, workspace, M, V, K,
                             temperature, banned_host, n_banned, stop_host, n_stop, finished,
                             row_mode, force_eos_all, eos_idx, tok, tok_stride, score,
                             score_stride, len_dev, stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// The per-row, per-workgroup selection partials of the fused vocabulary projection live in a
// fixed device array instead of a caller-provided workspace, for callers that cannot allocate
// device memory (code under graph capture, serving loops, harnesses that forbid it).  Every
// GPU the library runs on holds its own copy of the array (512 KiB) until the process ends.
// In host code the array's name is only a stand-in for the symbol: the address the kernels get
// is looked up once per device with hipGetSymbolAddress and kept in g_scratch_ptr.
constexpr int NA_MAX_ROWS = 64;    // activation rows
constexpr int NA_MAX_PARTS = 256;  // workgroups of the projection = partials per row
static __device__ __align__(256) unsigned char
    scratch[NA_MAX_ROWS * NA_MAX_PARTS * sizeof(SelectPartial)];

namespace {
constexpr int NA_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[NA_MAX_DEVICES] = {};

// the current device's copy of `scratch`; NULL (with the error text set) on failure
void* scratch_for_current_device(const char* name) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= NA_MAX_DEVICES) {
    msa_set_error("%s: no usable current device (%s, device %d)", name, hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      msa_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", name, dev,
                    hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int msa_lm_head_greedy_select_noalloc_f16(
    const void* x, const void* Ep, void* logits, int M, int V, int K, float temperature,
    const int32_t* banned_host, int n_banned, const int32_t* stop_host, int n_stop,
    uint8_t* finished, const uint8_t* row_mode, int force_eos_all, int eos_idx, int64_t* tok,
    int64_t tok_stride, float* score, int64_t score_stride, const int32_t* len_dev, void* stream) {
  const char* name = "msa_lm_head_greedy_select_noalloc_f16";
  MSA_REQUIRE(M >= 1 && M <= NA_MAX_ROWS, MSA_ERR_CAPACITY,
              "%s: M=%d rows exceed the %d the fixed scratch array holds", name, M, NA_MAX_ROWS);
  MSA_REQUIRE(num_cus() <= NA_MAX_PARTS, MSA_ERR_CAPACITY,
              "%s: %d compute units exceed the %d partials per row the fixed scratch array holds",
              name, num_cus(), NA_MAX_PARTS);
  void* ws = scratch_for_current_device(name);
  if (!ws) return MSA_ERR_HIP;
  // every partial the combine kernel reads is written by the projection of the same call, so
  // nothing in the array has to start at zero
  return lm_head_select_impl(name, x, Ep, logits, ws, M, V, K, temperature, banned_host, n_banned,
                             stop_host, n_stop, finished, row_mode, force_eos_all, eos_idx, tok,
                             tok_stride, score, score_stride, len_dev, stream);
}

namespace {
// Split count that minimises what one workgroup moves through its L1: its weight tiles over
// its K range, the activation fragments of that K range once per tile group, and its fp32
// partial sums (written here, read back by the LayerNorm tail).  More splits mean more tiles
// per workgroup over a shorter K range, i.e. fewer activation bytes per weight byte.
int pick_splits(int64_t M, int N, int K, int wbytes) {
  if (M < 1 || M > MSA_PACKED_MAX_ROWS || N % 16 || K % 64) return 1;
  const int MB = packed_row_blocks(M), ntiles = N / 16, nks = K / 32;
  // tiles that share one sweep over the activations (int8 has a 2 x 6 x 3 shape of the
  // shared-activation kernel for up to 18), and K steps per stage of the workgroup
  const int NT = MB > 2 ? (wbytes == 1 && MB <= 4 ? SH_GROUP_W8 : SH_GROUP) : ST_NT;
  const int stage = MB > 2 ? 16 : ST_KG * 4;
  int best = 1;
  double best_cost = 0;
  for (int S = 1; S <= 8; S *= 2) {
    const int G = num_cus() / S;
    if (G < 1 || nks / S < stage) break;  // every wave needs a full stage of K steps
    const int tpw = (ntiles + G - 1) / G;
    const int groups = (tpw + NT - 1) / NT;
    const double Ks = (double)K / S;
    double cost = tpw * 16.0 * Ks * wbytes + groups * MB * 16.0 * Ks * 2 + 2.0 * tpw * 16 * M * 4;
    cost *= 1.0 + 0.02 * S;  // ties go to fewer splits (fewer partial slices to sum)
    if (S == 1 || cost < best_cost) {
      best = S;
      best_cost = cost;
    }
  }
  return best;
}
}  // namespace

extern "C" int msa_linear_default_splits(int64_t M, int N, int K) {
  return pick_splits(M, N, K, 2);
}

extern "C" int msa_linear_default_splits_w8a16(int64_t M, int N, int K) {
  return pick_splits(M, N, K, 1);
}

extern "C" int msa_linear_default_splits_rows(int64_t M, int N, int K) {
  return pick_row_splits(M, N, K);
}

extern "C" int msa_linear_f16(const void* x, const void* Wp, const void* bias,
                              const void* residual, void* y, int64_t M, int N, int K,
                              unsigned flags, void* stream) {
  return linear_entry<false>("msa_linear_f16", x, Wp, nullptr, bias, residual, y, M, N, K, flags,
                             stream);
}

extern "C" int msa_linear_w8a16(const void* x, const int8_t* Wq, const void* scales,
                                const void* bias, const void* residual, void* y, int64_t M, int N,
                                int K, unsigned flags, void* stream) {
  return linear_entry<true>("msa_linear_w8a16", x, Wq, scales, bias, residual, y, M, N, K, flags,
                            stream);
}

extern "C" int msa_linear_partial_f16(const void* x, const void* Wp, float* part, int64_t M, int N,
                                      int K, int S, unsigned flags, void* stream) {
  return partial_entry<false>("msa_linear_partial_f16", x, Wp, nullptr, part, M, N, K, S, flags,
                              stream);
}

extern "C" int msa_linear_partial_w8a16(const void* x, const int8_t* Wq, const void* scales,
                                        float* part, int64_t M, int N, int K, int S,
                                        unsigned flags, void* stream) {
  return partial_entry<true>("msa_linear_partial_w8a16", x, Wq, scales, part, M, N, K, S, flags,
                             stream);
}

extern "C" int msa_qkv_proj_f16(const void* x, const void* Wqkv, const void* bqkv, void* q_out,
                                void* Kcache, void* Vcache, int B, int T, int H, int hd, int S0,
                                int S_cap, int K, unsigned flags, const int32_t* len_dev,
                                void* stream) {
  return qkv_entry<false>("msa_qkv_proj_f16", x, Wqkv, nullptr, bqkv, q_out, Kcache, Vcache, B, T,
                          H, hd, S0, S_cap, K, flags, len_dev, stream);
}

extern "C" int msa_qkv_proj_w8a16(const void* x, const int8_t* Wq, const void* scales,
                                  const void* bqkv, void* q_out, void* Kcache, void* Vcache, int B,
                                  int T, int H, int hd, int S0, int S_cap, int K, unsigned flags,
                                  const int32_t* len_dev, void* stream) {
  return qkv_entry<true>("msa_qkv_proj_w8a16", x, Wq, scales, bqkv, q_out, Kcache, Vcache, B, T, H,
                         hd, S0, S_cap, K, flags, len_dev, stream);
}
