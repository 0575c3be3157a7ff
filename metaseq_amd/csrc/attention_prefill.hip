// Causal prefill attention on MFMA, flash-style (never materialises the T x S score matrix),
// with the reference's fp16 rounding points kept: scores are rounded to fp16 before the fp32
// softmax and the normalised probabilities are rounded to fp16 before they multiply V.
// Because the probabilities are rounded AFTER normalisation, the row maximum and sum must be
// final before the first p*v product: the kernel sweeps the keys twice, pass 1 for the
// softmax statistics (QK^T only), pass 2 recomputing the same scores (bit-identical MFMAs)
// and accumulating P*V.  QK^T runs twice, 1.5x the MFMA work of one-pass flash attention.
//
// Query tiles are aligned to the END of the new positions: a ragged tile (T % 128 queries) comes
// first, where it sees the fewest keys (a prompt of 2^k tokens plus the leading EOS would
// otherwise spend a whole extra sweep over all keys on its single last query).
//
// Scores are kept as packed fp16 pairs (they are fp16 values at this point of the reference);
// the softmax reads them through mixed-precision FMAs: exp(s - m) / l is evaluated as
// exp2(s * log2(e) - (m * log2(e) + log2(l))), one FMA and one exp2 per element.
//
// Workgroup = 128 queries of one (batch row, head); 4 waves x 32 queries.  Everything is kept
// transposed so that softmax rows live in lanes: S^T = K * Q^T puts query j = lane & 31 in each
// lane with 16 keys in registers (plus the other half-wave), which is already the B-operand
// layout of O^T = V^T * P^T.  K tiles are staged row-major in LDS (A operand: 8 consecutive d
// per lane); V tiles are staged with key pairs interleaved ([key/2][d][2]) so that the A
// operand of the second product (8 keys of one d) is four conflict-free 32-bit LDS reads.
#include <math.h>

#include "common.h"

namespace {

constexpr int PF_BM = 128;  // queries per workgroup
constexpr int PF_BN = 64;   // keys per tile
constexpr int PF_THREADS = 256;

template <int HD>
__global__ __launch_bounds__(PF_THREADS) void prefill_attention_kernel(
    const half_t* __restrict__ q, const half_t* __restrict__ Kc, const half_t* __restrict__ Vc,
    const uint8_t* __restrict__ key_pad_mask, int64_t mask_stride, half_t* __restrict__ out,
    int H, int T, int S0, int S_cap) {
  constexpr int KSTEPS = HD / 16;  // MFMA k steps over the head dimension
  constexpr int DBLK = HD / 32;    // 32-row blocks of O^T
  constexpr int KLD = HD + 8;      // K tile row stride (halves)
  constexpr int VLD = HD + 16;     // V tile row stride (32-bit words, one word = a key pair)
  constexpr int PIECES = PF_BN * HD / 8 / PF_THREADS;  // 16-byte pieces per thread and tile
  __shared__ __attribute__((aligned(16))) half_t lk[PF_BN * KLD];
  __shared__ __attribute__((aligned(16))) uint32_t lv[(PF_BN / 2) * VLD];

  // query tiles are issued last-first: the tiles with the most keys start earliest
  const int bh = blockIdx.x, qt = gridDim.y - 1 - blockIdx.y;
  const int b = bh / H, h = bh - b * H;
  const int D = H * HD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 31, hl = lane >> 5;
  const int lead = (PF_BM - T % PF_BM) % PF_BM;   // queries missing from the first tile
  const int q0 = qt * PF_BM - lead + wave * 32;   // first query of this wave (may be negative)
  const int tq = q0 + j;                          // this lane's query
  const int tqc = tq < 0 ? 0 : tq;                // lanes before the first query repeat query 0
  const int pq = S0 + tqc;                        // its position = last key it may see
  const int wg_last_q = qt * PF_BM - lead + PF_BM - 1;
  const int n_keys = S0 + wg_last_q + 1;  // keys this workgroup needs
  const int ntiles = (n_keys + PF_BN - 1) / PF_BN;
  const half_t* kbase = Kc + (int64_t)bh * S_cap * HD;
  const half_t* vbase = Vc + (int64_t)bh * S_cap * HD;
  const uint8_t* mrow = key_pad_mask ? key_pad_mask + (int64_t)b * mask_stride : nullptr;

  // Q^T fragments (B operand): query j, 8 consecutive d at 16*ks + 8*hl
  half8_t qf[KSTEPS];
  {
    const half_t* qrow = q + ((int64_t)b * T + tqc) * D + h * HD + hl * 8;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
      qf[ks] = *reinterpret_cast<const half8_t*>(qrow + ks * 16);
  }

  // staging: piece c = tid + 256*i of a tile: key c / (HD/8), d offset 8*(c % (HD/8)).
  // V pieces are taken as key pairs: pair p = c / (HD/8) (c < PF_BN/2 * HD/8 per half), so a
  // thread loads the same d range of keys 2p and 2p+1 and writes them interleaved.
  half8_t rk[PIECES], rv[PIECES];
  auto load_k = [&](int tile) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int c = tid + PF_THREADS * i;
      int key = tile * PF_BN + c / (HD / 8);
      if (key >= n_keys) key = n_keys - 1;  // clamped rows are masked out below
      rk[i] = *reinterpret_cast<const half8_t*>(kbase + (int64_t)key * HD + (c % (HD / 8)) * 8);
    }
  };
  auto store_k = [&]() {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int c = tid + PF_THREADS * i;
      *reinterpret_cast<half8_t*>(&lk[(c / (HD / 8)) * KLD + (c % (HD / 8)) * 8]) = rk[i];
    }
  };
  // V: PIECES/2 pairs per thread; pair index pc = tid + 256*i, key pair pc / (HD/8)
  auto load_v = [&](int tile) {
#pragma unroll
    for (int i = 0; i < PIECES / 2; ++i) {
      const int pc = tid + PF_THREADS * i;
      const int kp = pc / (HD / 8), dcol = (pc % (HD / 8)) * 8;
      int k0 = tile * PF_BN + 2 * kp, k1 = k0 + 1;
      if (k0 >= n_keys) k0 = n_keys - 1;
      if (k1 >= n_keys) k1 = n_keys - 1;
      rv[2 * i] = *reinterpret_cast<const half8_t*>(vbase + (int64_t)k0 * HD + dcol);
      rv[2 * i + 1] = *reinterpret_cast<const half8_t*>(vbase + (int64_t)k1 * HD + dcol);
    }
  };
  auto store_v = [&]() {
#pragma unroll
    for (int i = 0; i < PIECES / 2; ++i) {
      const int pc = tid + PF_THREADS * i;
      const int kp = pc / (HD / 8), dcol = (pc % (HD / 8)) * 8;
      half8_t lo, hi;  // words d..d+3 and d+4..d+7, each word = (key 2p, key 2p+1)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[2 * e] = rv[2 * i][e];
        lo[2 * e + 1] = rv[2 * i + 1][e];
        hi[2 * e] = rv[2 * i][4 + e];
        hi[2 * e + 1] = rv[2 * i + 1][4 + e];
      }
      *reinterpret_cast<half8_t*>(&lv[kp * VLD + dcol]) = lo;
      *reinterpret_cast<half8_t*>(&lv[kp * VLD + dcol + 4]) = hi;
    }
  };

  // S^T tile of this wave: 64 keys x 32 queries = 2 accumulators, rounded to fp16, masked and kept
  // as packed pairs: pair v2 of block ib holds keys 32*ib + 8*(v2/2) + 4*hl + 2*(v2%2) + {0, 1}
  constexpr float LOG2E = 1.4426950408889634f;
  const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  half2_t sh[2][8];
  auto scores = [&](int tile) {
    float16_t s[2];
    // the two key blocks alternate so that no MFMA waits for the one just issued; the first
    // step takes a literal zero as its addend (no accumulator clearing)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
      for (int ib = 0; ib < 2; ++ib) {
        const half8_t a =
            *reinterpret_cast<const half8_t*>(&lk[(ib * 32 + j) * KLD + ks * 16 + hl * 8]);
        s[ib] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], ks == 0 ? zero16 : s[ib], 0, 0, 0);
      }
    }
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int v2 = 0; v2 < 8; ++v2)
        sh[ib][v2] = half2_t{(half_t)s[ib][2 * v2], (half_t)s[ib][2 * v2 + 1]};
    const int kt0 = tile * PF_BN;
    if (kt0 + PF_BN - 1 > S0 + max(q0, 0)) {  // wave-uniform: the tile reaches past a query's position
#pragma unroll
      for (int ib = 0; ib < 2; ++ib)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = kt0 + ib * 32 + 8 * (v >> 2) + 4 * hl + (v & 3);
          if (key > pq) sh[ib][v >> 1][v & 1] = (half_t)(-INFINITY);
        }
    }
    if (mrow != nullptr) {  // uniform: padded keys
#pragma unroll
      for (int ib = 0; ib < 2; ++ib)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = kt0 + ib * 32 + 8 * (v >> 2) + 4 * hl + (v & 3);
          if (mrow[key < n_keys ? key : n_keys - 1]) sh[ib][v >> 1][v & 1] = (half_t)(-INFINITY);
        }
    }
  };
  auto xor32 = [&](float v) { return __shfl_xor(v, 32, MSA_WAVE); };

  // ---------------- pass 1: row maximum and sum of exp ----------------
  float m = -INFINITY, l = 0.f;
  load_k(0);
  for (int tile = 0; tile < ntiles; ++tile) {
    __syncthreads();  // previous tile fully consumed
    store_k();
    __syncthreads();
    if (tile + 1 < ntiles) load_k(tile + 1);  // the branch also pins the loads ahead of the MFMAs
    scores(tile);
    half2_t t2 = sh[0][0];
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int v2 = 0; v2 < 8; ++v2) t2 = __builtin_elementwise_max(t2, sh[ib][v2]);
    float tm = fmaxf((float)t2[0], (float)t2[1]);
    tm = fmaxf(tm, xor32(tm));
    if (tm > -INFINITY) {
      const float mn = fmaxf(m, tm);
      const float c = mn * LOG2E;
      float t4[4] = {0.f, 0.f, 0.f, 0.f};  // four chains: the adds do not wait for each other
#pragma unroll
      for (int ib = 0; ib < 2; ++ib)
#pragma unroll
        for (int v2 = 0; v2 < 8; ++v2) {  // exp(s - mn); -inf gives 0
          t4[(2 * v2) & 3] += __builtin_amdgcn_exp2f(__builtin_fmaf((float)sh[ib][v2][0], LOG2E, -c));
          t4[(2 * v2 + 1) & 3] += __builtin_amdgcn_exp2f(__builtin_fmaf((float)sh[ib][v2][1], LOG2E, -c));
        }
      float ts = (t4[0] + t4[1]) + (t4[2] + t4[3]);
      ts += xor32(ts);
      l = l * __builtin_amdgcn_exp2f(m * LOG2E - c) + ts;
      m = mn;
    }
  }
  // exp(s - m) / l = exp2(s * log2(e) - c2)
  const float c2 = m * LOG2E + __builtin_amdgcn_logf(l);

  // ---------------- pass 2: O^T += V^T * P^T ----------------
  float16_t o[DBLK];
#pragma unroll
  for (int db = 0; db < DBLK; ++db)
#pragma unroll
    for (int v = 0; v < 16; ++v) o[db][v] = 0.f;
  load_k(0);
  load_v(0);
  for (int tile = 0; tile < ntiles; ++tile) {
    __syncthreads();
    store_k();
    store_v();
    __syncthreads();
    if (tile + 1 < ntiles) {
      load_k(tile + 1);
      load_v(tile + 1);
    }
    scores(tile);
    // k step c of S^T block ib covers keys 32*ib + 16*c + {4*hl + 0..3, 8 + 4*hl + 0..3}:
    // exactly pairs 4c .. 4c+3 of this lane, i.e. P^T is already a B operand
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        half8_t p;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const half2_t h = sh[ib][4 * c + e];
          p[2 * e] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf((float)h[0], LOG2E, -c2));
          p[2 * e + 1] = (half_t)__builtin_amdgcn_exp2f(__builtin_fmaf((float)h[1], LOG2E, -c2));
        }
        const int kp = (ib * 32 + c * 16 + 4 * hl) >> 1;  // first key pair of this lane's group
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          const int d = db * 32 + j;
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          u4 w;
          w[0] = lv[(kp + 0) * VLD + d];
          w[1] = lv[(kp + 1) * VLD + d];
          w[2] = lv[(kp + 4) * VLD + d];
          w[3] = lv[(kp + 5) * VLD + d];
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, w), p, o[db],
                                                         0, 0, 0);
        }
      }
  }
  // O^T accumulator: lane holds query j and d = 32*db + 8*blk + 4*hl + r
  if (tq >= 0) {
    half_t* orow = out + ((int64_t)b * T + tq) * D + h * HD;
#pragma unroll
    for (int db = 0; db < DBLK; ++db)
#pragma unroll
      for (int blk = 0; blk < 4; ++blk) {
        half4_t v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (half_t)o[db][4 * blk + r];
        *reinterpret_cast<half4_t*>(orow + db * 32 + blk * 8 + hl * 4) = v;
      }
  }
}

}  // namespace

int msa_launch_prefill_attention(const void* q, const void* Kc, const void* Vc,
                                 const uint8_t* key_pad_mask, int64_t mask_stride, void* out,
                                 int B, int H, int hd, int T, int S0, int S_cap,
                                 hipStream_t stream) {
  const dim3 grid((unsigned)(B * H), (unsigned)((T + PF_BM - 1) / PF_BM));
  if (hd == 64)
    hipLaunchKernelGGL(prefill_attention_kernel<64>, grid, dim3(PF_THREADS), 0, stream,
                       (const half_t*)q, (const half_t*)Kc, (const half_t*)Vc, key_pad_mask,
                       mask_stride, (half_t*)out, H, T, S0, S_cap);
  else
    hipLaunchKernelGGL(prefill_attention_kernel<128>, grid, dim3(PF_THREADS), 0, stream,
                       (const half_t*)q, (const half_t*)Kc, (const half_t*)Vc, key_pad_mask,
                       mask_stride, (half_t*)out, H, T, S0, S_cap);
  return 0;
}
