// Causal prefill attention on MFMA, flash-style (never materialises the T x S score matrix),
// with the reference's fp16 rounding points kept: scores are rounded to fp16 before the fp32
// softmax and the normalised probabilities are rounded to fp16 before they multiply V.
// Because the probabilities are rounded AFTER normalisation, the row maximum and sum must be
// final before the first p*v product: the kernel sweeps the keys twice, pass 1 for the
// softmax statistics (QK^T only), pass 2 recomputing the same scores (bit-identical MFMAs)
// and accumulating P*V.  QK^T runs twice, 1.5x the MFMA work of one-pass flash attention.
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
  const int q0 = qt * PF_BM + wave * 32;  // first query of this wave
  const int tq = q0 + j;                  // this lane's query
  const int tqc = tq < T ? tq : T - 1;
  const int pq = S0 + tq;                 // its position = last key it may see
  const int wg_last_q = min(T, qt * PF_BM + PF_BM) - 1;
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

  // S^T tile of this wave: 64 keys x 32 queries = 2 accumulators; rounded to fp16 and masked
  float16_t s[2];
  auto scores = [&](int tile) {
#pragma unroll
    for (int ib = 0; ib < 2; ++ib) {
#pragma unroll
      for (int v = 0; v < 16; ++v) s[ib][v] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        const half8_t a =
            *reinterpret_cast<const half8_t*>(&lk[(ib * 32 + j) * KLD + ks * 16 + hl * 8]);
        s[ib] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], s[ib], 0, 0, 0);
      }
    }
    const int kt0 = tile * PF_BN;
    const bool need_mask = (kt0 + PF_BN - 1 > S0 + q0) || mrow != nullptr;  // wave-uniform
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        float x = round_h(s[ib][v]);
        if (need_mask) {
          const int key = kt0 + ib * 32 + 8 * (v >> 2) + 4 * hl + (v & 3);
          if (key > pq || (mrow && mrow[key < n_keys ? key : n_keys - 1])) x = -INFINITY;
        }
        s[ib][v] = x;
      }
  };

  // ---------------- pass 1: row maximum and sum of exp ----------------
  float m = -INFINITY, l = 0.f;
  load_k(0);
  for (int tile = 0; tile < ntiles; ++tile) {
    __syncthreads();  // previous tile fully consumed
    store_k();
    __syncthreads();
    if (tile + 1 < ntiles) load_k(tile + 1);  // the branch also pins the loads ahead of the MFMAs
    scores(tile);
    float tm = -INFINITY;
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int v = 0; v < 16; ++v) tm = fmaxf(tm, s[ib][v]);
    tm = fmaxf(tm, __shfl_xor(tm, 32, MSA_WAVE));
    if (tm > -INFINITY) {
      const float mn = fmaxf(m, tm);
      float ts = 0.f;
#pragma unroll
      for (int ib = 0; ib < 2; ++ib)
#pragma unroll
        for (int v = 0; v < 16; ++v) ts += __expf(s[ib][v] - mn);  // -inf - finite = -inf -> 0
      ts += __shfl_xor(ts, 32, MSA_WAVE);
      l = l * __expf(m - mn) + ts;
      m = mn;
    }
  }
  const float inv_l = 1.0f / l;

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
    // exactly registers 8c .. 8c+7 of this lane, i.e. P^T is already a B operand
#pragma unroll
    for (int ib = 0; ib < 2; ++ib)
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        half8_t p;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          p[e] = (half_t)(__expf(s[ib][8 * c + e] - m) * inv_l);
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
  if (tq < T) {
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
