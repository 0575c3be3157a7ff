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
// layout of O^T = V^T * P^T.
//
// K and V tiles (64 keys) go global -> LDS directly (global_load_lds_dwordx4: the LDS address is
// M0 + 16 * lane, the lane's global address is free), row-major as the cache holds them, with the
// 16-byte chunks of a row XOR-swizzled so that the fragment reads are conflict free; no staging
// registers, no LDS stores, one barrier per tile.  The A operand of S^T (8 consecutive d of one
// key) is one 128-bit read.  The A operand of O^T needs 8 keys of one d, a column of the
// row-major tile: ds_read_b64_tr_b16 delivers it (within 16 lanes, lane 4 r + c loads 4
// consecutive d of key r; lane i then receives element i % 4 of the loads of lanes i / 4,
// 4 + i / 4, 8 + i / 4, 12 + i / 4, i.e. 4 consecutive keys of d = i), two reads per MFMA.
// Pass 1 keeps three K tiles in a ring (requests two tiles ahead), pass 2 two K and two V tiles.
#include <math.h>

#include "common.h"

namespace {

constexpr int PF_BM = 128;  // queries per workgroup
constexpr int PF_BN = 64;   // keys per tile
constexpr int PF_THREADS = 256;
typedef __fp16 pf_fp16x4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef __attribute__((address_space(3))) pf_fp16x4 pf_lds_fp16x4;
typedef __attribute__((address_space(3))) void pf_lds_void;

template <int HD>
__global__ __launch_bounds__(PF_THREADS) void prefill_attention_kernel(
    const half_t* __restrict__ q, const half_t* __restrict__ Kc, const half_t* __restrict__ Vc,
    const uint8_t* __restrict__ key_pad_mask, int64_t mask_stride, half_t* __restrict__ out,
    int BH, int n_qt, int grouped, int H, int T, int S0, int S_cap) {
  constexpr int KSTEPS = HD / 16;           // MFMA k steps over the head dimension
  constexpr int DBLK = HD / 32;             // 32-row blocks of O^T
  constexpr int ROWB = HD * 2;              // bytes of a key row
  constexpr int CH = HD / 8;                // 16-byte chunks of a key row
  constexpr int TILEB = PF_BN * ROWB;       // bytes of a tile
  constexpr int RPI = 1024 / ROWB;          // key rows per 1 KB load instruction
  constexpr int IPW = TILEB / 1024 / 4;     // load instructions per wave and tile
  __shared__ __attribute__((aligned(16))) char lds[4 * TILEB];

  // Workgroup -> (batch row and head, query tile).  Consecutive workgroups land on consecutive
  // XCDs, each with its own L2; all query tiles of one (row, head) share its K and V rows, so they
  // are given to one XCD, back to back (workgroups i, i + 8, i + 16, ...), the tile with the most
  // keys first: the rows are then fetched from memory once instead of once per query tile.
  // Small problems (all K and V rows fit the caches anyway) keep the plain order instead, every
  // (row, head)'s longest tile first, which balances the tail better.
  const int L = blockIdx.x;
  int bh, qt;
  if (grouped) {
    const int xcd = L & 7, seq = L >> 3;
    bh = (seq / n_qt) * 8 + xcd;
    qt = n_qt - 1 - seq % n_qt;
  } else {
    const int BHp = gridDim.x / n_qt;
    bh = L % BHp;
    qt = n_qt - 1 - L / BHp;
  }
  if (bh >= BH) return;  // the last group of 8 may be incomplete (uniform per workgroup)
  const int b = bh / H, h = bh - b * H;
  const int D = H * HD;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
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

  // chunk swizzles: K rows are read 16 keys at a time at one chunk index (swizzle by the key).
  // V rows are read by 32 lanes at a time as 4 keys x two neighbouring 32-byte chunk pairs: the
  // pair index is XORed with 2 * (key % 4), which sends the 8 pieces to the 8 pair positions of
  // the 256 bytes the banks span (128-byte rows: two rows span the banks, XOR with 2 * (key / 2 % 2))
  auto fk = [](int row) { return HD == 128 ? (row & 15) : ((row >> 1) & 7); };
  auto fv = [](int row) { return HD == 128 ? 4 * (row & 3) : 4 * ((row >> 1) & 1); };

  // direct loads: instruction u of this wave covers tile rows (IPW * wave + u) * RPI ..; lane l
  // lands at row l / CH, chunk position l % CH, which must hold chunk (l % CH) ^ f(row)
  const uint32_t lds0 = (uint32_t)(uintptr_t)(pf_lds_void*)lds;
  int drow[IPW];
  uint32_t kchunk[IPW], vchunk[IPW];
#pragma unroll
  for (int u = 0; u < IPW; ++u) {
    drow[u] = (wave * IPW + u) * RPI + lane / CH;
    kchunk[u] = ((lane % CH) ^ fk(drow[u])) * 16;
    vchunk[u] = ((lane % CH) ^ fv(drow[u])) * 16;
  }
  // keys past the last needed one repeat it (they are masked out below); a tile past the last
  // one loads that key 64 times, which keeps the number of loads in flight the same everywhere
  auto issue_tile = [&](const half_t* base, const uint32_t(&chunk)[IPW], int slot, int tile) {
#pragma unroll
    for (int u = 0; u < IPW; ++u) {
      const int key = min(tile * PF_BN + drow[u], n_keys - 1);
      const uint32_t vo = (uint32_t)key * ROWB + chunk[u];
      const uint32_t la = lds0 + slot * TILEB + (wave * IPW + u) * 1024;
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(vo), "s"(base),
                   "s"(la)
                   : "memory");
    }
  };
  // K fragment of step ks (block ib adds 32 rows): row j, chunk 2 ks + hl
  uint32_t kfo[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) kfo[ks] = j * ROWB + (((2 * ks + hl) ^ fk(j)) * 16);
  // V, this lane as a source of the transposing read: key row 4 * (lane / 32) + (lane % 16) / 4
  // of a 16-key step (+ 8 for the second read), d = 32 db + 16 * ((lane / 16) % 2) + 4 * (lane % 4)
  uint32_t vfo[DBLK];
  {
    const int g = lane >> 4, i = lane & 15;
    const int vrow = 4 * (g >> 1) + (i >> 2);
#pragma unroll
    for (int db = 0; db < DBLK; ++db) {
      const int chunk = 4 * db + 2 * (g & 1) + ((i & 3) >> 1);
      vfo[db] = vrow * ROWB + ((chunk ^ fv(vrow)) * 16) + (i & 1) * 8;
    }
  }

  // S^T tile of this wave: 64 keys x 32 queries = 2 accumulators, rounded to fp16, masked and kept
  // as packed pairs: pair v2 of block ib holds keys 32*ib + 8*(v2/2) + 4*hl + 2*(v2%2) + {0, 1}
  constexpr float LOG2E = 1.4426950408889634f;
  const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  half2_t sh[2][8];
  auto scores = [&](int tile, int slot) {
    const char* kt = lds + slot * TILEB;
    float16_t s[2];
    // the two key blocks alternate so that no MFMA waits for the one just issued; the first
    // step takes a literal zero as its addend (no accumulator clearing)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
      for (int ib = 0; ib < 2; ++ib) {
        const half8_t a = *reinterpret_cast<const half8_t*>(kt + ib * 32 * ROWB + kfo[ks]);
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
  issue_tile(kbase, kchunk, 0, 0);
  issue_tile(kbase, kchunk, 1, 1);
  for (int tile = 0, slot = 0; tile < ntiles; ++tile) {
    // all but this wave's newest IPW loads have landed: its part of this tile is there
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IPW) : "memory");
    __syncthreads();  // the tile is complete, and the slot of the previous tile is free
    issue_tile(kbase, kchunk, slot == 0 ? 2 : slot - 1, tile + 2);
    scores(tile, slot);
    slot = slot == 2 ? 0 : slot + 1;
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
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();  // pass 1's last loads have landed and its last tile is consumed
  issue_tile(kbase, kchunk, 0, 0);
  issue_tile(vbase, vchunk, 2, 0);
  for (int tile = 0; tile < ntiles; ++tile) {
    const int slot = tile & 1;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    issue_tile(kbase, kchunk, slot ^ 1, tile + 1);
    issue_tile(vbase, vchunk, 2 + (slot ^ 1), tile + 1);
    scores(tile, slot);
    const char* vt = lds + (2 + slot) * TILEB;
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
#pragma unroll
        for (int db = 0; db < DBLK; ++db) {
          const char* vp = vt + (ib * 32 + c * 16) * ROWB + vfo[db];
          typedef uint32_t u2 __attribute__((ext_vector_type(2)));
          typedef uint32_t u4 __attribute__((ext_vector_type(4)));
          const u2 lo = __builtin_bit_cast(
              u2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((pf_lds_fp16x4*)vp));
          const u2 hi = __builtin_bit_cast(
              u2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((pf_lds_fp16x4*)(vp + 8 * ROWB)));
          const u4 w = {lo[0], lo[1], hi[0], hi[1]};
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
  const int n_qt = (T + PF_BM - 1) / PF_BM, BH = B * H;
  const dim3 grid((unsigned)(((BH + 7) / 8) * 8 * n_qt));
  // K and V rows of all (row, head) pairs against the 32 MB of L2 + part of the memory-side cache
  const int grouped = (int64_t)BH * (S0 + T) * hd * 4 > (int64_t)64 * 1024 * 1024;
  if (hd == 64)
    hipLaunchKernelGGL(prefill_attention_kernel<64>, grid, dim3(PF_THREADS), 0, stream,
                       (const half_t*)q, (const half_t*)Kc, (const half_t*)Vc, key_pad_mask,
                       mask_stride, (half_t*)out, BH, n_qt, grouped, H, T, S0, S_cap);
  else
    hipLaunchKernelGGL(prefill_attention_kernel<128>, grid, dim3(PF_THREADS), 0, stream,
                       (const half_t*)q, (const half_t*)Kc, (const half_t*)Vc, key_pad_mask,
                       mask_stride, (half_t*)out, BH, n_qt, grouped, H, T, S0, S_cap);
  return 0;
}
