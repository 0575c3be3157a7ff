// Shared helpers for the gfx950 kernels: vector types, wave64 reductions, error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/metaseq_amd.h"

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

#define MSA_WAVE 64

void msa_set_error(const char* fmt, ...);

// MFMA flash-style causal attention for T > 1 new queries (attention_prefill.hip)
int msa_launch_prefill_attention(const void* q, const void* Kc, const void* Vc,
                                 const uint8_t* key_pad_mask, int64_t mask_stride, void* out,
                                 int B, int H, int hd, int T, int S0, int S_cap,
                                 hipStream_t stream);

#define MSA_REQUIRE(cond, code, ...) \
  do {                               \
    if (!(cond)) {                   \
      msa_set_error(__VA_ARGS__);    \
      return (code);                 \
    }                                \
  } while (0)

#define MSA_CHECK_LAUNCH(name)                                              \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      msa_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return MSA_ERR_HIP;                                                   \
    }                                                                       \
  } while (0)

// up to 16 token ids passed by value to a kernel (banned / stop lists of the generator)
struct IdList {
  int32_t n;
  int32_t id[16];
};

// Partial result of the greedy selection over a slice of one logits row: running log-sum-exp
// (max, sum of exp(z - max)) over every id, best eligible z with its id, NaN seen.
struct SelectPartial {
  float m, s, best;
  int32_t bidx;
  float nan;
  float pad[3];
};

int msa_launch_select_combine(const SelectPartial* partials, int n_parts, int B,
                              const IdList& stop, uint8_t* finished, int eos, int64_t* tok,
                              int64_t tok_stride, float* score, int64_t score_stride,
                              const int32_t* len_dev, hipStream_t stream);

// Packed activation layout for M <= 128 rows (the B operand of v_mfma_f32_16x16x32_f16, stored
// in lane order): element (m, k) of a [M, K] activation with MB row blocks lives at half offset
// ((k/32 * MB + m/16) * 64 + 16*((k%32)/8) + m%16) * 8 + k%8.  MB = ceil(M/16) up to 64 rows and
// 8 for 65 .. 128 rows (one kernel shape serves them all; the rows past M are never read back).
constexpr int MSA_PACKED_MAX_ROWS = 128;
__host__ __device__ __forceinline__ int packed_row_blocks(int64_t M) {
  return M <= 64 ? (int)((M + 15) / 16) : 8;
}
__host__ __device__ __forceinline__ int64_t packed_act_offset(int m, int k, int MB) {
  return ((((int64_t)(k >> 5) * MB + (m >> 4)) * 64 + (((k & 31) >> 3) << 4) + (m & 15)) << 3) +
         (k & 7);
}

// round-to-nearest-even fp32 -> fp16 -> fp32 (a "materialise in fp16" point)
__device__ __forceinline__ float round_h(float v) { return (float)(half_t)v; }

// (max, sum of exp(z - max)) pairs merge associatively: one pass over a row suffices
__device__ __forceinline__ void lse_merge(float& m, float& s, float om, float os) {
  if (om > m) {
    s = s * expf(m - om) + os;
    m = om;
  } else if (om > -INFINITY) {
    s += os * expf(om - m);
  }
}

// Cross-lane step of the wave reductions on the data-parallel-primitive path of the vector ALU
// (no LDS round trip).  Lanes of a row that ROW_MASK leaves out receive `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                         CTRL, ROW_MASK, 0xf, false));
}

// Reductions over the 64 lanes of a wave; every lane gets the result.  Order: pairs, quads,
// rows of 16 (two rotations), then the row totals are chained into lane 63 and broadcast.
// All 64 lanes must be active.
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1, 0xf>(0.f, v);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E, 0xf>(0.f, v);   // quad_perm [2,3,0,1]
  v += dpp_move<0x124, 0xf>(0.f, v);  // row_ror:4
  v += dpp_move<0x128, 0xf>(0.f, v);  // row_ror:8
  v += dpp_move<0x142, 0xa>(0.f, v);  // row_bcast15 into rows 1 and 3
  v += dpp_move<0x143, 0xc>(0.f, v);  // row_bcast31 into rows 2 and 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<0xB1, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x4E, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x124, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x128, 0xf>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x142, 0xa>(-INFINITY, v));
  v = fmaxf(v, dpp_move<0x143, 0xc>(-INFINITY, v));
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Block-wide reductions for blocks of up to 16 waves; `red` is >= 16 floats of LDS.
// All threads receive the result.  Contains barriers: call from uniform control flow.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  // all 16 slots are read at once (slots past nw hold stale values and are not added)
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float r = red[i];
    t += i < nw ? r : 0.f;
  }
  return t;
}

__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) {
    const float r = red[i];
    t = fmaxf(t, i < nw ? r : t);
  }
  return t;
}
