// Token + learned-position embedding.  Positions follow the reference's make_positions:
// pads keep pad_idx, every other token gets pad_idx + (number of non-pad tokens up to and
// including it).  Only the last T_out columns are embedded (T_out = 1 for a decode step).
#include "common.h"

namespace {

constexpr int EMB_THREADS = 256;

// number of non-pad tokens in row[0 .. upto) ; all threads get the result
__device__ __forceinline__ int count_nonpad(const int64_t* row, int upto, int pad, float* red) {
  int c = 0;
  for (int i = threadIdx.x; i < upto; i += blockDim.x) c += (row[i] != pad);
  // counts are < 2^24 so the float reduction is exact
  return (int)block_sum((float)c, red);
}

__device__ __forceinline__ void gather_row(const half_t* __restrict__ E,
                                           const half_t* __restrict__ P, int64_t tok, int pos,
                                           half_t* __restrict__ out, int D) {
  const half_t* e = E + tok * (int64_t)D;
  const half_t* p = P + (int64_t)pos * D;
  for (int i = threadIdx.x; i < (D >> 3); i += blockDim.x) {
    const half8_t a = *reinterpret_cast<const half8_t*>(e + (i << 3));
    const half8_t b = *reinterpret_cast<const half8_t*>(p + (i << 3));
    half8_t o;
#pragma unroll
    for (int k = 0; k < 8; ++k) o[k] = (half_t)((float)a[k] + (float)b[k]);
    *reinterpret_cast<half8_t*>(out + (i << 3)) = o;
  }
}

__device__ __forceinline__ void clamp_ids(int64_t& tok, int& pos, int V, int n_pos_rows,
                                          int32_t* status) {
  if (tok < 0 || tok >= V || pos >= n_pos_rows) {
    if (status && threadIdx.x == 0) *status = 1;
    tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
    pos = pos >= n_pos_rows ? n_pos_rows - 1 : pos;
  }
}

// decode step: one block per batch row, last token only.  With len_dev (per-row number of
// positions already in the KV cache = number of non-pad tokens before this one) the position
// comes from there instead of a scan over the row's history.
__global__ __launch_bounds__(EMB_THREADS) void embed_last_kernel(
    const int64_t* __restrict__ tokens, int64_t tok_stride, int n, const half_t* __restrict__ E,
    int V, const half_t* __restrict__ P, int n_pos_rows, int pad, int D, half_t* __restrict__ x,
    int64_t* __restrict__ positions_out, int32_t* status, const int32_t* __restrict__ len_dev,
    int32_t* __restrict__ step_len_out, bool col_from_len, bool rows_given) {
  __shared__ float red[16];
  const int b = blockIdx.x;
  const int64_t* row = tokens + b * tok_stride;
  int64_t tok;
  int pos = pad;
  if (len_dev) {
    const int raw = len_dev[b];
    const int len = max(raw, 0);  // an inactive row (negative) embeds as an empty one
    tok = row[col_from_len ? min(len, n - 1) : n - 1];
    if (tok != pad) pos = pad + 1 + len;
    // a pad as the new token leaves the row out of this step, like an inactive row
    if (step_len_out && threadIdx.x == 0) step_len_out[b] = (raw >= 0 && tok != pad) ? raw : -1;
  } else {
    tok = row[n - 1];
    const int cnt = count_nonpad(row, n, pad, red);
    if (tok != pad) pos = pad + cnt;
  }
  if (rows_given) tok = 0;  // E holds this row's token embedding itself: nothing to look up
  clamp_ids(tok, pos, V, n_pos_rows, status);
  if (positions_out && threadIdx.x == 0) positions_out[b] = pos;
  gather_row(E, P, rows_given ? (int64_t)b : tok, pos, x + (int64_t)b * D, D);
}

// prefill: positions for the last T_out columns of every row (one block per row)
__global__ __launch_bounds__(EMB_THREADS) void positions_kernel(
    const int64_t* __restrict__ tokens, int64_t tok_stride, int n, int T_out, int pad,
    int64_t* __restrict__ positions_out) {
  __shared__ int seg[EMB_THREADS];
  const int b = blockIdx.x;
  const int64_t* row = tokens + b * tok_stride;
  const int per = (n + EMB_THREADS - 1) / EMB_THREADS;
  const int lo = threadIdx.x * per, hi = min(n, lo + per);
  int c = 0;
  for (int i = lo; i < hi; ++i) c += (row[i] != pad);
  seg[threadIdx.x] = c;
  __syncthreads();
  int run = 0;
  for (int i = 0; i < (int)threadIdx.x; ++i) run += seg[i];
  const int first = n - T_out;
  for (int i = lo; i < hi; ++i) {
    const bool np = row[i] != pad;
    run += np;
    if (i >= first) positions_out[(int64_t)b * T_out + (i - first)] = np ? pad + run : pad;
  }
}

__global__ __launch_bounds__(EMB_THREADS) void embed_rows_kernel(
    const int64_t* __restrict__ tokens, int64_t tok_stride, int n, int T_out,
    const half_t* __restrict__ E, int V, const half_t* __restrict__ P, int n_pos_rows, int D,
    half_t* __restrict__ x, const int64_t* __restrict__ positions, int32_t* status,
    bool rows_given) {
  const int64_t r = blockIdx.x;  // b * T_out + j
  const int b = (int)(r / T_out), j = (int)(r % T_out);
  int64_t tok = rows_given ? 0 : tokens[b * tok_stride + (n - T_out + j)];
  int pos = (int)positions[r];
  clamp_ids(tok, pos, V, n_pos_rows, status);
  gather_row(E, P, rows_given ? r : tok, pos, x + r * D, D);
}

}  // namespace

extern "C" int msa_embed_f16(const int64_t* tokens, int64_t tok_stride, int B, int n, int T_out,
                             const void* E, int V, const void* P, int n_pos_rows, int pad_idx,
                             int D, void* x, int64_t* positions_out, int32_t* status_dev,
                             const int32_t* len_dev, int32_t* step_len_out, unsigned flags,
                             void* stream) {
  MSA_REQUIRE(tokens && E && P && x, MSA_ERR_INVALID_ARG, "msa_embed_f16: null pointer");
  MSA_REQUIRE(B > 0 && n > 0 && T_out > 0 && T_out <= n && tok_stride >= n, MSA_ERR_INVALID_ARG,
              "msa_embed_f16: bad shape B=%d n=%d T_out=%d stride=%lld", B, n, T_out,
              (long long)tok_stride);
  MSA_REQUIRE(D > 0 && D % 8 == 0 && V > 0 && n_pos_rows > pad_idx && pad_idx >= 0,
              MSA_ERR_INVALID_ARG, "msa_embed_f16: bad sizes D=%d V=%d n_pos_rows=%d pad=%d", D, V,
              n_pos_rows, pad_idx);
  MSA_REQUIRE(!len_dev || T_out == 1, MSA_ERR_INVALID_ARG,
              "msa_embed_f16: device-side lengths need T_out == 1");
  MSA_REQUIRE((flags & ~(MSA_EMBED_COL_FROM_LEN | MSA_EMBED_ROWS_GIVEN)) == 0 &&
                  (!(flags & MSA_EMBED_COL_FROM_LEN) || len_dev),
              MSA_ERR_INVALID_ARG,
              "msa_embed_f16: unsupported flags 0x%x (MSA_EMBED_COL_FROM_LEN needs len_dev)",
              flags);
  const bool rows_given = (flags & MSA_EMBED_ROWS_GIVEN) != 0;
  MSA_REQUIRE(!step_len_out || len_dev, MSA_ERR_INVALID_ARG,
              "msa_embed_f16: step_len_out needs len_dev");
  hipStream_t s = (hipStream_t)stream;
  if (T_out == 1) {
    hipLaunchKernelGGL(embed_last_kernel, dim3(B), dim3(EMB_THREADS), 0, s, tokens, tok_stride, n,
                       (const half_t*)E, V, (const half_t*)P, n_pos_rows, pad_idx, D, (half_t*)x,
                       positions_out, status_dev, len_dev, step_len_out,
                       (flags & MSA_EMBED_COL_FROM_LEN) != 0, rows_given);
  } else {
    MSA_REQUIRE(positions_out, MSA_ERR_INVALID_ARG,
                "msa_embed_f16: positions_out is required when T_out > 1");
    hipLaunchKernelGGL(positions_kernel, dim3(B), dim3(EMB_THREADS), 0, s, tokens, tok_stride, n,
                       T_out, pad_idx, positions_out);
    hipLaunchKernelGGL(embed_rows_kernel, dim3((unsigned)((int64_t)B * T_out)), dim3(EMB_THREADS),
                       0, s, tokens, tok_stride, n, T_out, (const half_t*)E, V, (const half_t*)P,
                       n_pos_rows, D, (half_t*)x, positions_out, status_dev, rows_given);
  }
  MSA_CHECK_LAUNCH("msa_embed_f16");
  return MSA_OK;
}

namespace {
__global__ __launch_bounds__(64) void advance_len_kernel(int32_t* len_dev,
                                                         const int32_t* __restrict__ gate, int n,
                                                         int delta) {
  const int i = blockIdx.x * 64 + threadIdx.x;
  // inactive rows (negative) and rows the gate leaves out of this step stay as they are
  if (i < n && len_dev[i] >= 0 && (!gate || gate[i] >= 0)) len_dev[i] += delta;
}
}  // namespace

extern "C" int msa_advance_len(int32_t* len_dev, const int32_t* gate, int n, int delta,
                               void* stream) {
  MSA_REQUIRE(len_dev && n > 0, MSA_ERR_INVALID_ARG, "msa_advance_len: null pointer or n=%d", n);
  hipLaunchKernelGGL(advance_len_kernel, dim3((n + 63) / 64), dim3(64), 0, (hipStream_t)stream,
                     len_dev, gate, n, delta);
  MSA_CHECK_LAUNCH("msa_advance_len");
  return MSA_OK;
}
