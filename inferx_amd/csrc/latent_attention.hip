// Attention over a compressed cache: per token ONE row [c | kr] is kept, c a latent of `rank` numbers from which
// every head's keys and values are linear maps (k_h = Wuk_h c, v_h = Wuv_h c), kr a rotated key part of `rot_dim`
// numbers that all heads share.  The maps are moved to the query's side, so that the cache is read as it is:
//
//     score_h[i, j] = (ql_h[i] . c[j] + qr_h[i] . kr[j]) * scale,   ql_h = Wuk_h^T q_h        (a product before)
//     ol_h[i]       = sum_j softmax_j(score_h[i, .]) c[j],           o_h = Wuv_h ol_h          (a product after)
//
// which is attention with one key/value head whose values are the first `rank` numbers of its keys.  Scores,
// softmax and the weighted sum are float32.
#include "common.h"

// ---------------------------------------------------------------------------
// Per token: rotate the rotated part of every query head in place, normalise the latent (RMS norm with a weight,
// float32), rotate the shared key part, and write [c | kr] to the token's row of the paged cache.
//   q        rows of heads x q_dim numbers, q_stride apart; the last rot_dim of each head are the rotated part
//   dkv      [T, >= rank + rot_dim] rows (may be strided)
//   cos_sin  float32 [T, pairs, 2]: element 2i of a rotated part is paired with 2i + 1, i < pairs; the rest passes
//   cache    [pages * page_size, rank + rot_dim]; slots[t] is the token's row
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(T* __restrict__ q, int64_t q_stride, const T* __restrict__ dkv, int64_t dkv_stride,
                      const void* __restrict__ norm_w, int nw_dtype, float eps, const float* __restrict__ cos_sin,
                      int pairs, const int32_t* __restrict__ slots, T* __restrict__ cache, int heads, int q_dim,
                      int rot_dim, int rank) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const float* cs = cos_sin ? cos_sin + t * pairs * 2 : nullptr;
  // the queries' rotated parts
  for (int i = tid; i < heads * pairs; i += blockDim.x) {
    const int h = i / pairs, p = i - h * pairs;
    T* at = q + t * q_stride + h * q_dim + (q_dim - rot_dim) + 2 * p;
    const float u = ix_load(at), v = ix_load(at + 1), c = cs[2 * p], s = cs[2 * p + 1];
    ix_store(at, u * c - v * s);
    ix_store(at + 1, v * c + u * s);
  }
  const T* row = dkv + t * dkv_stride;
  T* dst = slots ? cache + static_cast<int64_t>(slots[t]) * (rank + rot_dim) : nullptr;
  float ss = 0.f;
  for (int i = tid; i < rank; i += blockDim.x) {
    const float x = ix_load(row + i);
    ss += x * x;
  }
  ss = ix_block_sum(ss, red);
  if (!dst) return;
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(rank) + eps);
  for (int i = tid; i < rank; i += blockDim.x)
    ix_store(dst + i, ix_load(row + i) * inv * ix_load_rt(norm_w, nw_dtype, i));
  for (int p = tid; p < rot_dim / 2 + (rot_dim & 1); p += blockDim.x) {
    const int i = 2 * p;
    const float u = ix_load(row + rank + i);
    if (p < pairs) {
      const float v = ix_load(row + rank + i + 1), c = cs[2 * p], s = cs[2 * p + 1];
      ix_store(dst + rank + i, u * c - v * s);
      ix_store(dst + rank + i + 1, v * c + u * s);
    } else {
      ix_store(dst + rank + i, u);
      if (i + 1 < rot_dim) ix_store(dst + rank + i + 1, ix_load(row + rank + i + 1));
    }
  }
}

extern "C" int ix_latent_prepare(void* q, int64_t q_stride, const void* dkv, int64_t dkv_stride, int dtype, const void* norm_w,
                                 int nw_dtype, float eps, const float* cos_sin, int pairs, const int32_t* slots,
                                 void* cache, int64_t tokens, int heads, int q_dim, int rot_dim, int rank,
                                 hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && rank > 0 && rot_dim >= 0 && q_dim >= rot_dim, "sizes must be positive");
  IX_REQUIRE(pairs >= 0 && 2 * pairs <= rot_dim && (pairs == 0 || cos_sin != nullptr),
             "the rotated pairs must fit into the rotated part");
  if (tokens == 0) return 0;
  dim3 grid(static_cast<unsigned>(tokens)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, (float*)q, q_stride, (const float*)dkv, dkv_stride,
                       norm_w, nw_dtype, eps, cos_sin, pairs, slots, (float*)cache, heads, q_dim, rot_dim, rank);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)q, q_stride, (const bf16_t*)dkv,
                       dkv_stride, norm_w, nw_dtype, eps, cos_sin, pairs, slots, (bf16_t*)cache, heads, q_dim, rot_dim,
                       rank);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_latent_prepare");
}

// ---------------------------------------------------------------------------
// The plain kernel: one workgroup per (query token, head), softmax kept online over chunks of 256 keys.  Any
// element type and sizes (rank + rot_dim up to 1088, rank up to 1024); the float32 run uses it throughout.
//   ql   element (t, h, i) at ql[t * ql_t + h * ql_h + i], i < rank       (the query moved to the latent's side)
//   qr   element (t, h, i) at qr[t * qr_t + h * qr_h + i], i < rot_dim    (its rotated part)
//   out  element (t, h, i) at out[t * out_t + h * out_h + i], i < rank
#define LAT_THREADS 256
#define LAT_MAX_WIDTH 1088
#define LAT_ACC 4

template <typename T>
__global__ void __launch_bounds__(LAT_THREADS)
latent_attn_plain_kernel(const T* __restrict__ ql, int64_t ql_t, int64_t ql_h, const T* __restrict__ qr, int64_t qr_t,
                         int64_t qr_h, const T* __restrict__ cache, const int32_t* __restrict__ block_table,
                         const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ positions,
                         T* __restrict__ out, int64_t out_t, int64_t out_h, int rank, int rot_dim, int page_size,
                         int max_blocks, float scale) {
  __shared__ float qs[LAT_MAX_WIDTH];
  __shared__ float sc[LAT_THREADS];
  __shared__ int64_t at[LAT_THREADS];
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int head = blockIdx.y, tid = threadIdx.x;
  const int width = rank + rot_dim;
  const int64_t seq = seq_of_token[t];
  const int pos = positions[t];
  const int32_t* table = block_table + seq * max_blocks;
  for (int i = tid; i < width; i += LAT_THREADS)
    qs[i] = i < rank ? ix_load(ql + t * ql_t + head * ql_h + i) : ix_load(qr + t * qr_t + head * qr_h + (i - rank));
  __syncthreads();
  float m = -INFINITY, l = 0.f, acc[LAT_ACC] = {0.f, 0.f, 0.f, 0.f};
  for (int base = 0; base <= pos; base += LAT_THREADS) {
    const int j = base + tid;
    const bool live = j <= pos;
    float s = -INFINITY;
    int64_t row = 0;
    if (live) {
      row = (static_cast<int64_t>(table[j / page_size]) * page_size + j % page_size) * width;
      const T* kr = cache + row;
      float dot = 0.f;
      for (int i = 0; i < width; ++i) dot += qs[i] * ix_load(kr + i);
      s = dot * scale;
    }
    at[tid] = row;
    const float m_new = fmaxf(m, ix_block_max(s, red));
    const float p = live ? expf(s - m_new) : 0.f;
    sc[tid] = p;
    const float chunk_sum = ix_block_sum(p, red);  // its barriers publish sc and at
    const float alpha = expf(m - m_new);
    l = l * alpha + chunk_sum;
    m = m_new;
    const int n = min(LAT_THREADS, pos + 1 - base);
#pragma unroll
    for (int a = 0; a < LAT_ACC; ++a) {
      const int c = tid + a * LAT_THREADS;
      if (c < rank) {
        float v = acc[a] * alpha;
        for (int jj = 0; jj < n; ++jj) v += sc[jj] * ix_load(cache + at[jj] + c);
        acc[a] = v;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < LAT_ACC; ++a) {
    const int c = tid + a * LAT_THREADS;
    if (c < rank) ix_store(out + t * out_t + head * out_h + c, acc[a] / l);
  }
}

extern "C" int ix_latent_attention_plain(const void* ql, int64_t ql_t, int64_t ql_h, const void* qr, int64_t qr_t,
                                         int64_t qr_h, const void* cache, int dtype, const int32_t* block_table,
                                         const int32_t* seq_of_token, const int32_t* positions, void* out,
                                         int64_t out_t, int64_t out_h, int64_t tokens, int heads, int rank,
                                         int rot_dim, int page_size, int max_blocks, float scale,
                                         hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && rank > 0 && rot_dim >= 0 && page_size > 0 && max_blocks > 0,
             "sizes must be positive");
  IX_REQUIRE(rank <= LAT_ACC * LAT_THREADS && rank + rot_dim <= LAT_MAX_WIDTH,
             "the latent holds at most 1024 numbers, with the rotated part at most 1088");
  IX_REQUIRE(heads < 65536, "too many heads for one launch");
  if (tokens == 0) return 0;
  dim3 grid(static_cast<unsigned>(tokens), heads), block(LAT_THREADS);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(latent_attn_plain_kernel<float>, grid, block, 0, stream, (const float*)ql, ql_t, ql_h,
                       (const float*)qr, qr_t, qr_h, (const float*)cache, block_table, seq_of_token, positions,
                       (float*)out, out_t, out_h, rank, rot_dim, page_size, max_blocks, scale);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(latent_attn_plain_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)ql, ql_t, ql_h,
                       (const bf16_t*)qr, qr_t, qr_h, (const bf16_t*)cache, block_table, seq_of_token, positions,
                       (bf16_t*)out, out_t, out_h, rank, rot_dim, page_size, max_blocks, scale);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_latent_attention_plain");
}
