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
//            (`halves`: element i is paired with i + pairs instead, the first 2 * pairs numbers of the part)
//   cache    [pages * page_size, rank + rot_dim]; slots[t] is the token's row
template <typename T>
__global__ void __launch_bounds__(256)
latent_prepare_kernel(T* __restrict__ q, int64_t q_stride, const T* __restrict__ dkv, int64_t dkv_stride,
                      const void* __restrict__ norm_w, int nw_dtype, float eps, const float* __restrict__ cos_sin,
                      int pairs, const int32_t* __restrict__ slots, T* __restrict__ cache, int heads, int q_dim,
                      int rot_dim, int rank, int halves) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const float* cs = cos_sin ? cos_sin + t * pairs * 2 : nullptr;
  // the queries' rotated parts
  for (int i = tid; i < heads * pairs; i += blockDim.x) {
    const int h = i / pairs, p = i - h * pairs;
    T* at = q + t * q_stride + h * q_dim + (q_dim - rot_dim) + (halves ? p : 2 * p);
    T* with = at + (halves ? pairs : 1);
    const float u = ix_load(at), v = ix_load(with), c = cs[2 * p], s = cs[2 * p + 1];
    ix_store(at, u * c - v * s);
    ix_store(with, v * c + u * s);
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
  if (halves) {
    for (int i = tid; i < rot_dim; i += blockDim.x) {
      const float x = ix_load(row + rank + i);
      if (i < 2 * pairs) {
        const int p = i < pairs ? i : i - pairs;
        const float other = ix_load(row + rank + (i < pairs ? i + pairs : i - pairs)), c = cs[2 * p], s = cs[2 * p + 1];
        ix_store(dst + rank + i, i < pairs ? x * c - other * s : x * c + other * s);
      } else {
        ix_store(dst + rank + i, x);
      }
    }
    return;
  }
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
                                 void* cache, int64_t tokens, int heads, int q_dim, int rot_dim, int rank, int halves,
                                 hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && rank > 0 && rot_dim >= 0 && q_dim >= rot_dim, "sizes must be positive");
  IX_REQUIRE(pairs >= 0 && 2 * pairs <= rot_dim && (pairs == 0 || cos_sin != nullptr),
             "the rotated pairs must fit into the rotated part");
  if (tokens == 0) return 0;
  dim3 grid(static_cast<unsigned>(tokens)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, block, 0, stream, (float*)q, q_stride, (const float*)dkv, dkv_stride,
                       norm_w, nw_dtype, eps, cos_sin, pairs, slots, (float*)cache, heads, q_dim, rot_dim, rank, halves);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)q, q_stride, (const bf16_t*)dkv,
                       dkv_stride, norm_w, nw_dtype, eps, cos_sin, pairs, slots, (bf16_t*)cache, heads, q_dim, rot_dim,
                       rank, halves);
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
                         int max_blocks, float scale, int window) {
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
  // with a window W a query reads the keys pos + 1 - W .. pos only (pages before them may be gone)
  const int start = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  for (int base = start; base <= pos; base += LAT_THREADS) {
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
                                         int rot_dim, int page_size, int max_blocks, float scale, int window,
                                         hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && rank > 0 && rot_dim >= 0 && page_size > 0 && max_blocks > 0 && window >= 0,
             "sizes must be positive");
  IX_REQUIRE(rank <= LAT_ACC * LAT_THREADS && rank + rot_dim <= LAT_MAX_WIDTH,
             "the latent holds at most 1024 numbers, with the rotated part at most 1088");
  IX_REQUIRE(heads < 65536, "too many heads for one launch");
  if (tokens == 0) return 0;
  dim3 grid(static_cast<unsigned>(tokens), heads), block(LAT_THREADS);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(latent_attn_plain_kernel<float>, grid, block, 0, stream, (const float*)ql, ql_t, ql_h,
                       (const float*)qr, qr_t, qr_h, (const float*)cache, block_table, seq_of_token, positions,
                       (float*)out, out_t, out_h, rank, rot_dim, page_size, max_blocks, scale, window);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(latent_attn_plain_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)ql, ql_t, ql_h,
                       (const bf16_t*)qr, qr_t, qr_h, (const bf16_t*)cache, block_table, seq_of_token, positions,
                       (bf16_t*)out, out_t, out_h, rank, rot_dim, page_size, max_blocks, scale, window);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_latent_attention_plain");
}

// ---------------------------------------------------------------------------
// The same attention on the matrix cores (bfloat16; rank + rot_dim a multiple of 32 up to 576, rank a multiple of
// 16 up to 512).  All heads read the same cached rows, so a workgroup of four wavefronts shares them through LDS:
// 32 keys a round, the row [c | kr] as it is for the scores and the latent part once more transposed ([d][key])
// for the weighted sum, so that both products take their operands in 16-byte pieces:
//
//     S^T[key][column] = K[key][:] . Q[column][:]             (A = key rows, B = the column's query, in registers)
//     O^T[d][column]  += C^T[d][key] P^T[key][column]          (A = transposed latent rows, B = the weights)
//
// v_mfma_f32_16x16x32_bf16 leaves lane l with column l % 16 and rows 4 (l / 16) + i.  Row m of the first 16 keys
// of a round is key 8 (m / 4) + m % 4, of the second key 8 (m / 4) + 4 + m % 4, so a lane holds the scores of keys
// 8 (l / 16) .. + 7 of its column: the B operand of the second product as it stands.  Softmax online, float32, per
// column; a lane's accumulators all belong to its column, so rescaling is a multiplication by the lane's factor.
//
// What a column is: prompt portions (DEC false): a workgroup takes 16 consecutive rows of the step and four heads,
// a wavefront one head, a column one row.  Rows of several requests in a tile are worked request by request (the
// other rows' keys all masked: they change nothing).  One token per request (DEC true): a workgroup takes one token
// and one slice of its keys, a wavefront sixteen heads, a column one head; slices leave (max, sum, unnormalised
// sums) for `attn_combine_kernel`.  The next round's rows are on their way from memory while a round is multiplied.
typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 lat_bf16x4 __attribute__((ext_vector_type(4)));
typedef float lat_f32x4 __attribute__((ext_vector_type(4)));

#define LATM_KEYS 32
#define LATM_KPAD 8      // numbers between key rows in LDS (keeps 16-byte pieces aligned, spreads the banks)
#define LATM_VSTRIDE 40  // numbers per transposed row: 32 keys and 8 spare

template <int NW, int NR, bool DEC>  // rank + rot_dim <= 32 NW, rank <= 16 NR
__global__ void __launch_bounds__(256)
latent_attn_mfma_kernel(const __bf16* __restrict__ ql, int64_t ql_t, int64_t ql_h, const __bf16* __restrict__ qr,
                        int64_t qr_t, int64_t qr_h, const __bf16* __restrict__ cache,
                        const int32_t* __restrict__ block_table, const int32_t* __restrict__ seq_of_token,
                        const int32_t* __restrict__ positions, __bf16* __restrict__ out, int64_t out_t, int64_t out_h,
                        float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits, int tokens, int heads,
                        int rank, int rot_dim, int page_size, int max_blocks, float scale_log2, int n_tiles,
                        int window) {
  extern __shared__ __attribute__((aligned(16))) unsigned char latm_lds[];
  constexpr int NP = (4 * NW + 7) / 8;  // 16-byte pieces of a round's rows that a thread moves
  const int width = rank + rot_dim;
  const int kstride = ((width + 63) & ~63) + LATM_KPAD;
  // 16-byte piece p of key row r lies at place p ^ 4 for rows 8..15 and 24..31: the sixteen rows that one product
  // reads at one piece index (0-3, 8-11, 16-19, 24-27, or the four after each) then fall on all banks evenly
  auto key_place = [&](int r, int piece) { return r * kstride + ((piece ^ (((r >> 3) & 1) << 2)) << 3); };
  const int p8 = width / 8;
  const int nw = width / 32, nr = rank / 16;
  __bf16* k_s = reinterpret_cast<__bf16*>(latm_lds);  // [32][kstride]
  __bf16* vt_s = k_s + LATM_KEYS * kstride;            // [rank][LATM_VSTRIDE]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g = lane >> 4;
  int row, head, r0, r1;
  bool wave_on;
  if constexpr (DEC) {
    r0 = blockIdx.x;
    r1 = r0 + 1;
    row = r0;
    head = (blockIdx.y * 4 + wave) * 16 + n;
    wave_on = (blockIdx.y * 4 + wave) * 16 < heads;
  } else {
    // one row of workgroups, the tiles with the most keys first, a tile's groups of four heads side by side
    const int head_groups = (heads + 3) / 4;
    r0 = (n_tiles - 1 - static_cast<int>(blockIdx.x) / head_groups) * 16;
    r1 = min(r0 + 16, tokens);
    row = r0 + n;
    head = (static_cast<int>(blockIdx.x) % head_groups) * 4 + wave;
    wave_on = head < heads;
  }
  const bool col_ok = row < r1 && head < heads;

  lat_bf16x8 qf[NW];
#pragma unroll
  for (int s = 0; s < NW; ++s) {
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<__bf16>(0.f);
    if (s < nw && col_ok) {
      const int i = 32 * s + 8 * g;
      const __bf16* src = i < rank ? ql + row * ql_t + head * ql_h + i : qr + row * qr_t + head * qr_h + (i - rank);
      qf[s] = *reinterpret_cast<const lat_bf16x8*>(src);
    }
  }
  lat_f32x4 acc[NR];
#pragma unroll
  for (int d = 0; d < NR; ++d) acc[d] = lat_f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -1e30f, l = 0.f;
  const int ka0 = 8 * (n >> 2) + (n & 3), ka1 = ka0 + 4;  // the keys of this lane's rows of the two A operands

  int seg = r0;
  while (seg < r1) {  // (every decision in this loop is the same for the whole workgroup)
    const int seq = seq_of_token[seg];
    int end = seg + 1;
    if constexpr (!DEC)
      while (end < r1 && seq_of_token[end] == seq) ++end;
    int k_end = positions[end - 1] + 1;  // a request's rows come in the order of their positions
    // with a window W the first of these rows reads from key k_lo on, and no row reads an earlier one (whose page
    // may be gone); rounds start at multiples of their length
    const int k_lo = window > 0 ? max(positions[seg] + 1 - window, 0) : 0;
    int k_begin = k_lo & ~(LATM_KEYS - 1);
    if constexpr (DEC) {
      const int per = ((k_end - k_begin + n_splits - 1) / n_splits + LATM_KEYS - 1) & ~(LATM_KEYS - 1);
      k_begin += static_cast<int>(blockIdx.z) * per;
      k_end = min(k_end, k_begin + per);
    }
    const int my_pos = (col_ok && row >= seg && row < end) ? positions[row] : -1;
    const int my_lo = window > 0 ? my_pos - window : -1;  // the last key that this column does not read
    const int32_t* table = block_table + static_cast<int64_t>(seq) * max_blocks;

    uint4 st[NP];
    const int my_key = tid >> 3, my_sub = tid & 7;  // a thread moves pieces my_sub, my_sub + 8, .. of one key's row
    auto ask = [&](int k0) {
      const int j = k0 + my_key;
      const bool there = j < k_end && j >= k_lo;
      const int64_t at = there ? (static_cast<int64_t>(table[j / page_size]) * page_size + j % page_size) * width : 0;
#pragma unroll
      for (int u = 0; u < NP; ++u) {
        const int pc = my_sub + 8 * u;
        st[u] = uint4{0u, 0u, 0u, 0u};  // rows past the last key enter LDS as zeros
        if (there && pc < p8) st[u] = *reinterpret_cast<const uint4*>(cache + at + 8 * pc);
      }
    };
    auto put = [&]() {
#pragma unroll
      for (int u = 0; u < NP; ++u) {
        const int pc = my_sub + 8 * u;
        if (pc < p8) *reinterpret_cast<uint4*>(k_s + key_place(my_key, pc)) = st[u];
      }
    };
    // The latent part once more, transposed, from the rows in LDS: here neighbouring lanes take neighbouring keys of
    // the same eight numbers, so that their 2-byte writes fall side by side into a transposed row (lanes that
    // held neighbouring pieces of one key would all write to the same bank).
    auto turn = [&]() {
#pragma unroll
      for (int u = 0; u < (NR + 3) / 4; ++u) {
        const int id = u * 256 + tid;
        const int kk = id & (LATM_KEYS - 1), pc = id / LATM_KEYS;
        if (8 * pc < rank) {
          const uint4 x = *reinterpret_cast<const uint4*>(k_s + key_place(kk, pc));
          unsigned short* dst = reinterpret_cast<unsigned short*>(vt_s) + (8 * pc) * LATM_VSTRIDE + kk;
          const unsigned int w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            dst[(2 * e) * LATM_VSTRIDE] = static_cast<unsigned short>(w[e] & 0xffffu);
            dst[(2 * e + 1) * LATM_VSTRIDE] = static_cast<unsigned short>(w[e] >> 16);
          }
        }
      }
    };

    if (k_begin < k_end) {
      ask(k_begin);
      for (int k0 = k_begin; k0 < k_end; k0 += LATM_KEYS) {
        __syncthreads();  // the round before has been read
        put();
        __syncthreads();
        turn();
        __syncthreads();
        if (k0 + LATM_KEYS < k_end) ask(k0 + LATM_KEYS);
        if (!wave_on) continue;
        lat_f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NW; ++s) {
          if (s < nw) {
            const lat_bf16x8 a0 = *reinterpret_cast<const lat_bf16x8*>(k_s + key_place(ka0, 4 * s + g));
            const lat_bf16x8 a1 = *reinterpret_cast<const lat_bf16x8*>(k_s + key_place(ka1, 4 * s + g));
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[s], s1, 0, 0, 0);
          }
        }
        float p[8];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = k0 + 8 * g + i;
          p[i] = (j <= my_pos && j > my_lo && j < k_end) ? s0[i] * scale_log2 : -INFINITY;
          p[4 + i] = (j + 4 <= my_pos && j + 4 > my_lo && j + 4 < k_end) ? s1[i] * scale_log2 : -INFINITY;
          mx = fmaxf(mx, fmaxf(p[i], p[4 + i]));
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m, mx);
        const float alpha = exp2f(m - m_new);
        m = m_new;
        float sum = 0.f;
        lat_bf16x8 pb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          p[i] = exp2f(p[i] - m_new);
          sum += p[i];
          pb[i] = static_cast<__bf16>(p[i]);
        }
        l = l * alpha + sum;
        const bool rescale = !__all(alpha == 1.0f);
#pragma unroll
        for (int d = 0; d < NR; ++d) {
          if (d < nr) {
            if (rescale) acc[d] *= alpha;
            const lat_bf16x8 a = *reinterpret_cast<const lat_bf16x8*>(vt_s + (16 * d + n) * LATM_VSTRIDE + 8 * g);
            acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb, acc[d], 0, 0, 0);
          }
        }
      }
    }
    seg = end;
  }

  if (!wave_on) return;
  float lt = l + __shfl_xor(l, 16);
  lt += __shfl_xor(lt, 32);
  if (!col_ok) return;
  if (DEC && n_splits > 1) {
    const int64_t p = (static_cast<int64_t>(row) * heads + head) * n_splits + blockIdx.z;
#pragma unroll
    for (int d = 0; d < NR; ++d)
      if (d < nr) *reinterpret_cast<lat_f32x4*>(part_o + p * rank + 16 * d + 4 * g) = acc[d];
    if (g == 0) {
      part_ml[2 * p] = lt > 0.f ? m : -INFINITY;
      part_ml[2 * p + 1] = lt;
    }
  } else {
    const float inv = 1.0f / lt;
#pragma unroll
    for (int d = 0; d < NR; ++d) {
      if (d < nr) {
        lat_bf16x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<__bf16>(acc[d][i] * inv);
        *reinterpret_cast<lat_bf16x4*>(out + row * out_t + head * out_h + 16 * d + 4 * g) = o;
      }
    }
  }
}

// decode != 0: one token per request (tokens == requests); with n_splits > 1 the keys are cut into that many slices,
// part_o float32 [tokens * heads * n_splits, rank] and part_ml float32 [tokens * heads * n_splits, 2] take what the
// slices leave, and out must be contiguous [tokens, heads, rank].
extern "C" int ix_latent_attention_mfma(const void* ql, int64_t ql_t, int64_t ql_h, const void* qr, int64_t qr_t,
                                        int64_t qr_h, const void* cache, const int32_t* block_table,
                                        const int32_t* seq_of_token, const int32_t* positions, void* out,
                                        int64_t out_t, int64_t out_h, float* part_o, float* part_ml, int n_splits,
                                        int64_t tokens, int heads, int rank, int rot_dim, int page_size,
                                        int max_blocks, float scale, int decode, int window, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && tokens < (1 << 30) && heads > 0 && rank > 0 && rot_dim >= 0 && page_size > 0 && max_blocks > 0 &&
                 window >= 0, "sizes must be positive");
  const int width = rank + rot_dim;
  IX_REQUIRE(width % 32 == 0 && rank % 16 == 0 && width <= 576 && rank <= 512,
             "rank + rot_dim must be a multiple of 32 up to 576, rank a multiple of 16 up to 512");
  IX_REQUIRE(((reinterpret_cast<uintptr_t>(ql) | reinterpret_cast<uintptr_t>(qr) | reinterpret_cast<uintptr_t>(cache)) & 15) == 0 &&
                 (ql_t | ql_h | qr_t | qr_h) % 8 == 0 && (rot_dim == 0 || rank % 8 == 0),
             "queries and cache must lie on 16-byte boundaries");
  IX_REQUIRE((reinterpret_cast<uintptr_t>(out) & 7) == 0 && (out_t | out_h) % 4 == 0, "out must lie on 8-byte boundaries");
  IX_REQUIRE(n_splits >= 1 && n_splits <= 256 && (decode || n_splits == 1), "1 to 256 slices, and only for single tokens");
  IX_REQUIRE(n_splits == 1 || (part_o != nullptr && part_ml != nullptr && out_h == rank && out_t == static_cast<int64_t>(heads) * rank),
             "slices need their workspace and a contiguous result");
  IX_REQUIRE(heads < 65536 * 4, "too many heads for one launch");
  if (tokens == 0) return 0;
  const int n_tiles = static_cast<int>((tokens + 15) / 16);
  const size_t lds = (static_cast<size_t>(LATM_KEYS) * (((width + 63) & ~63) + LATM_KPAD) + static_cast<size_t>(rank) * LATM_VSTRIDE) * 2;
  const dim3 grid = decode ? dim3(static_cast<unsigned>(tokens), (heads + 63) / 64, n_splits)
                           : dim3(static_cast<unsigned>(n_tiles) * ((heads + 3) / 4), 1, 1);
  const float scale_log2 = scale * 1.4426950408889634f;
#define LAUNCH(NW, NR, DEC)                                                                                             \
  do {                                                                                                                  \
    auto kernel = latent_attn_mfma_kernel<NW, NR, DEC>;                                                                 \
    if (lds > 48 * 1024) {                                                                                              \
      static bool raised = false;                                                                                       \
      if (!raised) {                                                                                                    \
        /* (a refusal shows as the launch's own error) */                                                              \
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,    \
                                  96 * 1024);                                                                           \
        (void)hipGetLastError();                                                                                        \
        raised = true;                                                                                                  \
      }                                                                                                                 \
    }                                                                                                                   \
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, (const __bf16*)ql, ql_t, ql_h, (const __bf16*)qr, qr_t,     \
                       qr_h, (const __bf16*)cache, block_table, seq_of_token, positions, (__bf16*)out, out_t, out_h,     \
                       part_o, part_ml, n_splits, static_cast<int>(tokens), heads, rank, rot_dim, page_size, max_blocks, \
                       scale_log2, n_tiles, window);                                                                    \
  } while (0)
#define BY_SIZE(DEC)                                        \
  if (width <= 128 && rank <= 128) LAUNCH(4, 8, DEC);       \
  else if (width <= 320 && rank <= 256) LAUNCH(10, 16, DEC); \
  else LAUNCH(18, 32, DEC)
  if (decode) { BY_SIZE(true); } else { BY_SIZE(false); }
#undef BY_SIZE
#undef LAUNCH
  if (ix_check_launch("ix_latent_attention_mfma")) return 1;
  if (n_splits > 1) return ix_attention_combine(part_o, part_ml, out, tokens, heads, n_splits, rank, stream);
  return 0;
}
