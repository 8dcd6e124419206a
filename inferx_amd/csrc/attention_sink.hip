// What stands around an attention whose queries and keys are normalised head by head and whose values are rotated.
//
// ix_qkv_norm_rope_append, after the q|k|v product, a wavefront per (token, head of q, k or v):
//   q, k:  x <- x / sqrt(mean(x^2) + eps) * w   over the head (w [head_dim], shared by the heads; optional), then the
//          2 * half elements from rot_begin on are rotated: pair (i, i + half) by the token's angle i
//   v:     ALL of the head is rotated, pair (m, m + value_dim / 2) by the token's angle m of the values' own table
//   q goes to q_out [T, heads, head_dim]; k and v go to the token's slot of the paged caches, keys
//   [page][kv_head][offset][head_dim], values transposed [page][kv_head][value_dim][offset].
// ix_rotate_heads turns the heads of a result back (or forth) in place.
// Sums, norms and rotations are float32; tables are float32 (cos, sin) per token and pair.
#include "common.h"

#define NRA_MAX_DIM 256

template <typename T>
__global__ void __launch_bounds__(256)
qkv_norm_rope_append_kernel(const T* __restrict__ qkv, int64_t stride, const void* __restrict__ q_norm, int qn_dtype,
                            const void* __restrict__ k_norm, int kn_dtype, float eps, const float2* __restrict__ cs,
                            int rot_begin, int half, const float2* __restrict__ vcs, const int32_t* __restrict__ slots,
                            T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int heads,
                            int kv_heads, int head_dim, int value_dim, int page_size, int64_t total_slots) {
  __shared__ float buf[4][NRA_MAX_DIM];
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t slot = slots ? slots[t] : -1;
  const bool cache_ok = k_cache != nullptr && slot >= 0 && slot < total_slots;
  const int64_t page = cache_ok ? slot / page_size : 0;
  const int off = cache_ok ? static_cast<int>(slot % page_size) : 0;
  float* x = buf[wave];
  for (int item = blockIdx.y * 4 + wave; item < heads + 2 * kv_heads; item += gridDim.y * 4) {
    const bool is_q = item < heads, is_v = item >= heads + kv_heads;
    const int d = is_v ? value_dim : head_dim;
    const int g = is_q ? item : (is_v ? item - heads - kv_heads : item - heads);
    const T* in = qkv + t * stride +
                  (is_q ? static_cast<int64_t>(g) * head_dim
                        : (is_v ? static_cast<int64_t>(heads + kv_heads) * head_dim + static_cast<int64_t>(g) * value_dim
                                : static_cast<int64_t>(heads + g) * head_dim));
    if (!is_q && !cache_ok) continue;
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float v = ix_load(in + i);
      x[i] = v;
      ss += v * v;
    }
    const void* w = is_q ? q_norm : k_norm;
    const int w_dtype = is_q ? qn_dtype : kn_dtype;
    if (!is_v && w) {
      ss = ix_wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
      for (int i = lane; i < d; i += 64) x[i] = x[i] * inv * ix_load_rt(w, w_dtype, i);
    }
    // (a wavefront's lanes run together: what one wrote to its own rows of `buf` the others may read)
    __builtin_amdgcn_wave_barrier();
    const float2* table = is_v ? vcs : cs;
    const int first = is_v ? 0 : rot_begin, hf = is_v ? value_dim / 2 : half;
    for (int i = lane; i < d; i += 64) {
      float y = x[i];
      const int r = i - first;
      if (table && r >= 0 && r < 2 * hf) {
        const bool low = r < hf;
        const float2 c = table[t * hf + (low ? r : r - hf)];
        const float other = x[first + (low ? r + hf : r - hf)];
        y = low ? y * c.x - other * c.y : y * c.x + other * c.y;
      }
      if (is_q) ix_store(q_out + (t * heads + g) * head_dim + i, y);
      else if (is_v) ix_store(v_cache + ((page * kv_heads + g) * value_dim + i) * page_size + off, y);
      else ix_store(k_cache + ((page * kv_heads + g) * page_size + off) * head_dim + i, y);
    }
    __builtin_amdgcn_wave_barrier();
  }
}

extern "C" int ix_qkv_norm_rope_append(const void* qkv, int dtype, int64_t stride, const void* q_norm, int qn_dtype,
                                       const void* k_norm, int kn_dtype, float eps, const float* cs, int rot_begin,
                                       int half, const float* vcs, const int32_t* slots, void* q_out, void* k_cache,
                                       void* v_cache, int64_t tokens, int heads, int kv_heads, int head_dim,
                                       int value_dim, int page_size, int64_t total_slots, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && value_dim > 0 && page_size > 0,
             "sizes must be positive");
  IX_REQUIRE(head_dim <= NRA_MAX_DIM && value_dim <= NRA_MAX_DIM, "heads of at most 256 numbers");
  IX_REQUIRE(stride >= static_cast<int64_t>(heads + kv_heads) * head_dim + static_cast<int64_t>(kv_heads) * value_dim,
             "a row of the product is shorter than q, k and v together");
  IX_REQUIRE(half >= 0 && rot_begin >= 0 && rot_begin + 2 * half <= head_dim && (half == 0 || cs != nullptr),
             "the rotated part must lie within the head");
  IX_REQUIRE(vcs == nullptr || value_dim % 2 == 0, "rotated values need an even size");
  IX_REQUIRE((k_cache == nullptr) == (v_cache == nullptr), "give both caches or neither");
  if (tokens == 0) return 0;
  const int items = heads + 2 * kv_heads;
  dim3 grid(static_cast<unsigned>(tokens), std::min((items + 3) / 4, 16)), block(256);
  if (half == 0) cs = nullptr;
#define LAUNCH(TT)                                                                                                     \
  hipLaunchKernelGGL(qkv_norm_rope_append_kernel<TT>, grid, block, 0, stream, (const TT*)qkv, stride, q_norm, qn_dtype, \
                     k_norm, kn_dtype, eps, (const float2*)cs, rot_begin, half, (const float2*)vcs, slots, (TT*)q_out,  \
                     (TT*)k_cache, (TT*)v_cache, heads, kv_heads, head_dim, value_dim, page_size, total_slots)
  if (dtype == IX_F32) LAUNCH(float);
  else if (dtype == IX_BF16) LAUNCH(bf16_t);
  else IX_REQUIRE(false, "dtype must be float32 or bfloat16");
#undef LAUNCH
  return ix_check_launch("ix_qkv_norm_rope_append");
}

// x [T, heads, d] in place: pair (i, i + d / 2) of every head turned by the token's angle i (cs float32 [T, d / 2]
// of (cos, sin)); `inverse`: by minus that angle.
template <typename T>
__global__ void rotate_heads_kernel(T* __restrict__ x, const float2* __restrict__ cs, int64_t tokens, int heads, int d,
                                    int inverse) {
  const int half = d / 2;
  const int64_t n = tokens * heads * half;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < n;
       p += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int i = static_cast<int>(p % half);
    const int64_t th = p / half, t = th / heads;
    T* at = x + th * d + i;
    const float2 c = cs[t * half + i];
    const float s = inverse ? -c.y : c.y;
    const float u = ix_load(at), v = ix_load(at + half);
    ix_store(at, u * c.x - v * s);
    ix_store(at + half, v * c.x + u * s);
  }
}

extern "C" int ix_rotate_heads(void* x, int dtype, const float* cs, int64_t tokens, int heads, int d, int inverse,
                               hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && d > 0 && d % 2 == 0, "sizes must be positive, the head's size even");
  if (tokens == 0) return 0;
  const int64_t n = tokens * heads * (d / 2);
  dim3 grid(static_cast<unsigned>(std::min<int64_t>((n + 255) / 256, 65536))), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(rotate_heads_kernel<float>, grid, block, 0, stream, (float*)x, (const float2*)cs, tokens, heads, d, inverse);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(rotate_heads_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)x, (const float2*)cs, tokens, heads, d, inverse);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_rotate_heads");
}
