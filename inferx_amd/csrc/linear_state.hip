// Recurrent mixers whose state is a matrix S [dim, vdim] per head that every token scales row by row, corrects by
// a rank-one term read from the old state, and adds an outer product to:
//
//     S <- diag(w) S - a (b^T S) + k v^T;     o = S^T r                  (both terms read the old S)
//
// w, a, b are float32 rows per token and key channel (`w_rows`, `a_rows`, `b_rows`), or absent: then w is one
// number per head (`w_head`) and there is no correction.  That covers the generalized delta rule (w a decay per
// channel, a = rate * unit key, b = unit key) and plain decayed linear attention (lightning attention: a constant
// decay per head).  r, k, v come in the run's type, optionally through silu.  The state is float32, kept per
// request slot as [heads][vdim][dim] (a column's rows side by side), and the whole recurrence is float32.
//
// A column of S only ever meets its own value, so the work is spread over (request, head, column); the rows of a
// column are shared by four neighbouring lanes whose partial sums meet through DPP.  A wavefront owns 16 columns
// and walks the request's rows of this step in order.
#include "common.h"

__device__ __forceinline__ float ls_quad_sum(float v) {
  v += ix_dpp<IX_DPP_XOR1>(v);
  v += ix_dpp<IX_DPP_XOR2>(v);
  return v;
}

__device__ __forceinline__ float ls_silu(float x) { return x / (1.0f + expf(-x)); }

// R: rows of a column per lane (4 R >= dim)
template <typename T, int R>
__global__ void __launch_bounds__(64)
linear_state_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, int64_t r_stride,
                    int64_t k_stride, int64_t v_stride, const float* __restrict__ w_rows,
                    const float* __restrict__ w_head, const float* __restrict__ a_rows,
                    const float* __restrict__ b_rows, float* __restrict__ state, int64_t state_stride,
                    const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                    float* __restrict__ out, int heads, int dim, int vdim, int silu) {
  const int lane = threadIdx.x, part = lane & 3;
  const int col = blockIdx.x * 16 + (lane >> 2);
  const int head = blockIdx.y, seq = blockIdx.z;
  const int t0 = q_start[seq], t1 = q_start[seq + 1];
  if (t1 <= t0) return;
  const bool live = col < vdim;
  const int row0 = part * R;
  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride +
              (static_cast<int64_t>(head) * vdim + (live ? col : 0)) * dim;
  float s[R];
#pragma unroll
  for (int i = 0; i < R; ++i) s[i] = (live && row0 + i < dim) ? sp[row0 + i] : 0.f;
  const float wh = w_head ? w_head[head] : 1.0f;
  const int64_t ch = static_cast<int64_t>(head) * dim;  // first key channel of this head
  for (int t = t0; t < t1; ++t) {
    float rr[R], kk[R], ww[R], aa[R], bb[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const bool ok = row0 + i < dim;
      const int64_t c = ch + row0 + i;
      rr[i] = ok ? ix_load(r + t * r_stride + c) : 0.f;
      kk[i] = ok ? ix_load(k + t * k_stride + c) : 0.f;
      if (silu) {
        rr[i] = ls_silu(rr[i]);
        kk[i] = ls_silu(kk[i]);
      }
      ww[i] = (ok && w_rows) ? w_rows[static_cast<int64_t>(t) * heads * dim + c] : wh;
      aa[i] = (ok && a_rows) ? a_rows[static_cast<int64_t>(t) * heads * dim + c] : 0.f;
      bb[i] = (ok && b_rows) ? b_rows[static_cast<int64_t>(t) * heads * dim + c] : 0.f;
    }
    float vj = live ? ix_load(v + t * v_stride + static_cast<int64_t>(head) * vdim + col) : 0.f;
    if (silu) vj = ls_silu(vj);
    float read = 0.f;
    if (a_rows) {
#pragma unroll
      for (int i = 0; i < R; ++i) read += bb[i] * s[i];
      read = ls_quad_sum(read);
    }
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      s[i] = ww[i] * s[i] - aa[i] * read + kk[i] * vj;
      o += rr[i] * s[i];
    }
    o = ls_quad_sum(o);
    if (live && part == 0) out[(static_cast<int64_t>(t) * heads + head) * vdim + col] = o;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (row0 + i < dim) sp[row0 + i] = s[i];
  }
}

extern "C" int ix_linear_state(const void* r, const void* k, const void* v, int dtype, int64_t r_stride,
                               int64_t k_stride, int64_t v_stride, const float* w_rows, const float* w_head,
                               const float* a_rows, const float* b_rows, float* state, int64_t state_stride,
                               const int32_t* q_start, const int32_t* state_slots, float* out, int64_t tokens,
                               int requests, int heads, int dim, int vdim, int silu, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && requests > 0 && heads > 0 && dim > 0 && vdim > 0, "sizes must be positive");
  IX_REQUIRE(dim <= 256, "a head's keys hold at most 256 numbers");
  IX_REQUIRE((w_rows != nullptr) != (w_head != nullptr), "the decay comes per row and channel or per head");
  IX_REQUIRE((a_rows != nullptr) == (b_rows != nullptr), "the correction's two vectors come together");
  IX_REQUIRE(state_stride >= static_cast<int64_t>(heads) * dim * vdim, "a slot's state is too small");
  IX_REQUIRE(requests < 65536 && heads < 65536, "too many requests or heads for one launch");
  if (tokens == 0) return 0;
  dim3 grid((vdim + 15) / 16, heads, requests), block(64);
#define LAUNCH(T, R)                                                                                               \
  hipLaunchKernelGGL((linear_state_kernel<T, R>), grid, block, 0, stream, (const T*)r, (const T*)k, (const T*)v,    \
                     r_stride, k_stride, v_stride, w_rows, w_head, a_rows, b_rows, state, state_stride, q_start,    \
                     state_slots, out, heads, dim, vdim, silu)
#define PICK(T)                        \
  if (dim <= 16) LAUNCH(T, 4);         \
  else if (dim <= 32) LAUNCH(T, 8);    \
  else if (dim <= 64) LAUNCH(T, 16);   \
  else if (dim <= 128) LAUNCH(T, 32);  \
  else LAUNCH(T, 64)
  if (dtype == IX_F32) { PICK(float); }
  else if (dtype == IX_BF16) { PICK(bf16_t); }
  else IX_REQUIRE(false, "dtype must be float32 or bfloat16");
#undef PICK
#undef LAUNCH
  return ix_check_launch("ix_linear_state");
}

// ---------------------------------------------------------------------------
// What the generalized delta rule hands to the recurrence, per token, head and key channel, all float32:
//     w = exp(-decay_scale * sigmoid(w_logit + w_bias))         the decay
//     u = k / sqrt(sum over the head of k^2 + unit_eps)          the unit key
//     a = sigmoid(a_logit + a_bias) * u                           what is removed along u
// w_logit float32 [T, heads * dim]; a_logit and k in the run's type (rows may be strided).
template <typename T>
__global__ void __launch_bounds__(256)
delta_operands_kernel(const float* __restrict__ w_logit, const void* __restrict__ w_bias, int wb_dtype,
                      const T* __restrict__ a_logit, int64_t a_stride, const void* __restrict__ a_bias, int ab_dtype,
                      const T* __restrict__ k, int64_t k_stride, float* __restrict__ w, float* __restrict__ a,
                      float* __restrict__ u, int64_t pairs, int heads, int dim, float decay_scale, float unit_eps) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = p / heads;
  const int head = static_cast<int>(p % heads);
  const int64_t c0 = static_cast<int64_t>(head) * dim;
  float ss = 0.f;
  for (int i = lane; i < dim; i += 64) {
    const float kv = ix_load(k + t * k_stride + c0 + i);
    ss += kv * kv;
  }
  ss = ix_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss + unit_eps);
  for (int i = lane; i < dim; i += 64) {
    const int64_t c = c0 + i, at = t * heads * dim + c;
    const float uv = ix_load(k + t * k_stride + c) * inv;
    const float wl = w_logit[at] + ix_load_rt(w_bias, wb_dtype, c);
    const float al = ix_load(a_logit + t * a_stride + c) + ix_load_rt(a_bias, ab_dtype, c);
    w[at] = expf(-decay_scale / (1.0f + expf(-wl)));
    u[at] = uv;
    a[at] = uv / (1.0f + expf(-al));
  }
}

extern "C" int ix_delta_operands(const float* w_logit, const void* w_bias, int wb_dtype, const void* a_logit,
                                 int64_t a_stride, const void* a_bias, int ab_dtype, const void* k, int64_t k_stride,
                                 int dtype, float* w, float* a, float* u, int64_t tokens, int heads, int dim,
                                 float decay_scale, float unit_eps, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && dim > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  const int64_t pairs = tokens * heads;
  IX_REQUIRE((pairs + 3) / 4 < (1ll << 31), "too many rows for one launch");
  dim3 grid(static_cast<unsigned>((pairs + 3) / 4)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(delta_operands_kernel<float>, grid, block, 0, stream, w_logit, w_bias, wb_dtype,
                       (const float*)a_logit, a_stride, a_bias, ab_dtype, (const float*)k, k_stride, w, a, u, pairs,
                       heads, dim, decay_scale, unit_eps);
  else if (dtype == IX_BF16)
    hipLaunchKernelGGL(delta_operands_kernel<bf16_t>, grid, block, 0, stream, w_logit, w_bias, wb_dtype,
                       (const bf16_t*)a_logit, a_stride, a_bias, ab_dtype, (const bf16_t*)k, k_stride, w, a, u, pairs,
                       heads, dim, decay_scale, unit_eps);
  else
    IX_REQUIRE(false, "dtype must be float32 or bfloat16");
  return ix_check_launch("ix_delta_operands");
}

// y[i] = tanh(x[i]) in float32 (between the two small products behind a decay)
__global__ void tanh_rows_kernel(float* __restrict__ x, int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    x[i] = tanhf(x[i]);
}

extern "C" int ix_tanh_inplace(float* x, int64_t n, hipStream_t stream) {
  IX_REQUIRE(n >= 0, "the size must not be negative");
  if (n == 0) return 0;
  dim3 grid(static_cast<unsigned>(std::min<int64_t>((n + 255) / 256, 65536))), block(256);
  hipLaunchKernelGGL(tanh_rows_kernel, grid, block, 0, stream, x, n);
  return ix_check_launch("ix_tanh_inplace");
}
