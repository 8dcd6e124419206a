// A matrix memory with exponential gates (the mLSTM recurrence): per head a matrix S [dim, vdim], a vector n [dim] and
// a running maximum m of the gates' logarithms, all float32,
//
//   i = cap tanh(a / cap),  f = logsigmoid(cap tanh(b / cap))          a, b: the two gates' logits of the token
//   m' = max(f + m, i)
//   S <- exp(f + m - m') S + exp(i - m') k v^T;   n <- exp(f + m - m') n + exp(i - m') k
//   o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
//
// token after token; S, n and m start at zero (m at 0, not at minus infinity).  q arrives unscaled and is multiplied
// by dim^(-1/2) here.  Everything but the loads of q, k, v is float32.
//
// As for the delta rule, the columns of S are independent, so the work is spread over (request, head, block of 16
// value columns): a wavefront each, four lanes per column that own every fourth row (or, VEC, a quarter of the rows
// side by side, read in 16-byte pieces).  Every lane also carries n for its rows and m (the same in all columns).
// Every block of columns keeps a copy of n and m of its own in the slot and reads and writes no other's: a block that
// starts late must not find what an earlier one has already moved on.  In the slot a head's matrix lies
// [column][row]; after the matrices of all heads come, per block of 16 columns, n [heads][dim] and m [heads].
#include "common.h"

typedef float mm_f32x4 __attribute__((ext_vector_type(4)));

#define MM_COLS 16
#define MM_SPLIT 4

__device__ __forceinline__ void mm_load8(const float* p, float (&out)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
  out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
__device__ __forceinline__ void mm_load8(const bf16_t* p, float (&out)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  out[0] = __uint_as_float(a.x << 16); out[1] = __uint_as_float(a.x & 0xffff0000u);
  out[2] = __uint_as_float(a.y << 16); out[3] = __uint_as_float(a.y & 0xffff0000u);
  out[4] = __uint_as_float(a.z << 16); out[5] = __uint_as_float(a.z & 0xffff0000u);
  out[6] = __uint_as_float(a.w << 16); out[7] = __uint_as_float(a.w & 0xffff0000u);
}

// the two gates' logarithms from their logits
__device__ __forceinline__ void mm_gates(float a, float b, float cap, float& gi, float& gf) {
  gi = cap * tanhf(a / cap);
  const float y = cap * tanhf(b / cap);
  gf = fminf(y, 0.f) - log1pf(expf(-fabsf(y)));
}

template <typename T, int RPL, bool VEC>
__global__ void __launch_bounds__(64)
matrix_memory_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride,
                     int64_t k_stride, int64_t v_stride, const float* __restrict__ gates,
                     const float* __restrict__ gate_bias, float cap, float* __restrict__ state, int64_t state_stride,
                     const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                     float* __restrict__ out, int heads, int dim, int vdim) {
  const int lane = threadIdx.x;
  const int col = blockIdx.x * MM_COLS + lane / MM_SPLIT, part = lane % MM_SPLIT;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const bool live = col < vdim;
  const int cj = live ? col : vdim - 1;  // lanes past the last column repeat it and store nothing
  float* slot = state + static_cast<int64_t>(state_slots[seq]) * state_stride;
  float* sp = slot + static_cast<int64_t>(head) * dim * vdim;
  float* mine = slot + static_cast<int64_t>(heads) * dim * vdim + static_cast<int64_t>(blockIdx.x) * (heads * dim + heads);
  float* np_ = mine + static_cast<int64_t>(head) * dim;
  float* mp = mine + static_cast<int64_t>(heads) * dim + head;
  const int quarter = dim / MM_SPLIT;
  auto row_of = [&](int r) { return VEC ? (r < quarter ? part * quarter + r : dim) : r * MM_SPLIT + part; };
  float S[RPL], N[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int i = row_of(r);
    S[r] = i < dim ? sp[static_cast<int64_t>(cj) * dim + i] : 0.f;
    N[r] = i < dim ? np_[i] : 0.f;
  }
  float m = *mp;
  const float q_scale = 1.0f / sqrtf(static_cast<float>(dim));
  const float bias_i = gate_bias[head], bias_f = gate_bias[heads + head];

  float kc[RPL], qc[RPL], vc, ac, bc;
  auto fetch = [&](int64_t row, float (&kk)[RPL], float (&qq)[RPL], float& vv, float& aa, float& bb) {
    const T* qr = q + row * q_stride + head * dim;
    const T* kr = k + row * k_stride + head * dim;
    if constexpr (VEC) {
#pragma unroll
      for (int r = 0; r < RPL; r += 8) {
        if (r < quarter) {
          float k8[8], q8[8];
          mm_load8(kr + part * quarter + r, k8);
          mm_load8(qr + part * quarter + r, q8);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            kk[r + j] = k8[j];
            qq[r + j] = q8[j];
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) kk[r + j] = qq[r + j] = 0.f;
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        const int i = r * MM_SPLIT + part;
        kk[r] = i < dim ? ix_load(kr + i) : 0.f;
        qq[r] = i < dim ? ix_load(qr + i) : 0.f;
      }
    }
    vv = ix_load(v + row * v_stride + head * vdim + cj);
    aa = gates[row * 2 * heads + head];
    bb = gates[row * 2 * heads + heads + head];
  };
  fetch(row0, kc, qc, vc, ac, bc);
  for (int i = 0; i < n; ++i) {
    float kn[RPL], qn[RPL], vn, an, bn;
    fetch(row0 + min(i + 1, n - 1), kn, qn, vn, an, bn);  // the next row's, on their way while this one is worked
    float gi, gf;
    mm_gates(ac + bias_i, bc + bias_f, cap, gi, gf);
    const float m_new = fmaxf(gf + m, gi);
    const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
    m = m_new;
    const float tv = take * vc;
    float o = 0.f, nq = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      S[r] = fmaf(S[r], keep, kc[r] * tv);
      N[r] = fmaf(N[r], keep, kc[r] * take);
      o += S[r] * qc[r];
      nq += N[r] * qc[r];
    }
    o += ix_dpp<IX_DPP_XOR1>(o);
    o += ix_dpp<IX_DPP_XOR2>(o);
    nq += ix_dpp<IX_DPP_XOR1>(nq);
    nq += ix_dpp<IX_DPP_XOR2>(nq);
    const float below = fmaxf(fabsf(nq * q_scale), expf(-m)) + 1e-6f;
    if (live && part == 0) out[((row0 + i) * heads + head) * vdim + col] = o * q_scale / below;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
    }
    vc = vn;
    ac = an;
    bc = bn;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = row_of(r);
      if (i < dim) sp[static_cast<int64_t>(col) * dim + i] = S[r];
    }
  }
  if (lane < MM_SPLIT) {  // (the block's own copy of n and m)
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = row_of(r);
      if (i < dim) np_[i] = N[r];
    }
    if (lane == 0) *mp = m;
  }
}

// q, k [T, heads * dim] and v [T, heads * vdim] of the run's type with their row strides; gates float32 [T, 2 heads]
// (the input gate's logits, then the forget gate's) and gate_bias float32 [2 heads] likewise; state: slot s at
// state + s * state_stride, [heads, vdim, dim], then per block of 16 value columns [heads, dim] and [heads]; out
// float32 [T, heads, vdim].
extern "C" int ix_matrix_memory(const void* q, const void* k, const void* v, int dtype, int64_t q_stride, int64_t k_stride,
                                int64_t v_stride, const float* gates, const float* gate_bias, float cap, float* state,
                                int64_t state_stride, const int32_t* q_start, const int32_t* state_slots, float* out,
                                int64_t tokens, int requests, int heads, int dim, int vdim, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && dim > 0 && vdim > 0 && cap > 0.f, "sizes must be positive");
  IX_REQUIRE(dim <= 256, "at most 256 numbers per query and key head");
  IX_REQUIRE(state_stride >= static_cast<int64_t>(heads) * dim * vdim +
                                 static_cast<int64_t>((vdim + MM_COLS - 1) / MM_COLS) * (heads * dim + heads),
             "state blocks too small");
  IX_REQUIRE(heads <= 65535 && requests <= 65535, "too many heads or requests for one launch");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  if (tokens == 0 || requests == 0) return 0;
  dim3 grid((vdim + MM_COLS - 1) / MM_COLS, heads, requests), block(64);
  const int rpl = (dim + MM_SPLIT - 1) / MM_SPLIT;
  const bool vec = dtype == IX_BF16 && dim % (8 * MM_SPLIT) == 0 && (q_stride * 2) % 16 == 0 && (k_stride * 2) % 16 == 0 &&
                   ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) == 0;
#define LAUNCH(TT, RPL, VEC)                                                                                               \
  hipLaunchKernelGGL((matrix_memory_kernel<TT, RPL, VEC>), grid, block, 0, stream, (const TT*)q, (const TT*)k, (const TT*)v, \
                     q_stride, k_stride, v_stride, gates, gate_bias, cap, state, state_stride, q_start, state_slots, out,    \
                     heads, dim, vdim)
#define PICK(TT, VEC)                      \
  if (rpl <= 8) LAUNCH(TT, 8, VEC);        \
  else if (rpl <= 16) LAUNCH(TT, 16, VEC); \
  else if (rpl <= 32) LAUNCH(TT, 32, VEC); \
  else LAUNCH(TT, 64, VEC);
  if (dtype == IX_F32) { PICK(float, false) } else if (vec) { PICK(bf16_t, true) } else { PICK(bf16_t, false) }
#undef PICK
#undef LAUNCH
  return ix_check_launch("ix_matrix_memory");
}
