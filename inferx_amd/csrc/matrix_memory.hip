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
// Three steps.  (1) ix_memory_gates: the maxima are a chain over a request's tokens that involves no vectors, so it
// runs first, a wavefront per (request, head), sixty-four tokens at a time: with F the running sum of f,
// m_t = F_t + max(m_0, max_{s <= t}(i_s - F_s)), two scans over the lanes.  It leaves per token and head
// keep = exp(f + m - m'), take = exp(i - m') and exp(-m'), and the last m in the state.  (2) ix_matrix_memory: n is
// one more column of S whose value is always 1, so the recurrence is S <- keep S + k (take v)^T over vdim + 1
// independent columns, spread over wavefronts like the delta rule's (a few rows: four lanes a column, the next row's
// operands asked for ahead; portions: chunks of 32 rows staged in LDS as float32, sixteen or four lanes a column).
// Nothing is shared between the blocks of a head.  It leaves S^T q per column and n . q.  (3) The division by
// max(|n . q|, exp(-m')) + 1e-6 rides on the kernel that normalises the heads (ix_head_norm_gate).
// In the slot a head's matrix lies [column][row] with n as column vdim; after the matrices come the maxima [heads].
#include "common.h"

typedef unsigned int mm_u32x4 __attribute__((ext_vector_type(4)));
typedef float mm_f32x4 __attribute__((ext_vector_type(4)));

#define MM_COLS 16
#define MM_SPLIT 4
#define MM_CHUNK 32

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

// ---- (1) the gates ----------------------------------------------------------------------------------------------
// gates float32 [T, 2 heads] (the input gate's logits, then the forget gate's), gate_bias float32 [2 heads] likewise;
// out float32 [T, heads, 3] = keep, take, exp(-m'); maxima: the request's m [heads] in its slot, read and left.
__global__ void __launch_bounds__(64)
memory_gates_kernel(const float* __restrict__ gates, const float* __restrict__ gate_bias, float cap,
                    float* __restrict__ maxima, int64_t state_stride, const int32_t* __restrict__ q_start,
                    const int32_t* __restrict__ state_slots, float* __restrict__ out, int heads) {
  const int lane = threadIdx.x, head = blockIdx.x, seq = blockIdx.y;
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  float* mp = maxima + static_cast<int64_t>(state_slots[seq]) * state_stride + head;
  float m0 = *mp;
  const float bias_i = gate_bias[head], bias_f = gate_bias[heads + head];
  for (int base = 0; base < n; base += 64) {
    const int t = base + lane;
    const bool live = t < n;
    float gi = -INFINITY, gf = 0.f;  // (lanes past the end change nothing: they follow every live one)
    if (live) {
      gi = cap * tanhf((gates[(row0 + t) * 2 * heads + head] + bias_i) / cap);
      const float y = cap * tanhf((gates[(row0 + t) * 2 * heads + heads + head] + bias_f) / cap);
      gf = fminf(y, 0.f) - log1pf(expf(-fabsf(y)));
    }
    float F = gf;  // the sum of f up to and with this token
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float other = __shfl_up(F, d, 64);
      if (lane >= d) F += other;
    }
    float P = gi - F;  // the largest i_s - F_s up to and with this token
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float other = __shfl_up(P, d, 64);
      if (lane >= d) P = fmaxf(P, other);
    }
    const float m = F + fmaxf(m0, P);
    float before = __shfl_up(m, 1, 64);
    if (lane == 0) before = m0;
    if (live) {
      float* o = out + ((row0 + t) * heads + head) * 3;
      o[0] = expf(gf + before - m);
      o[1] = expf(gi - m);
      o[2] = expf(-m);
    }
    m0 = __shfl(m, 63, 64);
  }
  if (lane == 0) *mp = m0;
}

// ---- (2) the recurrence, a few rows per request -----------------------------------------------------------------------
template <typename T, int RPL, bool VEC>
__global__ void __launch_bounds__(64)
matrix_memory_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride,
                     int64_t k_stride, int64_t v_stride, const float* __restrict__ kt, float* __restrict__ state,
                     int64_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                     float* __restrict__ out, float* __restrict__ nq, int heads, int dim, int vdim) {
  const int lane = threadIdx.x;
  const int col = blockIdx.x * MM_COLS + lane / MM_SPLIT, part = lane % MM_SPLIT;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const int cols = vdim + 1;             // column vdim is n: its value is always 1
  const bool live = col < cols;
  const int cj = live ? col : cols - 1;  // lanes past the last column repeat it and store nothing
  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride + static_cast<int64_t>(head) * dim * cols;
  const int quarter = dim / MM_SPLIT;
  auto row_of = [&](int r) { return VEC ? (r < quarter ? part * quarter + r : dim) : r * MM_SPLIT + part; };
  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) {
    const int i = row_of(r);
    S[r] = i < dim ? sp[static_cast<int64_t>(cj) * dim + i] : 0.f;
  }
  const float q_scale = 1.0f / sqrtf(static_cast<float>(dim));

  float kc[RPL], qc[RPL], vc, keep_c, take_c;
  auto fetch = [&](int64_t row, float (&kk)[RPL], float (&qq)[RPL], float& vv, float& keep, float& take) {
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
    vv = cj < vdim ? ix_load(v + row * v_stride + head * vdim + cj) : 1.0f;
    keep = kt[(row * heads + head) * 3];
    take = kt[(row * heads + head) * 3 + 1];
  };
  fetch(row0, kc, qc, vc, keep_c, take_c);
  for (int i = 0; i < n; ++i) {
    float kn[RPL], qn[RPL], vn, keep_n, take_n;
    fetch(row0 + min(i + 1, n - 1), kn, qn, vn, keep_n, take_n);  // the next row's, on their way while this one is worked
    const float tv = take_c * vc;
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      S[r] = fmaf(S[r], keep_c, kc[r] * tv);
      o += S[r] * qc[r];
    }
    o += ix_dpp<IX_DPP_XOR1>(o);
    o += ix_dpp<IX_DPP_XOR2>(o);
    if (live && part == 0) {
      if (col < vdim) out[((row0 + i) * heads + head) * vdim + col] = o * q_scale;
      else nq[(row0 + i) * heads + head] = o * q_scale;
    }
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
    }
    vc = vn;
    keep_c = keep_n;
    take_c = take_n;
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = row_of(r);
      if (i < dim) sp[static_cast<int64_t>(col) * dim + i] = S[r];
    }
  }
}

// ---- (2) the same for portions: chunks of MM_CHUNK rows through LDS (bfloat16, heads of 32, 64 or 128 numbers) ------------
template <int SP>
__device__ __forceinline__ float mm_sum_over(float x) {  // over the SP neighbouring lanes of a column
  x += ix_dpp<IX_DPP_XOR1>(x);
  x += ix_dpp<IX_DPP_XOR2>(x);
  if constexpr (SP >= 8) x += ix_dpp<IX_DPP_HALF_MIRROR>(x);
  if constexpr (SP >= 16) x += ix_dpp<IX_DPP_MIRROR>(x);
  return x;
}

template <int SP, int RPL>
__global__ void __launch_bounds__(64)
matrix_memory_chunk_kernel(const bf16_t* q, const bf16_t* k, const bf16_t* v, int64_t q_stride, int64_t k_stride,
                           int64_t v_stride, const float* __restrict__ kt, float* __restrict__ state,
                           int64_t state_stride, const int32_t* __restrict__ q_start,
                           const int32_t* __restrict__ state_slots, float* __restrict__ out, float* __restrict__ nq,
                           int heads, int vdim) {
  constexpr int DIM = SP * RPL;
  constexpr int COLS = 64 / SP;                         // columns of a wavefront
  constexpr int PIECES = DIM / 8;                       // 16-byte pieces of a q or k row
  constexpr int PER_LANE = MM_CHUNK * 2 * PIECES / 64;  // pieces of a chunk's q and k rows that a lane moves
  constexpr int V_PER_LANE = (MM_CHUNK * COLS + 63) / 64;
  __shared__ mm_f32x4 qk_s[MM_CHUNK][2][DIM / 4];  // [row][k, q]: float32, q times dim^(-1/2)
  __shared__ float v_s[MM_CHUNK][COLS];
  __shared__ float kt_s[MM_CHUNK][2];              // keep, take
  const int lane = threadIdx.x;
  const int col0 = blockIdx.x * COLS;
  const int col = col0 + lane / SP, part = lane % SP;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const int cols = vdim + 1;
  const bool live = col < cols;
  const int cj = live ? col : cols - 1;
  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride + static_cast<int64_t>(head) * DIM * cols;
  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) S[r] = sp[static_cast<int64_t>(cj) * DIM + part * RPL + r];
  const float q_scale = 1.0f / sqrtf(static_cast<float>(DIM));

  mm_u32x4 st_qk[PER_LANE];
  float st_v[V_PER_LANE], st_kt;
  auto ask = [&](int first) {  // rows first .. first + MM_CHUNK - 1 of the portion (rows past its end repeat the last)
#pragma unroll
    for (int u = 0; u < PER_LANE; ++u) {
      const int id = u * 64 + lane;  // piece number within the chunk: [row][k, q][piece]
      const int r = id / (2 * PIECES), which = (id / PIECES) & 1, pc = id % PIECES;
      const int64_t row = row0 + min(first + r, n - 1);
      const bf16_t* src = which ? q + row * q_stride + head * DIM : k + row * k_stride + head * DIM;
      st_qk[u] = *reinterpret_cast<const mm_u32x4*>(src + 8 * pc);
    }
#pragma unroll
    for (int u = 0; u < V_PER_LANE; ++u) {
      const int id = min(u * 64 + lane, MM_CHUNK * COLS - 1);
      const int r = id / COLS, c = min(col0 + id % COLS, cols - 1);
      st_v[u] = c < vdim ? ix_load(v + (row0 + min(first + r, n - 1)) * v_stride + head * vdim + c) : 1.0f;
    }
    st_kt = kt[((row0 + min(first + lane / 2, n - 1)) * heads + head) * 3 + (lane & 1)];
  };
  auto put = [&]() {
#pragma unroll
    for (int u = 0; u < PER_LANE; ++u) {
      const int id = u * 64 + lane;
      const int r = id / (2 * PIECES), which = (id / PIECES) & 1, pc = id % PIECES;
      const float f = which ? q_scale : 1.0f;
      float x[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = __uint_as_float(st_qk[u][e] << 16) * f;
        x[2 * e + 1] = __uint_as_float(st_qk[u][e] & 0xffff0000u) * f;
      }
      qk_s[r][which][2 * pc] = mm_f32x4{x[0], x[1], x[2], x[3]};
      qk_s[r][which][2 * pc + 1] = mm_f32x4{x[4], x[5], x[6], x[7]};
    }
#pragma unroll
    for (int u = 0; u < V_PER_LANE; ++u) {
      const int id = u * 64 + lane;
      if (id < MM_CHUNK * COLS) v_s[id / COLS][id % COLS] = st_v[u];
    }
    kt_s[lane / 2][lane & 1] = st_kt;
  };
  auto fetch = [&](int r, float (&kk)[RPL], float (&qq)[RPL], float& tv, float& keep) {
#pragma unroll
    for (int j = 0; j < RPL / 4; ++j) {
      const mm_f32x4 a = qk_s[r][0][part * (RPL / 4) + j], b = qk_s[r][1][part * (RPL / 4) + j];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        kk[4 * j + e] = a[e];
        qq[4 * j + e] = b[e];
      }
    }
    keep = kt_s[r][0];
    tv = kt_s[r][1] * v_s[r][lane / SP];
  };

  ask(0);
  for (int first = 0; first < n; first += MM_CHUNK) {
    __syncthreads();  // the chunk before has been read
    put();
    __syncthreads();
    if (first + MM_CHUNK < n) ask(first + MM_CHUNK);  // on their way while this chunk is worked
    __builtin_amdgcn_sched_barrier(0);
    const int rows = min(MM_CHUNK, n - first);
    float kc[RPL], qc[RPL], tvc, keep_c;
    fetch(0, kc, qc, tvc, keep_c);
    for (int i = 0; i < rows; ++i) {
      float kn[RPL], qn[RPL], tvn, keep_n;
      fetch(min(i + 1, MM_CHUNK - 1), kn, qn, tvn, keep_n);
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        S[r] = fmaf(S[r], keep_c, kc[r] * tvc);
        o += S[r] * qc[r];
      }
      o = mm_sum_over<SP>(o);
      if (live && part == 0) {
        if (col < vdim) out[((row0 + first + i) * heads + head) * vdim + col] = o;
        else nq[(row0 + first + i) * heads + head] = o;
      }
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        kc[r] = kn[r];
        qc[r] = qn[r];
      }
      tvc = tvn;
      keep_c = keep_n;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) sp[static_cast<int64_t>(col) * DIM + part * RPL + r] = S[r];
  }
}

// q, k [T, heads * dim] and v [T, heads * vdim] of the run's type with their row strides; gates float32 [T, 2 heads]
// (the input gate's logits, then the forget gate's) and gate_bias float32 [2 heads] likewise; state: slot s at
// state + s * state_stride, [heads, vdim + 1, dim] (n is column vdim) then the maxima [heads]; work float32
// [T, heads, 3] takes keep, take and exp(-m'); out float32 [T, heads, vdim] = S^T q', nq float32 [T, heads] = n . q'
// (the division is left to whoever normalises the heads).
extern "C" int ix_matrix_memory(const void* q, const void* k, const void* v, int dtype, int64_t q_stride, int64_t k_stride,
                                int64_t v_stride, const float* gates, const float* gate_bias, float cap, float* state,
                                int64_t state_stride, const int32_t* q_start, const int32_t* state_slots, float* work,
                                float* out, float* nq, int64_t tokens, int requests, int heads, int dim, int vdim,
                                hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && dim > 0 && vdim > 0 && cap > 0.f, "sizes must be positive");
  IX_REQUIRE(dim <= 256, "at most 256 numbers per query and key head");
  const int64_t matrices = static_cast<int64_t>(heads) * dim * (vdim + 1);
  IX_REQUIRE(state_stride >= matrices + heads, "state blocks too small");
  IX_REQUIRE(heads <= 65535 && requests <= 65535, "too many heads or requests for one launch");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  IX_REQUIRE(work != nullptr && nq != nullptr, "the gates' workspace and the place for n . q are needed");
  if (tokens == 0 || requests == 0) return 0;
  hipLaunchKernelGGL(memory_gates_kernel, dim3(heads, requests), dim3(64), 0, stream, gates, gate_bias, cap, state + matrices,
                     state_stride, q_start, state_slots, work, heads);
  if (ix_check_launch("ix_matrix_memory")) return 1;
  const int cols = vdim + 1;
  dim3 grid((cols + MM_COLS - 1) / MM_COLS, heads, requests), block(64);
  const int rpl = (dim + MM_SPLIT - 1) / MM_SPLIT;
  const bool vec = dtype == IX_BF16 && dim % (8 * MM_SPLIT) == 0 && (q_stride * 2) % 16 == 0 && (k_stride * 2) % 16 == 0 &&
                   ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k)) & 15) == 0;
  // steps that bring a request many rows: chunks through LDS (heads of 32, 64 or 128 numbers)
  if (vec && tokens >= 4 * static_cast<int64_t>(requests) && (dim == 32 || dim == 64 || dim == 128)) {
#define CHUNKED(SP, RPL)                                                                                                   \
  hipLaunchKernelGGL((matrix_memory_chunk_kernel<SP, RPL>), dim3((cols + 64 / SP - 1) / (64 / SP), heads, requests), block, \
                     0, stream, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, q_stride, k_stride, v_stride, work,  \
                     state, state_stride, q_start, state_slots, out, nq, heads, vdim)
    if (dim == 32) CHUNKED(4, 8);
    else if (dim == 64) CHUNKED(16, 4);
    else CHUNKED(16, 8);
#undef CHUNKED
    return ix_check_launch("ix_matrix_memory");
  }
#define LAUNCH(TT, RPL, VEC)                                                                                               \
  hipLaunchKernelGGL((matrix_memory_kernel<TT, RPL, VEC>), grid, block, 0, stream, (const TT*)q, (const TT*)k, (const TT*)v, \
                     q_stride, k_stride, v_stride, work, state, state_stride, q_start, state_slots, out, nq, heads, dim,    \
                     vdim)
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
