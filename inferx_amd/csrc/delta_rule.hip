// The gated delta rule: a linear recurrence with a matrix of state per head,
//
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q          S [dim, vdim] float32 per head
//
// token after token, so that the read-out sees the token's own write.  q and k arrive as the short convolution left
// them and are made unit vectors here (x / sqrt(sum x^2 + 1e-6), q also times dim^(-1/2)); the decay and the step
// size come from two small projections a, b (float32):  g = exp(-exp(A_log) softplus(a + dt_bias)),  beta =
// sigmoid(b).  Everything but the loads of q, k, v is float32.
//
// A decay per key channel (`ach` given): g is a vector over the rows of S, S <- diag(g) S, and `ach` float32
// [T, heads * dim] holds the decays themselves, g_i = exp(-exp(A_log) softplus(a_i + dt_bias_i)), made once per token
// and channel by ix_channel_decays (every block of a head's columns needs them all); `ab` then holds the step size's
// logits alone, float32 [T, heads], and a_log and dt_bias are not read.
//
// The columns of S are independent recurrences (column j only ever meets v[j]), so the work is spread over
// (request, head, block of 16 value columns): one wavefront each, four lanes per column that own every fourth row
// of it (RPL rows a lane, in registers; VEC: a quarter of the rows each, side by side, where that quarter is a
// multiple of eight numbers and everything is 16-byte aligned, so that a lane reads its part of q and k, and of
// the state, in 16-byte pieces).  A wavefront walks its request's rows of this step in order, with the next row's
// operands asked for before the present row is worked; the state is read from the request's slot at the start and
// written back at the end.  In the slot a head's matrix lies [column][row], a column's rows side by side.
// Query head h reads the q/k head h / (heads / kv_heads).
#include "common.h"

typedef unsigned int delta_u32x4 __attribute__((ext_vector_type(4)));
typedef float delta_f32x4 __attribute__((ext_vector_type(4)));

#define DELTA_COLS 16   // value columns per wavefront
#define DELTA_SPLIT 4   // lanes per column

// eight consecutive numbers as floats
__device__ __forceinline__ void delta_load8(const float* p, float (&out)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
  out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
__device__ __forceinline__ void delta_load8(const bf16_t* p, float (&out)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  out[0] = __uint_as_float(a.x << 16); out[1] = __uint_as_float(a.x & 0xffff0000u);
  out[2] = __uint_as_float(a.y << 16); out[3] = __uint_as_float(a.y & 0xffff0000u);
  out[4] = __uint_as_float(a.z << 16); out[5] = __uint_as_float(a.z & 0xffff0000u);
  out[6] = __uint_as_float(a.w << 16); out[7] = __uint_as_float(a.w & 0xffff0000u);
}

template <typename T, int RPL, bool VEC, bool CH>
__global__ void __launch_bounds__(64)
delta_rule_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v, int64_t q_stride,
                  int64_t k_stride, int64_t v_stride, const float* __restrict__ ab, const float* __restrict__ ach,
                  const float* __restrict__ a_log,
                  const float* __restrict__ dt_bias, float* __restrict__ state, int64_t state_stride,
                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                  float* __restrict__ out, int heads, int kv_heads, int dim, int vdim) {
  const int lane = threadIdx.x;
  const int col = blockIdx.x * DELTA_COLS + lane / DELTA_SPLIT, part = lane % DELTA_SPLIT;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int kv = head / (heads / kv_heads);
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const bool live = col < vdim;
  const int cj = live ? col : vdim - 1;  // lanes past the last column repeat it and store nothing

  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride + static_cast<int64_t>(head) * dim * vdim;
  // the rows of this lane: VEC part * dim / 4 + r, else r * 4 + part
  const int quarter = dim / DELTA_SPLIT;
  auto row_of = [&](int r) { return VEC ? (r < quarter ? part * quarter + r : dim) : r * DELTA_SPLIT + part; };
  // the state keeps a column's rows side by side ([head][column][row]): a lane's rows are one run of memory
  float S[RPL];
  if constexpr (VEC) {  // (the entry point has seen to it that the runs are 16-byte aligned)
#pragma unroll
    for (int r = 0; r < RPL; r += 4) {
      if (r < quarter) {
        const delta_f32x4 x = *reinterpret_cast<const delta_f32x4*>(sp + static_cast<int64_t>(cj) * dim + part * quarter + r);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[r + e] = x[e];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) S[r + e] = 0.f;
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int i = row_of(r);
      S[r] = i < dim ? sp[static_cast<int64_t>(cj) * dim + i] : 0.f;
    }
  }
  const float rate = CH ? 0.f : expf(a_log[head]), bias = CH ? 0.f : dt_bias[head];
  const float q_scale = 1.0f / sqrtf(static_cast<float>(dim));

  float kc[RPL], qc[RPL], vc, ac, bc;  // the present row's operands
  float gc[CH ? RPL : 1];               // (and the decays of this lane's rows)
  auto fetch = [&](int64_t row, float (&kk)[RPL], float (&qq)[RPL], float& vv, float& aa, float& bb,
                   float (&gg)[CH ? RPL : 1]) {
    const T* qr = q + row * q_stride + kv * dim;
    const T* kr = k + row * k_stride + kv * dim;
    if constexpr (CH) {
      const float* ar = ach + (row * heads + head) * dim;
      if constexpr (VEC) {
#pragma unroll
        for (int r = 0; r < RPL; r += 4) {
          if (r < quarter) {
            const delta_f32x4 x = *reinterpret_cast<const delta_f32x4*>(ar + part * quarter + r);
#pragma unroll
            for (int e = 0; e < 4; ++e) gg[r + e] = x[e];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) gg[r + e] = 0.f;
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
          const int i = r * DELTA_SPLIT + part;
          gg[r] = i < dim ? ar[i] : 0.f;
        }
      }
    }
    if constexpr (VEC) {
#pragma unroll
      for (int r = 0; r < RPL; r += 8) {
        if (r < quarter) {
          float k8[8], q8[8];
          delta_load8(kr + part * quarter + r, k8);
          delta_load8(qr + part * quarter + r, q8);
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
        const int i = r * DELTA_SPLIT + part;
        kk[r] = i < dim ? ix_load(kr + i) : 0.f;
        qq[r] = i < dim ? ix_load(qr + i) : 0.f;
      }
    }
    vv = ix_load(v + row * v_stride + head * vdim + cj);
    if constexpr (CH) {
      aa = 0.f;
      bb = ab[row * heads + head];
    } else {
      aa = ab[row * 2 * heads + head];
      bb = ab[row * 2 * heads + heads + head];
    }
  };
  fetch(row0, kc, qc, vc, ac, bc, gc);
  for (int i = 0; i < n; ++i) {
    float kn[RPL], qn[RPL], vn, an, bn, gn[CH ? RPL : 1];
    fetch(row0 + min(i + 1, n - 1), kn, qn, vn, an, bn, gn);  // the next row's, on their way while this one is worked
    float kk = 0.f, qq = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kk += kc[r] * kc[r];
      qq += qc[r] * qc[r];
    }
    kk += ix_dpp<IX_DPP_XOR1>(kk);
    kk += ix_dpp<IX_DPP_XOR2>(kk);
    qq += ix_dpp<IX_DPP_XOR1>(qq);
    qq += ix_dpp<IX_DPP_XOR2>(qq);
    const float k_inv = 1.0f / sqrtf(kk + 1e-6f), q_inv = q_scale / sqrtf(qq + 1e-6f);
    const float x = ac + bias;
    const float softplus = x > 20.f ? x : log1pf(expf(x));
    const float g = expf(-rate * softplus);
    const float beta = 1.0f / (1.0f + expf(-bc));
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      if constexpr (CH) S[r] *= gc[r];
      else S[r] *= g;
      dot += S[r] * (kc[r] * k_inv);
    }
    dot += ix_dpp<IX_DPP_XOR1>(dot);
    dot += ix_dpp<IX_DPP_XOR2>(dot);
    const float u = beta * (vc - dot);
    float o = 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      S[r] += (kc[r] * k_inv) * u;
      o += S[r] * (qc[r] * q_inv);
    }
    o += ix_dpp<IX_DPP_XOR1>(o);
    o += ix_dpp<IX_DPP_XOR2>(o);
    if (live && part == 0) out[((row0 + i) * heads + head) * vdim + col] = o;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      kc[r] = kn[r];
      qc[r] = qn[r];
      if constexpr (CH) gc[r] = gn[r];
    }
    vc = vn;
    ac = an;
    bc = bn;
  }
  if (live) {
    if constexpr (VEC) {
#pragma unroll
      for (int r = 0; r < RPL; r += 4)
        if (r < quarter)
          *reinterpret_cast<delta_f32x4*>(sp + static_cast<int64_t>(col) * dim + part * quarter + r) =
              delta_f32x4{S[r], S[r + 1], S[r + 2], S[r + 3]};
    } else {
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        const int i = row_of(r);
        if (i < dim) sp[static_cast<int64_t>(col) * dim + i] = S[r];
      }
    }
  }
}

// The same recurrence for requests that bring many rows (prompt portions), bfloat16, heads of 32, 64 or 128 numbers.
// A wavefront at one wavefront per SIMD issues one vector instruction every few cycles, so what counts here is the
// number of instructions per row, and how many wavefronts share a head:
//   * the wavefront brings DELTA_CHUNK rows of its q/k head, its value columns and the two logits into LDS at a
//     time, all loads of a chunk in flight at once and a chunk ahead of the arithmetic (in registers while the
//     present chunk is worked);
//   * on the way into LDS the rows are made unit vectors (q also times dim^(-1/2)) and the logits become the decay
//     and the step size, once per row instead of once per lane and row;
//   * SP lanes share a column (4, or 16 where the head is a multiple of 64 numbers: four times the wavefronts, a
//     quarter of the rows each), RPL = dim / SP rows a lane.
// Per row and lane that leaves four sweeps over RPL numbers and two sums over SP lanes.  (The decay is applied to
// the product S^T k instead of to S first, which is the same number up to rounding.)
#define DELTA_CHUNK 32

template <int SP>
__device__ __forceinline__ float delta_sum_over(float x) {  // over the SP neighbouring lanes of a column
  x += ix_dpp<IX_DPP_XOR1>(x);
  x += ix_dpp<IX_DPP_XOR2>(x);
  if constexpr (SP >= 8) x += ix_dpp<IX_DPP_HALF_MIRROR>(x);
  if constexpr (SP >= 16) x += ix_dpp<IX_DPP_MIRROR>(x);
  return x;
}

template <int SP, int RPL, bool CH>
__global__ void __launch_bounds__(64)
delta_rule_chunk_kernel(const bf16_t* q, const bf16_t* k, const bf16_t* v, int64_t q_stride, int64_t k_stride,
                        int64_t v_stride, const float* ab, const float* ach, const float* __restrict__ a_log,
                        const float* __restrict__ dt_bias, float* __restrict__ state, int64_t state_stride,
                        const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                        float* __restrict__ out, int heads, int kv_heads, int vdim) {
  constexpr int DIM = SP * RPL;
  constexpr int COLS = 64 / SP;                      // value columns of a wavefront
  constexpr int PIECES = DIM / 8;                    // 16-byte pieces of a q or k row (4, 8 or 16: a power of two)
  constexpr int PER_LANE = DELTA_CHUNK * 2 * PIECES / 64;  // pieces of a chunk's q and k rows that a lane moves
  constexpr int V_PER_LANE = (DELTA_CHUNK * COLS + 63) / 64;
  __shared__ delta_f32x4 qk_s[DELTA_CHUNK][2][DIM / 4];  // [row][k, q]: unit vectors (q times dim^(-1/2))
  __shared__ float v_s[DELTA_CHUNK][COLS];
  __shared__ float gb_s[DELTA_CHUNK][2];             // decay, step size
  constexpr int G4 = DIM / 4;                        // 16-byte pieces of a row of decays (8, 16 or 32: divides 64)
  constexpr int G_PER_LANE = CH ? DELTA_CHUNK * G4 / 64 : 1;
  __shared__ delta_f32x4 g_s[CH ? DELTA_CHUNK : 1][CH ? G4 : 1];  // a decay per key channel: [row][channel]
  const int lane = threadIdx.x;
  const int col0 = blockIdx.x * COLS;
  const int col = col0 + lane / SP, part = lane % SP;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int kv = head / (heads / kv_heads);
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const bool live = col < vdim;
  const int cj = live ? col : vdim - 1;

  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride + static_cast<int64_t>(head) * DIM * vdim;
  float S[RPL];
#pragma unroll
  for (int r = 0; r < RPL; ++r) S[r] = sp[static_cast<int64_t>(cj) * DIM + part * RPL + r];
  const float rate = CH ? 0.f : expf(a_log[head]), bias = CH ? 0.f : dt_bias[head];
  const float q_scale = 1.0f / sqrtf(static_cast<float>(DIM));

  delta_u32x4 st_qk[PER_LANE];
  delta_f32x4 st_g[G_PER_LANE];
  float st_v[V_PER_LANE], st_ab;
  auto ask = [&](int first) {
    if constexpr (CH) {
#pragma unroll
      for (int u = 0; u < G_PER_LANE; ++u) {
        const int id = u * 64 + lane;
        const int64_t row = row0 + min(first + id / G4, n - 1);
        st_g[u] = *reinterpret_cast<const delta_f32x4*>(ach + (row * heads + head) * DIM + 4 * (id % G4));
      }
    }  // rows first .. first + DELTA_CHUNK - 1 of the portion (rows past its end repeat the last)
#pragma unroll
    for (int u = 0; u < PER_LANE; ++u) {
      const int id = u * 64 + lane;  // piece number within the chunk: [row][k, q][piece]
      const int r = id / (2 * PIECES), which = (id / PIECES) & 1, pc = id % PIECES;
      const int64_t row = row0 + min(first + r, n - 1);
      const bf16_t* src = which ? q + row * q_stride + kv * DIM : k + row * k_stride + kv * DIM;
      st_qk[u] = *reinterpret_cast<const delta_u32x4*>(src + 8 * pc);
    }
#pragma unroll
    for (int u = 0; u < V_PER_LANE; ++u) {
      const int id = min(u * 64 + lane, DELTA_CHUNK * COLS - 1);
      const int r = id / COLS, c = id % COLS;
      st_v[u] = ix_load(v + (row0 + min(first + r, n - 1)) * v_stride + head * vdim + min(col0 + c, vdim - 1));
    }
    {
      const int r = lane / 2, which = lane & 1;
      if constexpr (CH) st_ab = ab[(row0 + min(first + r, n - 1)) * heads + head];
      else st_ab = ab[(row0 + min(first + r, n - 1)) * 2 * heads + which * heads + head];
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int u = 0; u < PER_LANE; ++u) {
      const int id = u * 64 + lane;
      const int r = id / (2 * PIECES), which = (id / PIECES) & 1, pc = id % PIECES;
      float x[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x[2 * e] = __uint_as_float(st_qk[u][e] << 16);
        x[2 * e + 1] = __uint_as_float(st_qk[u][e] & 0xffff0000u);
      }
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
      ss = delta_sum_over<PIECES>(ss);  // a row's pieces lie in PIECES neighbouring lanes
      const float f = (which ? q_scale : 1.0f) / sqrtf(ss + 1e-6f);
      qk_s[r][which][2 * pc] = delta_f32x4{x[0] * f, x[1] * f, x[2] * f, x[3] * f};
      qk_s[r][which][2 * pc + 1] = delta_f32x4{x[4] * f, x[5] * f, x[6] * f, x[7] * f};
    }
#pragma unroll
    for (int u = 0; u < V_PER_LANE; ++u) {
      const int id = u * 64 + lane;
      if (id < DELTA_CHUNK * COLS) v_s[id / COLS][id % COLS] = st_v[u];
    }
    if (lane & 1) {
      gb_s[lane / 2][1] = 1.0f / (1.0f + expf(-st_ab));
    } else if constexpr (!CH) {
      const float x = st_ab + bias;
      gb_s[lane / 2][0] = expf(-rate * (x > 20.f ? x : log1pf(expf(x))));
    }
    if constexpr (CH) {
#pragma unroll
      for (int u = 0; u < G_PER_LANE; ++u) {
        const int id = u * 64 + lane;
        g_s[id / G4][id % G4] = st_g[u];
      }
    }
  };
  auto fetch = [&](int r, float (&kk)[RPL], float (&qq)[RPL], float& vv, float& gg, float& bb,
                   float (&gr)[CH ? RPL : 1]) {
    if constexpr (CH) {
#pragma unroll
      for (int j = 0; j < RPL / 4; ++j) {
        const delta_f32x4 a = g_s[r][part * (RPL / 4) + j];
#pragma unroll
        for (int e = 0; e < 4; ++e) gr[4 * j + e] = a[e];
      }
    }
#pragma unroll
    for (int j = 0; j < RPL / 4; ++j) {
      const delta_f32x4 a = qk_s[r][0][part * (RPL / 4) + j], b = qk_s[r][1][part * (RPL / 4) + j];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        kk[4 * j + e] = a[e];
        qq[4 * j + e] = b[e];
      }
    }
    vv = v_s[r][lane / SP];
    gg = CH ? 1.0f : gb_s[r][0];
    bb = gb_s[r][1];
  };

  ask(0);
  for (int first = 0; first < n; first += DELTA_CHUNK) {
    __syncthreads();  // the chunk before has been read
    put();
    __syncthreads();
    if (first + DELTA_CHUNK < n) ask(first + DELTA_CHUNK);  // on their way while this chunk is worked
    __builtin_amdgcn_sched_barrier(0);
    const int rows = min(DELTA_CHUNK, n - first);
    float kc[RPL], qc[RPL], vc, gc, bc, grc[CH ? RPL : 1];
    fetch(0, kc, qc, vc, gc, bc, grc);
    for (int i = 0; i < rows; ++i) {
      float kn[RPL], qn[RPL], vn, gn, bn, grn[CH ? RPL : 1];
      fetch(min(i + 1, DELTA_CHUNK - 1), kn, qn, vn, gn, bn, grn);
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        if constexpr (CH) S[r] *= grc[r];
        dot += S[r] * kc[r];
      }
      dot = delta_sum_over<SP>(dot);
      const float u = bc * (vc - gc * dot);
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        S[r] = fmaf(S[r], gc, kc[r] * u);
        o += S[r] * qc[r];
      }
      o = delta_sum_over<SP>(o);
      if (live && part == 0) out[((row0 + first + i) * heads + head) * vdim + col] = o;
#pragma unroll
      for (int r = 0; r < RPL; ++r) {
        kc[r] = kn[r];
        qc[r] = qn[r];
        if constexpr (CH) grc[r] = grn[r];
      }
      vc = vn;
      gc = gn;
      bc = bn;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < RPL; ++r) sp[static_cast<int64_t>(col) * DIM + part * RPL + r] = S[r];
  }
}

// q, k [T, kv_heads * dim] and v [T, heads * vdim] of the run's type with their row strides; ab float32 [T, 2 heads]
// (a then b); a_log, dt_bias float32 [heads]; or, with a decay per key channel, ach float32 [T, heads * dim] (the
// decays themselves) and ab float32 [T, heads] (b alone); state: slot s at state + s * state_stride, [heads, vdim, dim] (a column's rows side by side);
// out float32 [T, heads, vdim].
extern "C" int ix_delta_rule(const void* q, const void* k, const void* v, int dtype, int64_t q_stride,
                             int64_t k_stride, int64_t v_stride, const float* ab, const float* ach, const float* a_log,
                             const float* dt_bias, float* state, int64_t state_stride, const int32_t* q_start,
                             const int32_t* state_slots, float* out, int64_t tokens, int requests, int heads,
                             int kv_heads, int dim, int vdim, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && requests >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "sizes must be positive");
  IX_REQUIRE(heads % kv_heads == 0, "heads must be a multiple of kv_heads");
  IX_REQUIRE(dim <= 256, "at most 256 numbers per query and key head");
  IX_REQUIRE(state_stride >= static_cast<int64_t>(heads) * dim * vdim, "state blocks too small");
  IX_REQUIRE(heads <= 65535 && requests <= 65535, "too many heads or requests for one launch");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  if (tokens == 0 || requests == 0) return 0;
  dim3 grid((vdim + DELTA_COLS - 1) / DELTA_COLS, heads, requests), block(64);
  const int rpl = (dim + DELTA_SPLIT - 1) / DELTA_SPLIT;
  // 16-byte pieces: a lane's quarter of a head is a multiple of eight numbers, and rows and heads start aligned
  const int elt = 2;
  const bool vec = dtype == IX_BF16 && dim % (8 * DELTA_SPLIT) == 0 && (q_stride * elt) % 16 == 0 && (k_stride * elt) % 16 == 0 &&
                   state_stride % 4 == 0 &&
                   ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(state) |
                     reinterpret_cast<uintptr_t>(ach)) & 15) == 0;
#define LAUNCH_CH(TT, RPL, VEC, CH)                                                                                         \
  hipLaunchKernelGGL((delta_rule_kernel<TT, RPL, VEC, CH>), grid, block, 0, stream, (const TT*)q, (const TT*)k, (const TT*)v, \
                     q_stride, k_stride, v_stride, ab, ach, a_log, dt_bias, state, state_stride, q_start, state_slots, out,   \
                     heads, kv_heads, dim, vdim)
#define LAUNCH(TT, RPL, VEC)                \
  do {                                      \
    if (ach) LAUNCH_CH(TT, RPL, VEC, true); \
    else LAUNCH_CH(TT, RPL, VEC, false);    \
  } while (0)
#define PICK(TT, VEC)                      \
  if (rpl <= 8) LAUNCH(TT, 8, VEC);        \
  else if (rpl <= 16) LAUNCH(TT, 16, VEC); \
  else if (rpl <= 32) LAUNCH(TT, 32, VEC); \
  else LAUNCH(TT, 64, VEC);
  // steps that bring a request many rows: chunks through LDS (heads of 32, 64 or 128 numbers)
  if (vec && tokens >= 4 * static_cast<int64_t>(requests) && (dim == 32 || dim == 64 || dim == 128)) {
#define CHUNKED_CH(SP, RPL, CH)                                                                                               \
  hipLaunchKernelGGL((delta_rule_chunk_kernel<SP, RPL, CH>), dim3((vdim + 64 / SP - 1) / (64 / SP), heads, requests), block, \
                     0, stream, (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, q_stride, k_stride, v_stride, ab, ach, \
                     a_log, dt_bias, state, state_stride, q_start, state_slots, out, heads, kv_heads, vdim)
#define CHUNKED(SP, RPL)                \
  do {                                  \
    if (ach) CHUNKED_CH(SP, RPL, true); \
    else CHUNKED_CH(SP, RPL, false);    \
  } while (0)
    if (dim == 32) CHUNKED(4, 8);
    else if (dim == 64) CHUNKED(16, 4);
    else CHUNKED(16, 8);
#undef CHUNKED
#undef CHUNKED_CH
    return ix_check_launch("ix_delta_rule");
  }
  // (the 16-byte form is built for bfloat16, the type whose runs are timed)
  if (dtype == IX_F32) { PICK(float, false) } else if (vec) { PICK(bf16_t, true) } else { PICK(bf16_t, false) }
#undef PICK
#undef LAUNCH
#undef LAUNCH_CH
  return ix_check_launch("ix_delta_rule");
}

// x[t, h, i] <- exp(-exp(a_log[h]) softplus(x[t, h, i] + dt_bias[h, i])) in place: the decays per key channel
// from their logits, float32 [T, heads * dim].
__global__ void channel_decays_kernel(float* __restrict__ x, const float* __restrict__ a_log,
                                      const float* __restrict__ dt_bias, int64_t n, int heads, int dim) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int c = static_cast<int>(i % (static_cast<int64_t>(heads) * dim));
    const float v = x[i] + dt_bias[c];
    x[i] = expf(-expf(a_log[c / dim]) * (v > 20.f ? v : log1pf(expf(v))));
  }
}

extern "C" int ix_channel_decays(float* x, const float* a_log, const float* dt_bias, int64_t tokens, int heads, int dim,
                                 hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && dim > 0, "sizes must be positive");
  if (tokens == 0) return 0;
  const int64_t n = tokens * heads * dim;
  hipLaunchKernelGGL(channel_decays_kernel, dim3(static_cast<unsigned>(std::min<int64_t>((n + 255) / 256, 65536))), dim3(256), 0,
                     stream, x, a_log, dt_bias, n, heads, dim);
  return ix_check_launch("ix_channel_decays");
}

// ---------------------------------------------------------------------------
// What follows a mixer whose heads are normalised one by one, a wavefront per (token, head):
//
//   o = x - lambda x2  (x2 optional);  y = o / sqrt(mean(o^2) + eps) * weight (optional) * silu(gate) (optional) * mult
//
// With `den_a` (float32, one number per (token, head)) x is first divided by max(|den_a|, den_b) + 1e-6, den_b the
// number at den_b[(t * heads + head) * den_b_stride] (a read-out that is normalised by its own size).
//
// x, x2 float32 [T, heads, vdim]; weight [vdim], shared by the heads (or [heads, vdim] with `weight_per_head`);
// `gate_sigmoid`: sigmoid(gate) instead of silu(gate); gate of the run's type at
// gate[t * gate_stride + head * vdim + j]; out of the run's type [T, heads * vdim].
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(const float* __restrict__ x, const float* __restrict__ x2, float lambda,
                      const void* __restrict__ weight, int w_dtype, const T* __restrict__ gate, int64_t gate_stride,
                      T* __restrict__ out, int64_t pairs, int heads, int vdim, float eps, float mult,
                      int weight_per_head, int gate_sigmoid, const float* __restrict__ den_a,
                      const float* __restrict__ den_b, int den_b_stride) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = p / heads;
  const int head = static_cast<int>(p % heads);
  const float* xr = x + p * vdim;
  const float* x2r = x2 ? x2 + p * vdim : nullptr;
  const float pre = den_a ? 1.0f / (fmaxf(fabsf(den_a[p]), den_b[p * den_b_stride]) + 1e-6f) : 1.0f;
  float ss = 0.f;
  for (int j = lane; j < vdim; j += 64) {
    const float o = (x2r ? xr[j] - lambda * x2r[j] : xr[j]) * pre;
    ss += o * o;
  }
  ss = ix_wave_sum(ss);
  const float inv = pre * mult / sqrtf(ss / static_cast<float>(vdim) + eps);
  for (int j = lane; j < vdim; j += 64) {
    float y = (x2r ? xr[j] - lambda * x2r[j] : xr[j]) * inv;
    if (weight) y *= ix_load_rt(weight, w_dtype, weight_per_head ? head * vdim + j : j);
    if (gate) {
      const float gv = ix_load(gate + t * gate_stride + head * vdim + j);
      y *= (gate_sigmoid ? 1.0f : gv) / (1.0f + expf(-gv));
    }
    ix_store(out + p * vdim + j, y);
  }
}

// The same for wide rows (one norm over all heads' columns together: hundreds or thousands of numbers): a
// workgroup per (token, head), so that a row's numbers are in flight at once instead of sixty-four at a time.
template <typename T>
__global__ void __launch_bounds__(256)
head_norm_gate_wide_kernel(const float* __restrict__ x, const float* __restrict__ x2, float lambda,
                           const void* __restrict__ weight, int w_dtype, const T* __restrict__ gate,
                           int64_t gate_stride, T* __restrict__ out, int heads, int vdim, float eps, float mult,
                           int weight_per_head, int gate_sigmoid, const float* __restrict__ den_a,
                           const float* __restrict__ den_b, int den_b_stride) {
  __shared__ float red[16];
  const int64_t p = blockIdx.x;
  const int64_t t = p / heads;
  const int head = static_cast<int>(p % heads);
  const float* xr = x + p * vdim;
  const float* x2r = x2 ? x2 + p * vdim : nullptr;
  const float pre = den_a ? 1.0f / (fmaxf(fabsf(den_a[p]), den_b[p * den_b_stride]) + 1e-6f) : 1.0f;
  float ss = 0.f;
  for (int j = threadIdx.x; j < vdim; j += 256) {
    const float o = (x2r ? xr[j] - lambda * x2r[j] : xr[j]) * pre;
    ss += o * o;
  }
  ss = ix_block_sum(ss, red);
  const float inv = pre * mult / sqrtf(ss / static_cast<float>(vdim) + eps);
  for (int j = threadIdx.x; j < vdim; j += 256) {
    float y = (x2r ? xr[j] - lambda * x2r[j] : xr[j]) * inv;
    if (weight) y *= ix_load_rt(weight, w_dtype, weight_per_head ? head * vdim + j : j);
    if (gate) {
      const float gv = ix_load(gate + t * gate_stride + head * vdim + j);
      y *= (gate_sigmoid ? 1.0f : gv) / (1.0f + expf(-gv));
    }
    ix_store(out + p * vdim + j, y);
  }
}

extern "C" int ix_head_norm_gate(const float* x, const float* x2, float lambda, const void* weight, int w_dtype,
                                 const void* gate, int64_t gate_stride, void* out, int dtype, int64_t tokens,
                                 int heads, int vdim, float eps, float mult, int weight_per_head, int gate_sigmoid,
                                 const float* den_a, const float* den_b, int den_b_stride, hipStream_t stream) {
  IX_REQUIRE(tokens >= 0 && heads > 0 && vdim > 0, "sizes must be positive");
  IX_REQUIRE(den_a == nullptr || (den_b != nullptr && den_b_stride > 0), "a divisor comes as two numbers per row");
  IX_REQUIRE(dtype == IX_F32 || dtype == IX_BF16, "dtype must be float32 or bfloat16");
  if (tokens == 0) return 0;
  const int64_t pairs = tokens * heads;
  IX_REQUIRE((pairs + 3) / 4 < (1ll << 31), "too many rows for one launch");
  if (vdim >= 512) {
    IX_REQUIRE(pairs < (1ll << 31), "too many rows for one launch");
    dim3 wide(static_cast<unsigned>(pairs)), threads(256);
    if (dtype == IX_F32)
      hipLaunchKernelGGL(head_norm_gate_wide_kernel<float>, wide, threads, 0, stream, x, x2, lambda, weight, w_dtype,
                         (const float*)gate, gate_stride, (float*)out, heads, vdim, eps, mult, weight_per_head,
                         gate_sigmoid, den_a, den_b, den_b_stride);
    else
      hipLaunchKernelGGL(head_norm_gate_wide_kernel<bf16_t>, wide, threads, 0, stream, x, x2, lambda, weight, w_dtype,
                         (const bf16_t*)gate, gate_stride, (bf16_t*)out, heads, vdim, eps, mult, weight_per_head,
                         gate_sigmoid, den_a, den_b, den_b_stride);
    return ix_check_launch("ix_head_norm_gate");
  }
  dim3 grid(static_cast<unsigned>((pairs + 3) / 4)), block(256);
  if (dtype == IX_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, x, x2, lambda, weight, w_dtype,
                       (const float*)gate, gate_stride, (float*)out, pairs, heads, vdim, eps, mult, weight_per_head,
                       gate_sigmoid, den_a, den_b, den_b_stride);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, x, x2, lambda, weight, w_dtype,
                       (const bf16_t*)gate, gate_stride, (bf16_t*)out, pairs, heads, vdim, eps, mult, weight_per_head,
                       gate_sigmoid, den_a, den_b, den_b_stride);
  return ix_check_launch("ix_head_norm_gate");
}
