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

__device__ __forceinline__ void ls_load8(const float* p, float (&o)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
  o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
__device__ __forceinline__ void ls_load8(const bf16_t* p, float (&o)[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  o[0] = __uint_as_float(a.x << 16); o[1] = __uint_as_float(a.x & 0xffff0000u);
  o[2] = __uint_as_float(a.y << 16); o[3] = __uint_as_float(a.y & 0xffff0000u);
  o[4] = __uint_as_float(a.z << 16); o[5] = __uint_as_float(a.z & 0xffff0000u);
  o[6] = __uint_as_float(a.w << 16); o[7] = __uint_as_float(a.w & 0xffff0000u);
}

// eight consecutive numbers as they come from memory, opened into floats when they are used
template <typename T> struct ls_piece;
template <> struct ls_piece<float> { float4 a, b; };
template <> struct ls_piece<bf16_t> { uint4 a; };
__device__ __forceinline__ void ls_ask8(const float* p, ls_piece<float>& o) {
  o.a = *reinterpret_cast<const float4*>(p);
  o.b = *reinterpret_cast<const float4*>(p + 4);
}
__device__ __forceinline__ void ls_ask8(const bf16_t* p, ls_piece<bf16_t>& o) { o.a = *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ void ls_open8(const ls_piece<float>& x, float (&o)[8]) {
  o[0] = x.a.x; o[1] = x.a.y; o[2] = x.a.z; o[3] = x.a.w;
  o[4] = x.b.x; o[5] = x.b.y; o[6] = x.b.z; o[7] = x.b.w;
}
__device__ __forceinline__ void ls_open8(const ls_piece<bf16_t>& x, float (&o)[8]) {
  o[0] = __uint_as_float(x.a.x << 16); o[1] = __uint_as_float(x.a.x & 0xffff0000u);
  o[2] = __uint_as_float(x.a.y << 16); o[3] = __uint_as_float(x.a.y & 0xffff0000u);
  o[4] = __uint_as_float(x.a.z << 16); o[5] = __uint_as_float(x.a.z & 0xffff0000u);
  o[6] = __uint_as_float(x.a.w << 16); o[7] = __uint_as_float(x.a.w & 0xffff0000u);
}

// R: rows of a column per lane (4 R >= dim).  VEC: dim = 4 R, R a multiple of 8 and everything on 16-byte boundaries,
// so that a lane reads its part of the state and of every operand in 16-byte pieces.
template <typename T, int R, bool VEC>
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
  if constexpr (VEC) {
#pragma unroll
    for (int i = 0; i < R; i += 4) {
      const float4 x = live ? *reinterpret_cast<const float4*>(sp + row0 + i) : float4{0.f, 0.f, 0.f, 0.f};
      s[i] = x.x; s[i + 1] = x.y; s[i + 2] = x.z; s[i + 3] = x.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) s[i] = (live && row0 + i < dim) ? sp[row0 + i] : 0.f;
  }
  const float wh = w_head ? w_head[head] : 1.0f;
  const int64_t ch = static_cast<int64_t>(head) * dim;  // first key channel of this head
  for (int t = t0; t < t1; ++t) {
    float rr[R], kk[R], ww[R], aa[R], bb[R];
    if constexpr (VEC) {
      const int64_t c = ch + row0, at = static_cast<int64_t>(t) * heads * dim + c;
#pragma unroll
      for (int i = 0; i < R; i += 8) {
        float x[8], y[8];
        ls_load8(r + t * r_stride + c + i, x);
        ls_load8(k + t * k_stride + c + i, y);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          rr[i + e] = silu ? ls_silu(x[e]) : x[e];
          kk[i + e] = silu ? ls_silu(y[e]) : y[e];
        }
      }
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const float4 w4 = w_rows ? *reinterpret_cast<const float4*>(w_rows + at + i) : float4{wh, wh, wh, wh};
        const float4 a4 = a_rows ? *reinterpret_cast<const float4*>(a_rows + at + i) : float4{0.f, 0.f, 0.f, 0.f};
        const float4 b4 = b_rows ? *reinterpret_cast<const float4*>(b_rows + at + i) : float4{0.f, 0.f, 0.f, 0.f};
        ww[i] = w4.x; ww[i + 1] = w4.y; ww[i + 2] = w4.z; ww[i + 3] = w4.w;
        aa[i] = a4.x; aa[i + 1] = a4.y; aa[i + 2] = a4.z; aa[i + 3] = a4.w;
        bb[i] = b4.x; bb[i + 1] = b4.y; bb[i + 2] = b4.z; bb[i + 3] = b4.w;
      }
    } else
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
    if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < R; i += 4) *reinterpret_cast<float4*>(sp + row0 + i) = float4{s[i], s[i + 1], s[i + 2], s[i + 3]};
    } else {
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (row0 + i < dim) sp[row0 + i] = s[i];
    }
  }
}

// The same recurrence for requests that bring many rows (prompt portions).  The operands of a row are the same for
// every column of a head, so a workgroup (THREADS / 64 wavefronts) shares them: it brings CH rows of r and k (and of
// w, a, b) into LDS at a time, as float32 and through silu where asked, all loads of a chunk in flight at once and a
// chunk ahead of the arithmetic.  SP lanes share a column (RPL = dim / SP rows each, in registers), so a workgroup
// owns THREADS / SP columns, and a row costs a lane five (or two) reads of RPL numbers from LDS, three sweeps over
// them and two sums over SP lanes (DPP all the way: within a row of 16 lanes, then row_bcast15 and row_bcast31
// across rows, the total taken from the last lane).  The rows are a chain, so what counts is how few instructions
// a row is and how many wavefronts there are: heads of 64 numbers take 32 lanes a column, heads of 128 a whole
// wavefront while that makes at most two wavefronts a SIMD (2,048 for 16 heads of 128 columns), else 32 lanes.
// CORR: w, a, b come per row and channel; else the decay is one number per head.

template <int SP>
__device__ __forceinline__ float ls_sum_over(float x) {  // over the SP neighbouring lanes of a column
  x += ix_dpp<IX_DPP_XOR1>(x);
  x += ix_dpp<IX_DPP_XOR2>(x);
  if constexpr (SP >= 8) x += ix_dpp<IX_DPP_HALF_MIRROR>(x);
  if constexpr (SP >= 16) x += ix_dpp<IX_DPP_MIRROR>(x);
  if constexpr (SP >= 64) {
    // all four rows of 16 lanes: rows 1 and 3 take the row before, rows 2 and 3 the first pair's total (row_bcast31:
    // lane 31, for rows 2 and 3); the last lane's total goes to all lanes as a scalar
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x143, 0xc, 0xf, false));
    x = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
  } else if constexpr (SP >= 32) {
    // rows of 16 lanes in pairs: the odd row takes the even row's total through DPP (row_bcast15: lane 15 of the
    // row before, for rows 1 and 3), and the pair's total goes from its last lane to all of its lanes as a scalar
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));
    const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 31));
    const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
    x = (threadIdx.x & 32) ? hi : lo;
  }
  return x;
}

// the same sum where only the last of the SP lanes needs it
template <int SP>
__device__ __forceinline__ float ls_sum_last(float x) {
  x += ix_dpp<IX_DPP_XOR1>(x);
  x += ix_dpp<IX_DPP_XOR2>(x);
  if constexpr (SP >= 8) x += ix_dpp<IX_DPP_HALF_MIRROR>(x);
  if constexpr (SP >= 16) x += ix_dpp<IX_DPP_MIRROR>(x);
  if constexpr (SP >= 32)
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));
  if constexpr (SP >= 64)
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x143, 0xc, 0xf, false));
  return x;
}

template <typename T, int SP, int RPL, bool CORR, int CH, int THREADS>  // CH: rows per chunk; THREADS per workgroup
__global__ void __launch_bounds__(THREADS)
linear_state_chunk_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, int64_t r_stride,
                          int64_t k_stride, int64_t v_stride, const float* __restrict__ w_rows,
                          const float* __restrict__ w_head, const float* __restrict__ a_rows,
                          const float* __restrict__ b_rows, float* __restrict__ state, int64_t state_stride,
                          const int32_t* __restrict__ q_start, const int32_t* __restrict__ state_slots,
                          float* __restrict__ out, int heads, int vdim, int silu) {
  constexpr int DIM = SP * RPL;
  constexpr int COLS = THREADS / SP;                 // value columns of a workgroup
  constexpr int P8 = DIM / 8, P4 = DIM / 4;             // pieces of a row: of eight numbers (r, k), of four (w, a, b)
  constexpr int RK_PIECES = CH * 2 * P8;
  constexpr int RK_PER = (RK_PIECES + THREADS - 1) / THREADS;
  constexpr int WAB_PIECES = CORR ? CH * 3 * P4 : 0;
  constexpr int WAB_PER = CORR ? (WAB_PIECES + THREADS - 1) / THREADS : 1;
  constexpr int V_PER = (CH * COLS + THREADS - 1) / THREADS;
  __shared__ float4 rk_s[CH][2][P4];              // [row][k, r]
  __shared__ float4 wab_s[CORR ? CH : 1][3][P4];  // [row][w, a, b]
  __shared__ float v_s[CH][COLS];
  const int tid = threadIdx.x;
  const int col0 = blockIdx.x * COLS;
  const int col = col0 + tid / SP, part = tid % SP;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int64_t row0 = q_start[seq];
  const int n = q_start[seq + 1] - static_cast<int>(row0);
  if (n <= 0) return;
  const bool live = col < vdim;
  const int cj = live ? col : vdim - 1;  // lanes past the last column repeat it and store nothing
  float* sp = state + static_cast<int64_t>(state_slots[seq]) * state_stride +
              (static_cast<int64_t>(head) * vdim + cj) * DIM + part * RPL;
  // RPL numbers that lie side by side (RPL is 2 or a multiple of 4), to and from registers
  auto take = [](const float* src, float (&dst)[RPL]) {
    if constexpr (RPL == 2) {
      const float2 x = *reinterpret_cast<const float2*>(src);
      dst[0] = x.x; dst[1] = x.y;
    } else {
#pragma unroll
      for (int i = 0; i < RPL; i += 4) {
        const float4 x = *reinterpret_cast<const float4*>(src + i);
        dst[i] = x.x; dst[i + 1] = x.y; dst[i + 2] = x.z; dst[i + 3] = x.w;
      }
    }
  };
  float S[RPL];
  take(sp, S);
  const float wh = CORR ? 1.0f : w_head[head];
  const int64_t chan = static_cast<int64_t>(heads) * DIM;  // channels of a row of w, a, b

  ls_piece<T> st_rk[RK_PER];
  float st_v[V_PER];
  float4 st_wab[WAB_PER];
  auto ask = [&](int first) {  // rows first .. first + CH - 1 of the portion (rows past its end repeat the last)
#pragma unroll
    for (int u = 0; u < RK_PER; ++u) {
      const int id = min(u * THREADS + tid, RK_PIECES - 1);
      const int row = id / (2 * P8), which = (id / P8) & 1, pc = id % P8;
      const int64_t at = row0 + min(first + row, n - 1);
      ls_ask8((which ? r + at * r_stride : k + at * k_stride) + head * DIM + 8 * pc, st_rk[u]);
    }
    if constexpr (CORR) {
#pragma unroll
      for (int u = 0; u < WAB_PER; ++u) {
        const int id = min(u * THREADS + tid, WAB_PIECES - 1);
        const int row = id / (3 * P4), which = (id / P4) % 3, pc = id % P4;
        const float* src = which == 0 ? w_rows : (which == 1 ? a_rows : b_rows);
        st_wab[u] = *reinterpret_cast<const float4*>(src + (row0 + min(first + row, n - 1)) * chan + head * DIM + 4 * pc);
      }
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int id = min(u * THREADS + tid, CH * COLS - 1);
      const int row = id / COLS, c = id % COLS;
      st_v[u] = ix_load(v + (row0 + min(first + row, n - 1)) * v_stride + head * vdim + min(col0 + c, vdim - 1));
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int u = 0; u < RK_PER; ++u) {
      const int id = u * THREADS + tid;
      if (id < RK_PIECES) {
        const int row = id / (2 * P8), which = (id / P8) & 1, pc = id % P8;
        float x[8];
        ls_open8(st_rk[u], x);
        if (silu) {
#pragma unroll
          for (int e = 0; e < 8; ++e) x[e] = ls_silu(x[e]);
        }
        rk_s[row][which][2 * pc] = float4{x[0], x[1], x[2], x[3]};
        rk_s[row][which][2 * pc + 1] = float4{x[4], x[5], x[6], x[7]};
      }
    }
    if constexpr (CORR) {
#pragma unroll
      for (int u = 0; u < WAB_PER; ++u) {
        const int id = u * THREADS + tid;
        if (id < WAB_PIECES) wab_s[id / (3 * P4)][(id / P4) % 3][id % P4] = st_wab[u];
      }
    }
#pragma unroll
    for (int u = 0; u < V_PER; ++u) {
      const int id = u * THREADS + tid;
      if (id < CH * COLS) v_s[id / COLS][id % COLS] = silu ? ls_silu(st_v[u]) : st_v[u];
    }
  };
  auto fetch = [&](int row, float (&kk)[RPL], float (&rr)[RPL], float (&ww)[RPL], float (&aa)[RPL], float (&bb)[RPL],
                   float& vv) {
    take(reinterpret_cast<const float*>(&rk_s[row][0][0]) + part * RPL, kk);
    take(reinterpret_cast<const float*>(&rk_s[row][1][0]) + part * RPL, rr);
    if constexpr (CORR) {
      take(reinterpret_cast<const float*>(&wab_s[row][0][0]) + part * RPL, ww);
      take(reinterpret_cast<const float*>(&wab_s[row][1][0]) + part * RPL, aa);
      take(reinterpret_cast<const float*>(&wab_s[row][2][0]) + part * RPL, bb);
    }
    vv = v_s[row][tid / SP];
  };

  ask(0);
  for (int first = 0; first < n; first += CH) {
    __syncthreads();  // the chunk before has been read
    put();
    __syncthreads();
    if (first + CH < n) ask(first + CH);  // on their way while this chunk is worked
    __builtin_amdgcn_sched_barrier(0);
    const int rows = min(CH, n - first);
    float kc[RPL], rc[RPL], wc[RPL], ac[RPL], bc[RPL];
    float vc;
    fetch(0, kc, rc, wc, ac, bc, vc);
    float* op = out + ((row0 + first) * heads + head) * vdim + (live ? col : 0);
    const int64_t o_step = static_cast<int64_t>(heads) * vdim;
    auto row_step = [&](int i) {
      float kn[RPL], rn[RPL], wn[RPL], an[RPL], bn[RPL];
      float vn;
      fetch(min(i + 1, CH - 1), kn, rn, wn, an, bn, vn);
      float read = 0.f;
      if constexpr (CORR) {
#pragma unroll
        for (int j = 0; j < RPL; ++j) read += bc[j] * S[j];
        read = ls_sum_over<SP>(read);
      }
      float o = 0.f;
#pragma unroll
      for (int j = 0; j < RPL; ++j) {
        if constexpr (CORR) S[j] = wc[j] * S[j] - ac[j] * read + kc[j] * vc;
        else S[j] = wh * S[j] + kc[j] * vc;
        o += rc[j] * S[j];
      }
      o = ls_sum_last<SP>(o);
      if (live && part == SP - 1) op[i * o_step] = o;
#pragma unroll
      for (int j = 0; j < RPL; ++j) {
        kc[j] = kn[j];
        rc[j] = rn[j];
        if constexpr (CORR) {
          wc[j] = wn[j];
          ac[j] = an[j];
          bc[j] = bn[j];
        }
      }
      vc = vn;
    };
    // a whole chunk with the rows' places in LDS known when the code is built (eight rows a turn of the loop: the
    // copies from one row's operands to the next become names, the addresses constants); the last chunk row by row
    if (rows == CH) {
#pragma unroll 8
      for (int i = 0; i < CH; ++i) row_step(i);
    } else {
      for (int i = 0; i < rows; ++i) row_step(i);
    }
  }
  if (live) {
    if constexpr (RPL == 2) {
      *reinterpret_cast<float2*>(sp) = float2{S[0], S[1]};
    } else {
#pragma unroll
      for (int i = 0; i < RPL; i += 4) *reinterpret_cast<float4*>(sp + i) = float4{S[i], S[i + 1], S[i + 2], S[i + 3]};
    }
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
  // steps that bring a request many rows: chunks through LDS, where a head's keys are 16 .. 128 numbers, the
  // operands come in the two usual combinations, and every row starts on a 16-byte boundary
  bool vec16 = false;
  {
    const int elt = dtype == IX_F32 ? 4 : 2;
    const bool corr = w_rows != nullptr && a_rows != nullptr;
    const bool none = w_head != nullptr && a_rows == nullptr;
    const uintptr_t all = reinterpret_cast<uintptr_t>(r) | reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(state) |
                          reinterpret_cast<uintptr_t>(w_rows) | reinterpret_cast<uintptr_t>(a_rows) |
                          reinterpret_cast<uintptr_t>(b_rows);
    const bool aligned = (all & 15) == 0 && (r_stride * elt) % 16 == 0 && (k_stride * elt) % 16 == 0 && state_stride % 4 == 0;
    vec16 = aligned;
    if ((dtype == IX_F32 || dtype == IX_BF16) && (corr || none) && aligned && tokens >= 4 * static_cast<int64_t>(requests) &&
        (dim == 16 || dim == 32 || dim == 64 || dim == 128)) {
#define CHUNKED(T, SP, RPL, CORR, THREADS)                                                                               \
  hipLaunchKernelGGL((linear_state_chunk_kernel<T, SP, RPL, CORR, (CORR ? (SP * RPL >= 128 ? 16 : 32) : 64), THREADS>),  \
                     dim3((vdim + THREADS / SP - 1) / (THREADS / SP), heads, requests), dim3(THREADS), 0, stream,        \
                     (const T*)r, (const T*)k, (const T*)v, r_stride, k_stride, v_stride, w_rows, w_head, a_rows, b_rows, \
                     state, state_stride, q_start, state_slots, out, heads, vdim, silu)
#define BY_DIM(T, CORR)                                 \
  if (dim == 16) CHUNKED(T, 4, 4, CORR, 256);           \
  else if (dim == 32) CHUNKED(T, 8, 4, CORR, 256);      \
  else if (dim == 64) CHUNKED(T, 32, 2, CORR, 256);     \
  else if (static_cast<int64_t>(heads) * vdim >= 4096) CHUNKED(T, 32, 4, CORR, 256); \
  else CHUNKED(T, 64, 2, CORR, 512) /* few columns: a wavefront each, two wavefronts a SIMD at 2,048 of them */
      if (dtype == IX_F32) {
        if (corr) { BY_DIM(float, true); } else { BY_DIM(float, false); }
      } else {
        if (corr) { BY_DIM(bf16_t, true); } else { BY_DIM(bf16_t, false); }
      }
#undef BY_DIM
#undef CHUNKED
      return ix_check_launch("ix_linear_state");
    }
  }
  dim3 grid((vdim + 15) / 16, heads, requests), block(64);
#define LAUNCH(T, R, VEC)                                                                                          \
  hipLaunchKernelGGL((linear_state_kernel<T, R, VEC>), grid, block, 0, stream, (const T*)r, (const T*)k,             \
                     (const T*)v, r_stride, k_stride, v_stride, w_rows, w_head, a_rows, b_rows, state, state_stride, \
                     q_start, state_slots, out, heads, dim, vdim, silu)
#define PICK(T)                                              \
  if (vec16 && dim == 32) LAUNCH(T, 8, true);                \
  else if (vec16 && dim == 64) LAUNCH(T, 16, true);          \
  else if (vec16 && dim == 128) LAUNCH(T, 32, true);         \
  else if (vec16 && dim == 256) LAUNCH(T, 64, true);         \
  else if (dim <= 16) LAUNCH(T, 4, false);                   \
  else if (dim <= 32) LAUNCH(T, 8, false);                   \
  else if (dim <= 64) LAUNCH(T, 16, false);                  \
  else if (dim <= 128) LAUNCH(T, 32, false);                 \
  else LAUNCH(T, 64, false)
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
