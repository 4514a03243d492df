// The gated delta rule: a matrix S [d, dv] a head that every token decays and then corrects
// towards its own value,
//
//   S <- g_t S;   w = beta_t (v_t - S^T k_t);   S <- S + k_t w^T;   o_t = S^T q_t
//
// with one decay g_t = exp(-exp(A) softplus(z_a + dt)) and one step size beta_t = sigmoid(z_b) a
// head and token, and the short convolutions that feed it.  All arithmetic is 32-bit.
//
//  * short_conv        rows of a projection -> silu(causal convolution over time a channel); the
//                      leading channels are heads that are made unit vectors (and the first of
//                      those multiplied by a scale).  The taps - 1 rows before a step come from the
//                      request's state.
//  * short_conv_state  the state takes the step's last taps - 1 rows.
//  * delta_recurrence  the recurrence over the rows of a step, sequence by sequence.
//
// With r = S^T k and p = S^T q of the matrix *before* the token (both formed in one pass over
// it), w = beta (v - g r), o = g p + (q . k) w and S <- g S + k w^T: the same numbers as the
// four lines above with one pass over S less.
#include "zf_common.h"

__device__ __forceinline__ float dl_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float dl_softplus(float z) {
  return z > 20.f ? z : log1pf(expf(z));
}

// The sum over the CG lanes (a power of two up to 64, aligned) that share a
// column, in every one of them, through the data-parallel lane moves: neighbours, pairs, then the
// mirrored half row and row (a lane and its mirror hold sums over different halves).
template <int CTRL>
__device__ __forceinline__ float dl_move(float v) {
  // (every lane has a source lane: the value a lane without one would keep is never used)
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL,
                                                    0xf, 0xf, true));
}
template <int CG>
__device__ __forceinline__ float dl_lanes_sum(float v) {
  if constexpr (CG >= 2) v += dl_move<0xB1>(v);      // quad_perm [1, 0, 3, 2]
  if constexpr (CG >= 4) v += dl_move<0x4E>(v);      // quad_perm [2, 3, 0, 1]
  if constexpr (CG >= 8) v += dl_move<0x141>(v);     // row_half_mirror
  if constexpr (CG >= 16) v += dl_move<0x140>(v);    // row_mirror
  if constexpr (CG >= 32) {
    // rows of 16 lanes in pairs: one copy takes its odd rows from the other's even rows and
    // gives its own odd rows for them, so the two copies hold a pair's two rows lane by lane
    typedef unsigned int dl_u2 __attribute__((ext_vector_type(2)));
    const dl_u2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r.x) + __uint_as_float(r.y);
    if constexpr (CG >= 64) {
      const dl_u2 q = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
      v = __uint_as_float(q.x) + __uint_as_float(q.y);      // the wave's two halves
    }
  }
  return v;
}

// ------------------------------------------------------------------ short convolutions
// src [T, >= C] (row stride given), taps [C, n] float32 (the last column is the token's own),
// out float32 [T, C].  Channels [0, unit_heads * hd) are heads of hd that leave as unit vectors
// x / sqrt(sum x^2 + unit_eps), the first scaled_heads of them times `scale`.  State of a
// request: [n - 1, C] floats at state + slot * state_stride + state_off, oldest row first.
// Grid (token, block of channels): the first head_blocks blocks hold hpb whole heads each, a
// head in one, two or four whole waves and a thread a channel (a head wider than the workgroup:
// a thread several channels), the others DL_CONV_THREADS plain channels.  A head's sum of
// squares is added up over a wave's lanes and then over the head's waves in their order.
// update_state (only when every sequence of the step brings one token: a thread is then the
// only reader of its channel's kept rows): the state is moved on by this kernel.
#define DL_CONV_THREADS 256
#define DL_CONV_MAX_TAPS 8
#define DL_CONV_PER_THREAD 4     // channels a thread takes of a head wider than the workgroup

template <typename T>
__global__ __launch_bounds__(DL_CONV_THREADS) void short_conv_kernel(
    const T* __restrict__ src, long long src_stride, const float* __restrict__ taps, int n_taps,
    float* __restrict__ state, long long state_stride, long long state_off,
    const int* __restrict__ state_slots, const int* __restrict__ seq_index,
    const int* __restrict__ q_start, float* __restrict__ out, int C, int unit_heads, int hd,
    int scaled_heads, float scale, float unit_eps, int update_state, int head_blocks, int hpb) {
#pragma clang fp contract(off)
  __shared__ float sq[DL_CONV_THREADS / ZF_WAVE];
  const int t = blockIdx.x;
  const int s = seq_index[t];
  const int i0 = t - q_start[s];                       // the token's place in its portion
  float* st = state + (size_t)state_slots[s] * state_stride + state_off;
  const int hist = n_taps - 1;
  auto conv = [&](int c) -> float {
    float x[DL_CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < DL_CONV_MAX_TAPS; ++j) {
      x[j] = 0.f;
      if (j < n_taps) {
        const int back = hist - j;                     // rows before the token's own
        if (back <= i0) x[j] = load_as_float<T>(src + (size_t)(t - back) * src_stride + c);
        else x[j] = st[(size_t)(hist + i0 - back) * C + c];
      }
    }
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < DL_CONV_MAX_TAPS; ++j)
      if (j < n_taps) acc = acc + taps[(size_t)c * n_taps + j] * x[j];
    if (update_state) {
      // the kept rows move on by one: rows 1 .. of what was read, then the token's own
#pragma unroll
      for (int j = 1; j < DL_CONV_MAX_TAPS; ++j)
        if (j < n_taps) st[(size_t)(j - 1) * C + c] = x[j];
    }
    return dl_silu(acc);
  };
  float* o = out + (size_t)t * C;
  const int b = blockIdx.y;
  if (b >= head_blocks) {
    const int c = unit_heads * hd + (b - head_blocks) * DL_CONV_THREADS + threadIdx.x;
    if (c < C) o[c] = conv(c);
    return;
  }
  // a head takes tph threads, whole waves of them (hpb heads a block), a thread `per` channels
  const int tph = DL_CONV_THREADS / hpb;
  const int per = (hd + tph - 1) / tph;
  const int head = b * hpb + threadIdx.x / tph;
  const int d0 = threadIdx.x % tph;
  const bool mine = head < unit_heads;
  float v[DL_CONV_PER_THREAD];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < DL_CONV_PER_THREAD; ++j) {
    v[j] = 0.f;
    const int dd = d0 + j * tph;
    if (j < per && mine && dd < hd) v[j] = conv(head * hd + dd);
    ss += v[j] * v[j];
  }
  // over the lanes of a wave, then over the head's waves in their order
  ss = dl_lanes_sum<16>(ss);
  ss += __shfl_xor(ss, 16, ZF_WAVE);
  ss += __shfl_xor(ss, 32, ZF_WAVE);
  const int wave = threadIdx.x / ZF_WAVE, wph = tph / ZF_WAVE;
  if (threadIdx.x % ZF_WAVE == 0) sq[wave] = ss;
  __syncthreads();
  if (!mine) return;
  float total = 0.f;
  for (int w = 0; w < wph; ++w) total += sq[(wave / wph) * wph + w];
  float inv = 1.0f / sqrtf(total + unit_eps);
  if (head < scaled_heads) inv = inv * scale;
#pragma unroll
  for (int j = 0; j < DL_CONV_PER_THREAD; ++j) {
    const int dd = d0 + j * tph;
    if (j < per && dd < hd) o[head * hd + dd] = v[j] * inv;
  }
}

// The state after a step: the last n - 1 rows the convolution has seen.  Grid (sequence, block of
// channels), a thread a channel.
template <typename T>
__global__ __launch_bounds__(DL_CONV_THREADS) void short_conv_state_kernel(
    const T* __restrict__ src, long long src_stride, int n_taps, float* __restrict__ state,
    long long state_stride, long long state_off, const int* __restrict__ state_slots,
    const int* __restrict__ q_start, int C) {
  const int s = blockIdx.x;
  const int first = q_start[s], len = q_start[s + 1] - first;
  const int c = blockIdx.y * DL_CONV_THREADS + threadIdx.x;
  if (len <= 0 || c >= C) return;
  float* st = state + (size_t)state_slots[s] * state_stride + state_off;
  const int hist = n_taps - 1;
  // row r of the new state is the portion's row len - hist + r, or (before the portion) the
  // old state's row r + len, which lies behind the row being written: ascending r is safe
  for (int r = 0; r < hist; ++r) {
    const int i = len - hist + r;
    st[(size_t)r * C + c] = i >= 0 ? load_as_float<T>(src + (size_t)(first + i) * src_stride + c)
                                   : st[(size_t)(r + len) * C + c];
  }
}

extern "C" int zf_short_conv(const void* src, int dtype, long long src_stride, const float* taps,
                             int n_taps, float* state, long long state_stride,
                             long long state_off, const int* state_slots, const int* seq_index,
                             const int* q_start, float* out, int T, int n_seqs, int C,
                             int unit_heads, int hd, int scaled_heads, float scale,
                             float unit_eps, int single_tokens, hipStream_t stream) {
  if (T <= 0) return 0;
  if (C <= 0 || n_taps < 1 || n_taps > DL_CONV_MAX_TAPS || unit_heads < 0 || hd < 1 ||
      (size_t)unit_heads * hd > (size_t)C || scaled_heads > unit_heads || n_seqs < 1 ||
      (single_tokens && T != n_seqs) || hd > DL_CONV_THREADS * DL_CONV_PER_THREAD)
    return -2;
  // a head takes whole waves (one, two or four): as many heads a block as fit
  const int hw = hd > 128 ? 4 : (hd > 64 ? 2 : 1);
  const int hpb = DL_CONV_THREADS / (hw * ZF_WAVE);
  const int head_blocks = (unit_heads + hpb - 1) / hpb;
  const int plain = C - unit_heads * hd;
  const dim3 grid(T, head_blocks + (plain + DL_CONV_THREADS - 1) / DL_CONV_THREADS);
  const dim3 sgrid(n_seqs, (C + DL_CONV_THREADS - 1) / DL_CONV_THREADS);
#define DL_CONV_LAUNCH(TT)                                                                        \
  hipLaunchKernelGGL(short_conv_kernel<TT>, grid, dim3(DL_CONV_THREADS), 0, stream,              \
                     (const TT*)src, src_stride, taps, n_taps, state, state_stride, state_off,   \
                     state_slots, seq_index, q_start, out, C, unit_heads, hd, scaled_heads,      \
                     scale, unit_eps, single_tokens, head_blocks, hpb);                          \
  if (!single_tokens && n_taps > 1)                                                               \
    hipLaunchKernelGGL(short_conv_state_kernel<TT>, sgrid, dim3(DL_CONV_THREADS), 0, stream,     \
                       (const TT*)src, src_stride, n_taps, state, state_stride, state_off,       \
                       state_slots, q_start, C)
  if (dtype == ZF_F32) { DL_CONV_LAUNCH(float); } else { DL_CONV_LAUNCH(bf16_t); }
  ZF_CHECK_LAUNCH();
}

// ------------------------------------------------------------------ the recurrence
#define DL_STAGE 16            // tokens staged in LDS at a time
#define DL_MAX_LANES 64        // lanes that share a column's key channels
#define DL_PF 4                // 16-byte pieces of q and of k, and values of v, a thread fetches ahead

// A thread holds R key channels of one value column of S; CG lanes side by side hold the
// column's P = CG * R channels (zeros beyond d).  A request's matrices lie [head][column][P] in
// its state, so a thread's channels are consecutive.  Grid (column tiles, heads, sequences).
// qkv float32 [T, C]: q heads at q_off, k heads at k_off (KH heads of d each), v heads at v_off
// (H heads of dv); ab float32 [T, 2 H]: the decays' numbers z_a, then the step sizes' z_b.
// Sixteen tokens at a time lie in LDS; the next sixteen are asked for before these are walked
// (16-byte pieces, where the rows' offsets allow: VEC), and a token's operands are read from LDS
// while the token before it is computed.
template <int R, int CG, bool VEC>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ qkv, int C, int q_off, int k_off, int v_off,
    const float* __restrict__ ab, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, long long state_stride,
    const int* __restrict__ state_slots, const int* __restrict__ q_start, float* __restrict__ out,
    int H, int KH, int d, int dv, int cols) {
  // (fused multiply-adds as the compiler forms them: this one kernel walks every portion, whole
  // prompt or single token, so every cut of a sequence gets the same instructions)
  extern __shared__ float lds[];
  const int P = CG * R;
  float* qs = lds;                          // [DL_STAGE][P]
  float* ks = qs + DL_STAGE * P;            // [DL_STAGE][P]
  float* vs = ks + DL_STAGE * P;            // [DL_STAGE][cols]
  float* gs = vs + DL_STAGE * cols;         // [DL_STAGE] decay
  float* bs = gs + DL_STAGE;                // [DL_STAGE] step size
  float* ds = bs + DL_STAGE;                // [DL_STAGE] q . k
  float* os = ds + DL_STAGE;                // [DL_STAGE][cols] the stage's outputs
  const int h = blockIdx.y, seq = blockIdx.z;
  const int kh = h / (H / KH);
  const int first = q_start[seq], len = q_start[seq + 1] - first;
  if (len <= 0) return;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int cg = tid % CG, col_l = tid / CG;
  const int col = blockIdx.x * cols + col_l;
  const bool live = col < dv;
  float* S_mem = state + (size_t)state_slots[seq] * state_stride
                 + ((size_t)h * dv + (live ? col : 0)) * P + cg * R;
  float S[R];
  if constexpr (R % 4 == 0) {
#pragma unroll
    for (int r = 0; r < R; r += 4) {
      const float4 v = live ? *(const float4*)(S_mem + r) : make_float4(0.f, 0.f, 0.f, 0.f);
      S[r] = v.x; S[r + 1] = v.y; S[r + 2] = v.z; S[r + 3] = v.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < R; r += 2) {
      const float2 v = live ? *(const float2*)(S_mem + r) : make_float2(0.f, 0.f);
      S[r] = v.x; S[r + 1] = v.y;
    }
  }
  const float decay_rate = expf(a_log[h]);
  const float dtb = dt_bias[h];
  const int P4 = P / 4;
  // what a thread fetches ahead: pieces tid, tid + nthreads, ... of the stage's q and k rows,
  // one value of its v columns, and (the first threads) a token's two numbers
  float4 fq[DL_PF], fk[DL_PF];
  float fv[DL_PF], fa = 0.f, fb = 0.f;
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  auto fetch = [&](int t0, int n) {
    if constexpr (VEC) {
#pragma unroll
      for (int j = 0; j < DL_PF; ++j) {
        const int i = tid + j * nthreads;
        fq[j] = fk[j] = zero4;
        if (i < n * P4) {
          const int tok = i / P4, c = (i % P4) * 4;
          const float* row = qkv + (size_t)(first + t0 + tok) * C;
          if (c < d) {
            fq[j] = *(const float4*)(row + q_off + kh * d + c);
            fk[j] = *(const float4*)(row + k_off + kh * d + c);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < DL_PF; ++j) {
        const int i = tid + j * nthreads;
        fv[j] = 0.f;
        if (i < n * cols) {
          const int tok = i / cols, c = blockIdx.x * cols + i % cols;
          if (c < dv) fv[j] = qkv[(size_t)(first + t0 + tok) * C + v_off + h * dv + c];
        }
      }
      if (tid < n) {
        const float* z = ab + (size_t)(first + t0 + tid) * 2 * H;
        fa = z[h];
        fb = z[H + h];
      }
    }
  };
  auto stage = [&](int t0, int n) {
    if constexpr (VEC) {
#pragma unroll
      for (int j = 0; j < DL_PF; ++j) {
        const int i = tid + j * nthreads;
        if (i < n * P4) {
          *(float4*)(qs + 4 * i) = fq[j];
          *(float4*)(ks + 4 * i) = fk[j];
        }
      }
#pragma unroll
      for (int j = 0; j < DL_PF; ++j)
        if (tid + j * nthreads < n * cols) vs[tid + j * nthreads] = fv[j];
      if (tid < n) {
        gs[tid] = expf(-(decay_rate * dl_softplus(fa + dtb)));
        bs[tid] = 1.0f / (1.0f + expf(-fb));
      }
    } else {
      for (int i = tid; i < n * P; i += nthreads) {
        const int tok = i / P, c = i % P;
        const float* row = qkv + (size_t)(first + t0 + tok) * C;
        qs[i] = c < d ? row[q_off + kh * d + c] : 0.f;
        ks[i] = c < d ? row[k_off + kh * d + c] : 0.f;
      }
      for (int i = tid; i < n * cols; i += nthreads) {
        const int tok = i / cols, c = blockIdx.x * cols + i % cols;
        vs[i] = c < dv ? qkv[(size_t)(first + t0 + tok) * C + v_off + h * dv + c] : 0.f;
      }
      if (tid < n) {
        const float* z = ab + (size_t)(first + t0 + tid) * 2 * H;
        gs[tid] = expf(-(decay_rate * dl_softplus(z[h] + dtb)));
        bs[tid] = 1.0f / (1.0f + expf(-z[H + h]));
      }
    }
  };
  fetch(0, min(DL_STAGE, len));
  for (int t0 = 0; t0 < len; t0 += DL_STAGE) {
    const int n = min(DL_STAGE, len - t0);
    __syncthreads();                        // the tokens staged before are done with
    stage(t0, n);
    __syncthreads();
    if (t0 + DL_STAGE < len) fetch(t0 + DL_STAGE, min(DL_STAGE, len - t0 - DL_STAGE));
    // q . k of every staged token: sixteen lanes a token
    for (int tok = tid / 16; tok < n; tok += nthreads / 16) {
      float dot = 0.f;
      for (int c = tid % 16; c < P; c += 16) dot += qs[tok * P + c] * ks[tok * P + c];
      dot = dl_lanes_sum<16>(dot);
      if (tid % 16 == 0) ds[tok] = dot;
    }
    __syncthreads();
    // a token's operands are read a token ahead
    float kk[R], qq[R], g, b, v, qk;

    auto read = [&](int tok) {
      const float* qrow = qs + tok * P + cg * R;
      const float* krow = ks + tok * P + cg * R;
      if constexpr (R % 4 == 0) {
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          const float4 kv = *(const float4*)(krow + r);
          const float4 qv = *(const float4*)(qrow + r);
          kk[r] = kv.x; kk[r + 1] = kv.y; kk[r + 2] = kv.z; kk[r + 3] = kv.w;
          qq[r] = qv.x; qq[r + 1] = qv.y; qq[r + 2] = qv.z; qq[r + 3] = qv.w;
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; r += 2) {
          const float2 kv = *(const float2*)(krow + r);
          const float2 qv = *(const float2*)(qrow + r);
          kk[r] = kv.x; kk[r + 1] = kv.y;
          qq[r] = qv.x; qq[r + 1] = qv.y;
        }
      }
      g = gs[tok]; b = bs[tok]; v = vs[tok * cols + col_l]; qk = ds[tok];
    };
    read(0);
    for (int tok = 0; tok < n; ++tok) {
      float r0 = 0.f, r1 = 0.f, p0 = 0.f, p1 = 0.f;
      float kc[R];
#pragma unroll
      for (int r = 0; r < R; r += 2) {
        kc[r] = kk[r]; kc[r + 1] = kk[r + 1];
        r0 += kk[r] * S[r]; r1 += kk[r + 1] * S[r + 1];
        p0 += qq[r] * S[r]; p1 += qq[r + 1] * S[r + 1];
      }
      const float gc = g, bc = b, vc = v, qkc = qk;
      if (tok + 1 < n) read(tok + 1);
      const float rs = dl_lanes_sum<CG>(r0 + r1), ps = dl_lanes_sum<CG>(p0 + p1);
      const float w = bc * (vc - gc * rs);
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = gc * S[r] + kc[r] * w;
      if (cg == 0) os[tok * cols + col_l] = gc * ps + qkc * w;
    }
    // the stage's outputs leave side by side (the next stage's barrier stands between these
    // reads and the next writes)
    __syncthreads();
    for (int i = tid; i < n * cols; i += nthreads) {
      const int tok = i / cols, c = blockIdx.x * cols + i % cols;
      if (c < dv) out[(size_t)(first + t0 + tok) * H * dv + (size_t)h * dv + c] = os[i];
    }
  }
  if (live) {
    if constexpr (R % 4 == 0) {
#pragma unroll
      for (int r = 0; r < R; r += 4)
        *(float4*)(S_mem + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else {
#pragma unroll
      for (int r = 0; r < R; r += 2) *(float2*)(S_mem + r) = make_float2(S[r], S[r + 1]);
    }
  }
}

// R * CG >= d is the padded key size P the state is laid out with; cols * CG threads a workgroup
// (a multiple of 64, at most 256).
extern "C" int zf_delta_recurrence(const float* qkv, int C, int q_off, int k_off, int v_off,
                                   const float* ab, const float* a_log, const float* dt_bias,
                                   float* state, long long state_stride, const int* state_slots,
                                   const int* q_start, float* out, int n_seqs, int H, int KH,
                                   int d, int dv, int R, int CG, int cols, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  const int threads = cols * CG;
  if (H < 1 || KH < 1 || H % KH != 0 || d < 1 || dv < 1 || CG < 1 || CG > DL_MAX_LANES ||
      (CG & (CG - 1)) != 0 || R * CG < d || cols < 1 || threads > 256 || threads % ZF_WAVE != 0 ||
      ZF_WAVE % CG != 0)
    return -2;
  const dim3 grid((dv + cols - 1) / cols, H, n_seqs), block(threads);
  const size_t smem = (size_t)(DL_STAGE * (2 * R * CG + 2 * cols) + 3 * DL_STAGE) * sizeof(float);
  // 16-byte pieces: every row offset a multiple of four floats, and few enough pieces a thread
  const bool vec = C % 4 == 0 && q_off % 4 == 0 && k_off % 4 == 0 && d % 4 == 0 &&
                   ((uintptr_t)qkv % 16) == 0 &&
                   DL_STAGE * (R * CG / 4) <= DL_PF * threads && DL_STAGE * cols <= DL_PF * threads &&
                   DL_STAGE <= threads;
#define DL_REC_LAUNCH(RR, GG)                                                                    \
  if (R == RR && CG == GG) {                                                                     \
    if (vec)                                                                                     \
      hipLaunchKernelGGL((delta_recurrence_kernel<RR, GG, true>), grid, block, smem, stream,     \
                         qkv, C, q_off, k_off, v_off, ab, a_log, dt_bias, state, state_stride,   \
                         state_slots, q_start, out, H, KH, d, dv, cols);                         \
    else                                                                                         \
      hipLaunchKernelGGL((delta_recurrence_kernel<RR, GG, false>), grid, block, smem, stream,    \
                         qkv, C, q_off, k_off, v_off, ab, a_log, dt_bias, state, state_stride,   \
                         state_slots, q_start, out, H, KH, d, dv, cols);                         \
    launched = true;                                                                             \
  }
  bool launched = false;
  // (the padded key sizes 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256)
  DL_REC_LAUNCH(8, 1) DL_REC_LAUNCH(12, 1) DL_REC_LAUNCH(8, 2) DL_REC_LAUNCH(12, 2)
  DL_REC_LAUNCH(8, 4) DL_REC_LAUNCH(12, 4) DL_REC_LAUNCH(8, 8) DL_REC_LAUNCH(12, 8)
  DL_REC_LAUNCH(8, 16) DL_REC_LAUNCH(12, 16) DL_REC_LAUNCH(16, 16)
  if (!launched) return -2;
  ZF_CHECK_LAUNCH();
}
