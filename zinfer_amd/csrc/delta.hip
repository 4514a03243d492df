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

// ------------------------------------------------------------------ short convolutions
// src [T, >= C] (row stride given), taps [C, n] float32 (the last column is the token's own),
// out float32 [T, C].  Channels [0, unit_heads * hd) are heads of hd that leave as unit vectors
// x / sqrt(sum x^2 + unit_eps), the first scaled_heads of them times `scale`.  State of a
// request: [n - 1, C] floats at state + slot * state_stride + state_off, oldest row first.
// update_state (only when every sequence of the step brings one token: a workgroup is then the
// only reader of its state): the state is moved on by this kernel.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(
    const T* __restrict__ src, long long src_stride, const float* __restrict__ taps, int n_taps,
    float* __restrict__ state, long long state_stride, long long state_off,
    const int* __restrict__ state_slots, const int* __restrict__ seq_index,
    const int* __restrict__ q_start, float* __restrict__ out, int C, int unit_heads, int hd,
    int scaled_heads, float scale, float unit_eps, int update_state) {
#pragma clang fp contract(off)
  const int t = blockIdx.x;
  const int s = seq_index[t];
  const int i0 = t - q_start[s];                       // the token's place in its portion
  float* st = state + (size_t)state_slots[s] * state_stride + state_off;
  const int hist = n_taps - 1;
  auto conv = [&](int c) -> float {
    float acc = 0.f;
    for (int j = 0; j < n_taps; ++j) {
      const int back = hist - j;                       // rows before the token's own
      float x;
      if (back <= i0) x = load_as_float<T>(src + (size_t)(t - back) * src_stride + c);
      else x = st[(size_t)(hist + i0 - back) * C + c];
      acc = acc + taps[(size_t)c * n_taps + j] * x;
    }
    return dl_silu(acc);
  };
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  float* o = out + (size_t)t * C;
  for (int head = wave; head < unit_heads; head += blockDim.x / ZF_WAVE) {
    float ss = 0.f;
    for (int d = lane; d < hd; d += ZF_WAVE) {
      const float v = conv(head * hd + d);
      o[head * hd + d] = v;
      ss += v * v;
    }
    ss = wave_sum(ss);
    float inv = 1.0f / sqrtf(ss + unit_eps);
    if (head < scaled_heads) inv = inv * scale;
    // (a lane reads back what it wrote itself)
    for (int d = lane; d < hd; d += ZF_WAVE) o[head * hd + d] = o[head * hd + d] * inv;
  }
  for (int c = unit_heads * hd + threadIdx.x; c < C; c += blockDim.x) o[c] = conv(c);
  if (update_state) {
    __syncthreads();                                   // every channel's old rows have been read
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
      for (int r = 0; r + 1 < hist; ++r) st[(size_t)r * C + c] = st[(size_t)(r + 1) * C + c];
      if (hist > 0) st[(size_t)(hist - 1) * C + c] = load_as_float<T>(src + (size_t)t * src_stride + c);
    }
  }
}

// The state after a step: the last n - 1 rows the convolution has seen.  A workgroup a sequence.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_state_kernel(
    const T* __restrict__ src, long long src_stride, int n_taps, float* __restrict__ state,
    long long state_stride, long long state_off, const int* __restrict__ state_slots,
    const int* __restrict__ q_start, int C) {
  const int s = blockIdx.x;
  const int first = q_start[s], len = q_start[s + 1] - first;
  if (len <= 0) return;
  float* st = state + (size_t)state_slots[s] * state_stride + state_off;
  const int hist = n_taps - 1;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    // row r of the new state is the portion's row len - hist + r, or (before the portion) the
    // old state's row r + len, which lies behind the row being written: ascending r is safe
    for (int r = 0; r < hist; ++r) {
      const int i = len - hist + r;
      st[(size_t)r * C + c] = i >= 0 ? load_as_float<T>(src + (size_t)(first + i) * src_stride + c)
                                     : st[(size_t)(r + len) * C + c];
    }
  }
}

extern "C" int zf_short_conv(const void* src, int dtype, long long src_stride, const float* taps,
                             int n_taps, float* state, long long state_stride,
                             long long state_off, const int* state_slots, const int* seq_index,
                             const int* q_start, float* out, int T, int n_seqs, int C,
                             int unit_heads, int hd, int scaled_heads, float scale,
                             float unit_eps, int single_tokens, hipStream_t stream) {
  if (T <= 0) return 0;
  if (C <= 0 || n_taps < 1 || unit_heads < 0 || hd < 1 || (size_t)unit_heads * hd > (size_t)C ||
      scaled_heads > unit_heads || n_seqs < 1 || (single_tokens && T != n_seqs))
    return -2;
#define DL_CONV_LAUNCH(TT)                                                                        \
  hipLaunchKernelGGL(short_conv_kernel<TT>, dim3(T), dim3(256), 0, stream, (const TT*)src,       \
                     src_stride, taps, n_taps, state, state_stride, state_off, state_slots,      \
                     seq_index, q_start, out, C, unit_heads, hd, scaled_heads, scale, unit_eps,  \
                     single_tokens);                                                              \
  if (!single_tokens && n_taps > 1)                                                               \
    hipLaunchKernelGGL(short_conv_state_kernel<TT>, dim3(n_seqs), dim3(256), 0, stream,          \
                       (const TT*)src, src_stride, n_taps, state, state_stride, state_off,       \
                       state_slots, q_start, C)
  if (dtype == ZF_F32) { DL_CONV_LAUNCH(float); } else { DL_CONV_LAUNCH(bf16_t); }
  ZF_CHECK_LAUNCH();
}

// ------------------------------------------------------------------ the recurrence
#define DL_STAGE 16            // tokens staged in LDS at a time
#define DL_MAX_LANES 16        // lanes that share a column's key channels

// A thread holds R key channels of one value column of S; CG lanes side by side hold the
// column's P = CG * R channels (zeros beyond d).  A request's matrices lie [head][column][P] in
// its state, so a thread's channels are consecutive.  Grid (column tiles, heads, sequences).
// qkv float32 [T, C]: q heads at q_off, k heads at k_off (KH heads of d each), v heads at v_off
// (H heads of dv); ab float32 [T, 2 H]: the decays' numbers z_a, then the step sizes' z_b.
template <int R>
__global__ __launch_bounds__(256) void delta_recurrence_kernel(
    const float* __restrict__ qkv, int C, int q_off, int k_off, int v_off,
    const float* __restrict__ ab, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, long long state_stride,
    const int* __restrict__ state_slots, const int* __restrict__ q_start, float* __restrict__ out,
    int H, int KH, int d, int dv, int CG, int cols) {
#pragma clang fp contract(off)
  extern __shared__ float lds[];
  const int P = CG * R;
  float* qs = lds;                          // [DL_STAGE][P]
  float* ks = qs + DL_STAGE * P;            // [DL_STAGE][P]
  float* vs = ks + DL_STAGE * P;            // [DL_STAGE][cols]
  float* gs = vs + DL_STAGE * cols;         // [DL_STAGE] decay
  float* bs = gs + DL_STAGE;                // [DL_STAGE] step size
  float* ds = bs + DL_STAGE;                // [DL_STAGE] q . k
  const int h = blockIdx.y, seq = blockIdx.z;
  const int kh = h / (H / KH);
  const int first = q_start[seq], len = q_start[seq + 1] - first;
  if (len <= 0) return;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int cg = tid % CG, col_l = tid / CG;
  const int col = blockIdx.x * cols + col_l;
  const bool live = col_l < cols && col < dv;
  float* S_mem = state + (size_t)state_slots[seq] * state_stride
                 + ((size_t)h * dv + (live ? col : 0)) * P + cg * R;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; r += 4) {
    const float4 v = live ? *(const float4*)(S_mem + r) : make_float4(0.f, 0.f, 0.f, 0.f);
    S[r] = v.x; S[r + 1] = v.y; S[r + 2] = v.z; S[r + 3] = v.w;
  }
  const float decay_rate = expf(a_log[h]);
  const float dtb = dt_bias[h];
  const int wave = tid / ZF_WAVE, lane = tid % ZF_WAVE, nwaves = (nthreads + ZF_WAVE - 1) / ZF_WAVE;
  for (int t0 = 0; t0 < len; t0 += DL_STAGE) {
    const int n = min(DL_STAGE, len - t0);
    __syncthreads();                        // the tokens staged before are done with
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
    __syncthreads();
    for (int tok = wave; tok < n; tok += nwaves) {
      float dot = 0.f;
      for (int c = lane; c < P; c += ZF_WAVE) dot += qs[tok * P + c] * ks[tok * P + c];
      dot = wave_sum(dot);
      if (lane == 0) ds[tok] = dot;
    }
    __syncthreads();
    for (int tok = 0; tok < n; ++tok) {
      const float* qrow = qs + tok * P + cg * R;
      const float* krow = ks + tok * P + cg * R;
      float kk[R];
      float r0 = 0.f, r1 = 0.f, p0 = 0.f, p1 = 0.f;
#pragma unroll
      for (int r = 0; r < R; r += 4) {
        const float4 kv = *(const float4*)(krow + r);
        const float4 qv = *(const float4*)(qrow + r);
        kk[r] = kv.x; kk[r + 1] = kv.y; kk[r + 2] = kv.z; kk[r + 3] = kv.w;
        r0 += kv.x * S[r]; r1 += kv.y * S[r + 1]; r0 += kv.z * S[r + 2]; r1 += kv.w * S[r + 3];
        p0 += qv.x * S[r]; p1 += qv.y * S[r + 1]; p0 += qv.z * S[r + 2]; p1 += qv.w * S[r + 3];
      }
      float rs = r0 + r1, ps = p0 + p1;
      for (int off = 1; off < CG; off <<= 1) {
        rs += __shfl_xor(rs, off, ZF_WAVE);
        ps += __shfl_xor(ps, off, ZF_WAVE);
      }
      const float g = gs[tok];
      const float w = bs[tok] * (vs[tok * cols + (col_l < cols ? col_l : 0)] - g * rs);
#pragma unroll
      for (int r = 0; r < R; ++r) S[r] = g * S[r] + kk[r] * w;
      if (live && cg == 0)
        out[(size_t)(first + t0 + tok) * H * dv + (size_t)h * dv + col] = g * ps + ds[tok] * w;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; r += 4)
      *(float4*)(S_mem + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
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
  const size_t smem = (size_t)(DL_STAGE * (2 * R * CG + cols) + 3 * DL_STAGE) * sizeof(float);
#define DL_REC_LAUNCH(RR)                                                                        \
  hipLaunchKernelGGL(delta_recurrence_kernel<RR>, grid, block, smem, stream, qkv, C, q_off,      \
                     k_off, v_off, ab, a_log, dt_bias, state, state_stride, state_slots,         \
                     q_start, out, H, KH, d, dv, CG, cols)
  switch (R) {
    case 8: DL_REC_LAUNCH(8); break;
    case 12: DL_REC_LAUNCH(12); break;
    case 16: DL_REC_LAUNCH(16); break;
    case 24: DL_REC_LAUNCH(24); break;
    case 32: DL_REC_LAUNCH(32); break;
    default: return -2;
  }
  ZF_CHECK_LAUNCH();
}
