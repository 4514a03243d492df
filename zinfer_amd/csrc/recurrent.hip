// Mixers whose memory of a sequence is a matrix of fixed size a head, carried from token to
// token in 32-bit, instead of a cache that grows:
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T          S is [d, dv] a head, a_t in (0, 1) a key channel
//   after:   o_t = S_t^T q_t                     (the output reads the new state)
//   before:  o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t      (the old state, and the token's own
//                                                 outer product weighted by a learned u)
//
// The decay a_t comes from 32-bit numbers z_t (a projection's output) by one of two rules:
//   rule 0:  a = sigmoid(z + b)^(1 / tau) = exp(-softplus(-(z + b)) / tau)
//   rule 1:  a = exp(-exp(z + b))
// Everything but the rows q, k, v themselves is 32-bit in both storage types.
//
//  * token_shift_mix     m_s[t] = h[t] + (h[t-1] - h[t]) * mu_s for several s at once; the row
//                        before a portion's first is the request's state (zero at the start),
//                        which then takes the portion's last row
//  * decay_recurrence    the recurrence, token by token; a request's state is read at the start
//                        of its portion and written at its end
//  * decay_recurrence_spans   the same for long portions, cut into spans that run side by side:
//                        every span's own sum from a zero state, then the states at the spans'
//                        starts one after the other (S <- diag(product of the span's decays) S +
//                        the span's sum), then every span's outputs from the state at its start
//  * head_norm_gate      out = o / rms_head(o) * gain * silu(g)
#include "zf_common.h"

// 8 neighbouring numbers of a row as floats, through 16-byte loads (the address is a multiple of
// 16 bytes).
template <typename T> __device__ __forceinline__ void load8(const T* p, float (&o)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&o)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w; o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
}
template <> __device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&o)[8]) {
  const uint4 a = *(const uint4*)p;
  const unsigned w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

template <typename T> __device__ __forceinline__ void store8(T* p, const float (&v)[8]);
template <> __device__ __forceinline__ void store8<float>(float* p, const float (&v)[8]) {
  *(float4*)p = float4{v[0], v[1], v[2], v[3]};
  *(float4*)(p + 4) = float4{v[4], v[5], v[6], v[7]};
}
template <> __device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float (&v)[8]) {
  unsigned w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    w[i] = (unsigned)float_to_bf16(v[2 * i]) | ((unsigned)float_to_bf16(v[2 * i + 1]) << 16);
  *(uint4*)p = uint4{w[0], w[1], w[2], w[3]};
}

// The same in two steps: the bits as they were loaded (a bfloat16 row's 8 numbers take 4
// registers while they wait), then the floats.
template <typename T> struct Raw8;
template <> struct Raw8<float> { float4 a, b; };
template <> struct Raw8<bf16_t> { uint4 a; };
__device__ __forceinline__ void load_raw8(const float* p, Raw8<float>& r) {
  r.a = *(const float4*)p; r.b = *(const float4*)(p + 4);
}
__device__ __forceinline__ void load_raw8(const bf16_t* p, Raw8<bf16_t>& r) {
  r.a = *(const uint4*)p;
}
__device__ __forceinline__ void widen8(const Raw8<float>& r, float (&o)[8]) {
  o[0] = r.a.x; o[1] = r.a.y; o[2] = r.a.z; o[3] = r.a.w;
  o[4] = r.b.x; o[5] = r.b.y; o[6] = r.b.z; o[7] = r.b.w;
}
__device__ __forceinline__ void widen8(const Raw8<bf16_t>& r, float (&o)[8]) {
  const unsigned w[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    o[2 * i] = __uint_as_float(w[i] << 16);
    o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// ---------------------------------------------------------------- token shift
// grid (token, block of columns), an element a thread: mixes [n_mix][T][W] in the rows' type.
// The workgroups of a portion's first token read the state row and are the ones that overwrite
// it (with the portion's last row), element by element in the thread that read it: no other
// thread touches that element.
template <typename T>
__global__ void token_shift_mix_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                       float* __restrict__ state, long long slot_stride,
                                       const int* __restrict__ state_slots,
                                       const int* __restrict__ seq_index,
                                       const int* __restrict__ q_start, T* __restrict__ out,
                                       int n_tokens, int W, int n_mix) {
  const int t = blockIdx.x;
  const int s = seq_index[t];
  const int t0 = q_start[s], t1 = q_start[s + 1];
  const bool first = t == t0;
  const T* row = h + (size_t)t * W;
  const T* before = first ? nullptr : row - W;
  float* st = state + (size_t)state_slots[s] * slot_stride;
  const T* last = h + (size_t)(t1 - 1) * W;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < W) {
    const float x = load_as_float<T>(row + i);
    const float p = first ? st[i] : load_as_float<T>(before + i);
    const float dx = p - x;
    for (int m = 0; m < n_mix; ++m)
      store_from_float<T>(out + ((size_t)m * n_tokens + t) * W + i,
                          fmaf(dx, mu[(size_t)m * W + i], x));
    if (first) st[i] = load_as_float<T>(last + i);
  }
}

// The same with 8 neighbouring columns a thread (W a multiple of 8, rows at multiples of 16
// bytes): 16-byte loads and stores.  grid (token, block of 8-column groups).
template <typename T>
__global__ void token_shift_mix8_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                        float* __restrict__ state, long long slot_stride,
                                        const int* __restrict__ state_slots,
                                        const int* __restrict__ seq_index,
                                        const int* __restrict__ q_start, T* __restrict__ out,
                                        int n_tokens, int W, int n_mix) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= W) return;
  const int s = seq_index[t];
  const int t0 = q_start[s], t1 = q_start[s + 1];
  const bool first = t == t0;
  const T* row = h + (size_t)t * W;
  float* st = state + (size_t)state_slots[s] * slot_stride;
  float x[8], p[8];
  load8<T>(row + i, x);
  if (first) {
#pragma unroll
    for (int j = 0; j < 8; ++j) p[j] = st[i + j];
  } else {
    load8<T>(row - W + i, p);
  }
  for (int m = 0; m < n_mix; ++m) {
    float g[8], y[8];
    load8<float>(mu + (size_t)m * W + i, g);
#pragma unroll
    for (int j = 0; j < 8; ++j) y[j] = fmaf(p[j] - x[j], g[j], x[j]);
    store8<T>(out + ((size_t)m * n_tokens + t) * W + i, y);
  }
  if (first) {
    float l[8];
    load8<T>(h + (size_t)(t1 - 1) * W + i, l);
#pragma unroll
    for (int j = 0; j < 8; ++j) st[i + j] = l[j];
  }
}

extern "C" int zf_token_shift_mix(const void* h, int dtype, const float* mu, float* state,
                                  long long slot_stride, const int* state_slots,
                                  const int* seq_index, const int* q_start, void* out, int T,
                                  int W, int n_mix, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || n_mix <= 0) return -2;
  if (W % 8 == 0 && (uintptr_t)h % 16 == 0 && (uintptr_t)out % 16 == 0 && (uintptr_t)mu % 16 == 0) {
    const int groups = W / 8;
    const int block = groups >= 256 ? 256 : (groups + ZF_WAVE - 1) / ZF_WAVE * ZF_WAVE;
    const dim3 grid(T, (groups + block - 1) / block);
    if (dtype == ZF_F32)
      hipLaunchKernelGGL(token_shift_mix8_kernel<float>, grid, dim3(block), 0, stream,
                         (const float*)h, mu, state, slot_stride, state_slots, seq_index, q_start,
                         (float*)out, T, W, n_mix);
    else
      hipLaunchKernelGGL(token_shift_mix8_kernel<bf16_t>, grid, dim3(block), 0, stream,
                         (const bf16_t*)h, mu, state, slot_stride, state_slots, seq_index,
                         q_start, (bf16_t*)out, T, W, n_mix);
    ZF_CHECK_LAUNCH();
  }
  const int block = W >= 1024 ? 256 : (W >= 256 ? 128 : 64);
  const dim3 grid(T, (W + block - 1) / block);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(token_shift_mix_kernel<float>, grid, dim3(block), 0, stream,
                       (const float*)h, mu, state, slot_stride, state_slots, seq_index, q_start,
                       (float*)out, T, W, n_mix);
  else
    hipLaunchKernelGGL(token_shift_mix_kernel<bf16_t>, grid, dim3(block), 0, stream,
                       (const bf16_t*)h, mu, state, slot_stride, state_slots, seq_index, q_start,
                       (bf16_t*)out, T, W, n_mix);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- the recurrence
#define REC_R 8            // key channels of a value column a thread keeps in registers
#define REC_TC 16          // tokens staged at a time (half of that for more than 128 channels)
#define REC_MAX_THREADS 256
#define REC_MAX_LDS 65536
#define REC_TB 4           // tokens whose partial outputs are summed over the lanes together
#define REC_STAGE 2        // 8-channel loads a thread has in flight when a chunk comes in

__device__ __forceinline__ float decay_of(float z, int rule, float inv_tau) {
  if (rule == 0) {
    // log sigmoid(z) = -softplus(-z)
    const float x = -z;
    const float sp = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
    return expf(-sp * inv_tau);
  }
  if (rule == 2) return z;                // the decays themselves
  return expf(-expf(z));
}

// z <- the decays of z, in place, an element a thread: spans of a portion then read them as they
// are (rule 2) instead of each forming them again.
__global__ void decays_in_place_kernel(float* __restrict__ z, const float* __restrict__ z_bias,
                                       long long n, int width, int rule, float inv_tau) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) z[i] = decay_of(z[i] + z_bias[i % width], rule, inv_tau);
}

// grid (sequence, head, block of VB value columns); thread (vl, cg) = (tid / CS, tid % CS)
// holds S[8 cg .. 8 cg + 8, v0 + RV vl .. + RV]: RV value columns (4, 2 or 1: what divides VB),
// so that a token's q, k and decays, read from LDS once, serve RV columns.  A request's state is
// laid out [head][dv][CS * 8]: the channels a thread holds lie side by side (channels beyond d
// are padding that stays zero).  A token's partial outputs (one a thread and column) go to LDS
// (rows of CS, padded to an odd length so that the sums' reads spread over the banks) and are
// added in ascending cg; where CS is a power of two (``shuffle``) the CS lanes of a column add
// their partial outputs among themselves instead, pair by pair, and lane 0 stores the sum.
// Either way the sum over channels has one order whatever VB is and however a prompt is cut.  ``wide``: d, dv and VB are multiples of 8 and rows start at multiples of 16
// bytes; a chunk's rows then come in through 16-byte loads, all of a thread's in flight at once.
//
// MODE 0: a sequence's whole portion in one workgroup.  With spans of ``span`` tokens
// (blockIdx.x = sequence * max_spans + span number): MODE 1 runs a span from a zero state, writes
// no output and leaves the span's sum in span_state and the product of its decays in span_decay
// (the workgroups of value block 0 do); MODE 2 starts from span_state (by then the state at the
// span's start) and writes the outputs.  A sequence of a single span is left alone by MODE 1 and
// runs as in MODE 0 under MODE 2.
template <typename T, bool BEFORE, int MODE, int RV>
__global__ __launch_bounds__(REC_MAX_THREADS) void decay_recurrence_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride,
    const T* __restrict__ v, long long v_stride, const float* __restrict__ z,
    const float* __restrict__ z_bias, const float* __restrict__ bonus,
    float* __restrict__ state, long long slot_stride, const int* __restrict__ state_slots,
    const int* __restrict__ q_start, float* __restrict__ out, int H, int d, int dv, int CS,
    int VB, int TC, int rule, float inv_tau, float q_scale, int span, int max_spans,
    float* __restrict__ span_state, float* __restrict__ span_decay, int wide, int shuffle) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int DP = CS * REC_R;
  const int CSP = CS | 1;
  float* qs = lds;                        // [TC][DP]
  float* ks = qs + TC * DP;               // [TC][DP]
  float* ds = ks + TC * DP;               // [TC][DP]
  float* us = ds + TC * DP;               // [DP]
  float* pd = us + DP;                    // [DP], MODE 1: the product of the span's decays
  float* vs = pd + DP;                    // [TC][VB]
  float* po = vs + TC * VB;               // [TC][VB][CSP]
  const int hd = blockIdx.y, v0 = blockIdx.z * VB;
  int s = blockIdx.x, t0, t1;
  bool alone = true;                      // the portion is this workgroup's from end to end
  if (MODE == 0) {
    t0 = q_start[s], t1 = q_start[s + 1];
  } else {
    s = blockIdx.x / max_spans;
    const int a = q_start[s], b = q_start[s + 1];
    alone = b - a <= span;
    t0 = a + (blockIdx.x % max_spans) * span;
    t1 = min(b, t0 + span);
    if (MODE == 1 && alone) return;
  }
  if (t0 >= t1) return;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int vl = tid / CS, cg = tid % CS;
  const int col = vl * RV;                // the thread's first column within the block
  const bool active = col < VB;
  const size_t mine_at = ((size_t)hd * dv + v0 + col) * DP + cg * REC_R;
  float* st = state + (size_t)state_slots[s] * slot_stride + mine_at;
  if (!alone) st = span_state + (size_t)blockIdx.x * ((size_t)H * dv * DP) + mine_at;
  const bool decays_out = MODE == 1 && blockIdx.z == 0;
  if (decays_out)
    for (int c = tid; c < DP; c += nthreads) pd[c] = 1.f;
  float S[RV][REC_R];
#pragma unroll
  for (int r = 0; r < RV; ++r) {
#pragma unroll
    for (int j = 0; j < REC_R; ++j) S[r][j] = 0.f;
    if (MODE != 1 && active && v0 + col + r < dv) {
      const float4 a = *(const float4*)(st + (size_t)r * DP);
      const float4 b = *(const float4*)(st + (size_t)r * DP + 4);
      S[r][0] = a.x; S[r][1] = a.y; S[r][2] = a.z; S[r][3] = a.w;
      S[r][4] = b.x; S[r][5] = b.y; S[r][6] = b.z; S[r][7] = b.w;
    }
  }
  for (int c = tid; c < DP; c += nthreads)
    us[c] = (BEFORE && c < d) ? bonus[hd * d + c] : 0.f;
  for (int tc = t0; tc < t1; tc += TC) {
    const int n = min(TC, t1 - tc);
    __syncthreads();                      // the chunk before is read and reduced
    if (wide && n * CS * 4 >= nthreads) {
      // a task: 8 channels of a token; REC_STAGE tasks of a thread are in flight at once
      const int tasks = n * CS;
      for (int base = 0; base < tasks; base += REC_STAGE * nthreads) {
        Raw8<T> qr[REC_STAGE], kr[REC_STAGE];
        Raw8<float> zr[REC_STAGE];
#pragma unroll
        for (int u = 0; u < REC_STAGE; ++u) {
          const int task = base + tid + u * nthreads;
          if (task < tasks) {
            const size_t row = (size_t)(tc + task / CS);
            const int c = hd * d + (task % CS) * 8;
            if (MODE != 1) load_raw8(q + row * q_stride + c, qr[u]);
            load_raw8(k + row * k_stride + c, kr[u]);
            load_raw8(z + row * ((size_t)H * d) + c, zr[u]);
          }
        }
#pragma unroll
        for (int u = 0; u < REC_STAGE; ++u) {
          const int task = base + tid + u * nthreads;
          if (task < tasks) {
            const int at = (task / CS) * DP + (task % CS) * 8;
            float x8[8];
            widen8(zr[u], x8);
            if (rule != 2) {
              const float* zb = z_bias + hd * d + (task % CS) * 8;
#pragma unroll
              for (int j = 0; j < 8; ++j) x8[j] = decay_of(x8[j] + zb[j], rule, inv_tau);
            }
            *(float4*)(ds + at) = float4{x8[0], x8[1], x8[2], x8[3]};
            *(float4*)(ds + at + 4) = float4{x8[4], x8[5], x8[6], x8[7]};
            widen8(kr[u], x8);
            *(float4*)(ks + at) = float4{x8[0], x8[1], x8[2], x8[3]};
            *(float4*)(ks + at + 4) = float4{x8[4], x8[5], x8[6], x8[7]};
            if (MODE != 1) {
              widen8(qr[u], x8);
              *(float4*)(qs + at) = float4{x8[0] * q_scale, x8[1] * q_scale, x8[2] * q_scale,
                                           x8[3] * q_scale};
              *(float4*)(qs + at + 4) = float4{x8[4] * q_scale, x8[5] * q_scale, x8[6] * q_scale,
                                               x8[7] * q_scale};
            }
          }
        }
      }
      const int VG = VB / 8;
      for (int task = tid; task < n * VG; task += nthreads) {
        const int t = task / VG, x = (task % VG) * 8;
        float v8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (v0 + x < dv) load8<T>(v + (size_t)(tc + t) * v_stride + hd * dv + v0 + x, v8);
        *(float4*)(vs + t * VB + x) = float4{v8[0], v8[1], v8[2], v8[3]};
        *(float4*)(vs + t * VB + x + 4) = float4{v8[4], v8[5], v8[6], v8[7]};
      }
    } else {
    for (int i = tid; i < n * DP; i += nthreads) {
      const int t = i / DP, c = i % DP;
      float qv = 0.f, kv = 0.f, dc = 1.f;
      if (c < d) {
        const size_t row = (size_t)(tc + t);
        if (MODE != 1) qv = load_as_float<T>(q + row * q_stride + hd * d + c) * q_scale;
        kv = load_as_float<T>(k + row * k_stride + hd * d + c);
        const float zv = z[row * ((size_t)H * d) + hd * d + c];
        dc = rule == 2 ? zv : decay_of(zv + z_bias[hd * d + c], rule, inv_tau);
      }
      qs[i] = qv; ks[i] = kv; ds[i] = dc;
    }
    for (int i = tid; i < n * VB; i += nthreads) {
      const int t = i / VB, x = i % VB;
      vs[i] = v0 + x < dv ? load_as_float<T>(v + (size_t)(tc + t) * v_stride + hd * dv + v0 + x)
                          : 0.f;
    }
    }
    __syncthreads();
    if (decays_out)
      for (int c = tid; c < DP; c += nthreads) {
        float p = pd[c];
        for (int t = 0; t < n; ++t) p *= ds[t * DP + c];
        pd[c] = p;
      }
    if (active) {
      float u8[REC_R];
      if (BEFORE) {
        const float4* up = (const float4*)(us + cg * REC_R);
        const float4 u0 = up[0], u1 = up[1];
        u8[0] = u0.x; u8[1] = u0.y; u8[2] = u0.z; u8[3] = u0.w;
        u8[4] = u1.x; u8[5] = u1.y; u8[6] = u1.z; u8[7] = u1.w;
      }
      // REC_TB tokens at a time, so that their sums over the lanes are in flight together
      for (int tb = 0; tb < n; tb += REC_TB) {
        float acc[REC_TB][RV];
#pragma unroll
        for (int tt = 0; tt < REC_TB; ++tt) {
#pragma unroll
          for (int r = 0; r < RV; ++r) acc[tt][r] = 0.f;
          const int t = tb + tt;
          if (t >= n) continue;
          float vv[RV];
#pragma unroll
          for (int r = 0; r < RV; ++r) vv[r] = vs[t * VB + col + r];
          const float4* kp = (const float4*)(ks + t * DP + cg * REC_R);
          const float4* dp = (const float4*)(ds + t * DP + cg * REC_R);
          const float4 k0 = kp[0], k1 = kp[1], d0 = dp[0], d1 = dp[1];
          const float k8[REC_R] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
          const float d8[REC_R] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w};
          if (MODE == 1) {
#pragma unroll
            for (int r = 0; r < RV; ++r)
#pragma unroll
              for (int j = 0; j < REC_R; ++j) S[r][j] = fmaf(d8[j], S[r][j], k8[j] * vv[r]);
            continue;
          }
          const float4* qp = (const float4*)(qs + t * DP + cg * REC_R);
          const float4 q0 = qp[0], q1 = qp[1];
          const float q8[REC_R] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
          for (int r = 0; r < RV; ++r) {
            float a = 0.f;
            if (BEFORE) {
#pragma unroll
              for (int j = 0; j < REC_R; ++j) {
                const float kv = k8[j] * vv[r];
                a = fmaf(q8[j], fmaf(u8[j], kv, S[r][j]), a);
                S[r][j] = fmaf(d8[j], S[r][j], kv);
              }
            } else {
#pragma unroll
              for (int j = 0; j < REC_R; ++j) {
                S[r][j] = fmaf(d8[j], S[r][j], k8[j] * vv[r]);
                a = fmaf(q8[j], S[r][j], a);
              }
            }
            acc[tt][r] = a;
          }
        }
        if (MODE == 1) continue;
        if (shuffle) {
          // CS is a power of two: the CS lanes of a column lie side by side in the wave
          for (int m = 1; m < CS; m <<= 1) {
#pragma unroll
            for (int tt = 0; tt < REC_TB; ++tt)
#pragma unroll
              for (int r = 0; r < RV; ++r) acc[tt][r] += __shfl_xor(acc[tt][r], m, ZF_WAVE);
          }
          // every lane has the sums: lane tt of a column's lanes stores token tt (lane 0 all of
          // them where there are fewer lanes than tokens)
#pragma unroll
          for (int tt = 0; tt < REC_TB; ++tt) {
            const int t = tb + tt;
            if (t < n && cg == (CS >= REC_TB ? tt : 0)) {
              float* o = out + (size_t)(tc + t) * ((size_t)H * dv) + hd * dv + v0 + col;
              if (RV == 4 && (dv & 3) == 0) {    // a thread's four columns: all within dv or none
                if (v0 + col < dv)
                  *(float4*)o = float4{acc[tt][0], acc[tt][1], acc[tt][2], acc[tt][3]};
              } else {
#pragma unroll
                for (int r = 0; r < RV; ++r)
                  if (v0 + col + r < dv) o[r] = acc[tt][r];
              }
            }
          }
        } else {
#pragma unroll
          for (int tt = 0; tt < REC_TB; ++tt)
            if (tb + tt < n) {
#pragma unroll
              for (int r = 0; r < RV; ++r) po[((tb + tt) * VB + col + r) * CSP + cg] = acc[tt][r];
            }
        }
      }
    }
    if (MODE == 1 || shuffle) continue;
    __syncthreads();
    for (int i = tid; i < n * VB; i += nthreads) {
      const int t = i / VB, x = i % VB;
      if (v0 + x >= dv) continue;
      float sum = 0.f;
      for (int c = 0; c < CS; ++c) sum += po[i * CSP + c];
      out[(size_t)(tc + t) * ((size_t)H * dv) + hd * dv + v0 + x] = sum;
    }
  }
  if (MODE == 1 || alone) {
#pragma unroll
    for (int r = 0; r < RV; ++r)
      if (active && v0 + col + r < dv) {
        *(float4*)(st + (size_t)r * DP) = float4{S[r][0], S[r][1], S[r][2], S[r][3]};
        *(float4*)(st + (size_t)r * DP + 4) = float4{S[r][4], S[r][5], S[r][6], S[r][7]};
      }
  }
  if (decays_out)                         // each thread wrote the entries it reads here
    for (int c = tid; c < DP; c += nthreads)
      span_decay[((size_t)blockIdx.x * H + hd) * DP + c] = pd[c];
}

// The states at the spans' starts, one after the other: a thread keeps 4 neighbouring entries of
// a sequence's state (same head, same value column), walks the sequence's spans, leaves in
// span_state[n] the state before span n where the span's own sum was, and writes the state behind
// the last span to the request's slot.  grid (ceil(size / 4 / 256), sequence).
__global__ __launch_bounds__(256) void span_states_kernel(
    float* __restrict__ state, long long slot_stride, const int* __restrict__ state_slots,
    const int* __restrict__ q_start, float* __restrict__ span_state,
    const float* __restrict__ span_decay, int H, int dv, int DP, int span, int max_spans) {
  const int s = blockIdx.y;
  const int len = q_start[s + 1] - q_start[s];
  if (len <= span) return;
  const int n_spans = (len + span - 1) / span;
  const long long e = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= (long long)H * dv * DP) return;
  const int hd = (int)(e / ((long long)dv * DP)), c = (int)(e % DP);
  float* st = state + (size_t)state_slots[s] * slot_stride + e;
  float4 S = *(const float4*)st;
  for (int n = 0; n < n_spans; ++n) {
    const size_t w = (size_t)s * max_spans + n;
    float4* at = (float4*)(span_state + w * ((size_t)H * dv * DP) + e);
    const float4 own = *at;
    const float4 dc = *(const float4*)(span_decay + (w * H + hd) * DP + c);
    *at = S;
    S = float4{fmaf(dc.x, S.x, own.x), fmaf(dc.y, S.y, own.y), fmaf(dc.z, S.z, own.z),
               fmaf(dc.w, S.w, own.w)};
  }
  *(float4*)st = S;
}

// q, k [T, >= H d], v [T, >= H dv] with contiguous rows (strides in elements), z [T, H d] and
// out [T, H dv] float32, dense.  CS = ceil(d / 8) <= 32; VB <= 256 value columns a workgroup,
// RV (1, 2 or 4, dividing VB; another number: the most that divides) of them a thread,
// CS * VB / RV <= 256.
extern "C" int zf_decay_recurrence(const void* q, long long q_stride, const void* k,
                                   long long k_stride, const void* v, long long v_stride,
                                   int dtype, const float* z, const float* z_bias,
                                   const float* bonus, float* state, long long slot_stride,
                                   const int* state_slots, const int* q_start, float* out,
                                   int n_seqs, int H, int d, int dv, int VB, int RV, int rule,
                                   float inv_tau, float q_scale, hipStream_t stream) {
  if (n_seqs <= 0) return 0;
  const int CS = (d + REC_R - 1) / REC_R;
  if (H <= 0 || d <= 0 || dv <= 0 || CS > 32 || VB < 1 || VB > 256 ||
      rule < 0 || rule > 1 || slot_stride < (long long)H * dv * CS * REC_R)
    return -2;
  const int DP = CS * REC_R;
  const int TC = DP > 128 ? REC_TC / 2 : REC_TC;
  if (RV != 1 && RV != 2 && RV != 4) RV = VB % 4 == 0 ? 4 : (VB % 2 == 0 ? 2 : 1);
  if (VB % RV != 0 || CS * (VB / RV) > REC_MAX_THREADS) return -2;
  const int shuffle = (CS & (CS - 1)) == 0;
  const size_t smem = sizeof(float) * ((size_t)3 * TC * DP + 2 * DP + (size_t)TC * VB +
                                       (shuffle ? 0 : (size_t)TC * VB * (CS | 1)));
  if (smem > REC_MAX_LDS) return -2;
  const size_t esz = dtype == ZF_F32 ? 4 : 2;
  const int wide = d % 8 == 0 && dv % 8 == 0 && VB % 8 == 0 && q_stride % 8 == 0 &&
                   k_stride % 8 == 0 && v_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                   (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 && (uintptr_t)z % 16 == 0 &&
                   (uintptr_t)z_bias % 16 == 0 && esz > 0;
  const int threads = (CS * (VB / RV) + ZF_WAVE - 1) / ZF_WAVE * ZF_WAVE;
  const dim3 grid(n_seqs, H, (dv + VB - 1) / VB), block(threads);
#define REC_LAUNCH_RV(TT, BEF, MODE, RVV, GRID, RULE, SPAN, MAXS, SST, SDC)                      \
  hipLaunchKernelGGL((decay_recurrence_kernel<TT, BEF, MODE, RVV>), GRID, block, smem, stream,   \
                     (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v, v_stride, z,  \
                     z_bias, bonus, state, slot_stride, state_slots, q_start, out, H, d, dv, CS, \
                     VB, TC, RULE, inv_tau, q_scale, SPAN, MAXS, SST, SDC, wide, shuffle)
#define REC_LAUNCH(TT, BEF, MODE, GRID, RULE, SPAN, MAXS, SST, SDC)                              \
  if (RV == 4) REC_LAUNCH_RV(TT, BEF, MODE, 4, GRID, RULE, SPAN, MAXS, SST, SDC);                \
  else if (RV == 2) REC_LAUNCH_RV(TT, BEF, MODE, 2, GRID, RULE, SPAN, MAXS, SST, SDC);           \
  else REC_LAUNCH_RV(TT, BEF, MODE, 1, GRID, RULE, SPAN, MAXS, SST, SDC)
#define REC_LAUNCH_ANY(MODE, GRID, RULE, SPAN, MAXS, SST, SDC)                                   \
  if (dtype == ZF_F32) {                                                                         \
    if (bonus != nullptr) { REC_LAUNCH(float, true, MODE, GRID, RULE, SPAN, MAXS, SST, SDC); }   \
    else { REC_LAUNCH(float, false, MODE, GRID, RULE, SPAN, MAXS, SST, SDC); }                   \
  } else {                                                                                       \
    if (bonus != nullptr) { REC_LAUNCH(bf16_t, true, MODE, GRID, RULE, SPAN, MAXS, SST, SDC); }  \
    else { REC_LAUNCH(bf16_t, false, MODE, GRID, RULE, SPAN, MAXS, SST, SDC); }                  \
  }
  REC_LAUNCH_ANY(0, grid, rule, 0, 1, nullptr, nullptr)
  ZF_CHECK_LAUNCH();
}

// The same for portions cut into spans of ``span`` tokens (a multiple of 16), at most max_spans a
// sequence.  z [T, H d] is overwritten with the decays.  span_state float32 [n_seqs * max_spans,
// H dv padded d] and span_decay float32 [n_seqs * max_spans, H, padded d] are scratch.
extern "C" int zf_decay_recurrence_spans(const void* q, long long q_stride, const void* k,
                                         long long k_stride, const void* v, long long v_stride,
                                         int dtype, float* z, const float* z_bias,
                                         const float* bonus, float* state, long long slot_stride,
                                         const int* state_slots, const int* q_start, float* out,
                                         int n_tokens, int n_seqs, int H, int d, int dv, int VB,
                                         int RV, int rule, float inv_tau, float q_scale, int span,
                                         int max_spans, float* span_state, float* span_decay,
                                         hipStream_t stream) {
  if (n_seqs <= 0 || n_tokens <= 0) return 0;
  const int CS = (d + REC_R - 1) / REC_R;
  if (H <= 0 || d <= 0 || dv <= 0 || CS > 32 || VB < 1 || VB > 256 ||
      rule < 0 || rule > 1 || slot_stride < (long long)H * dv * CS * REC_R || span < REC_TC || span % REC_TC != 0 || max_spans < 1 ||
      span_state == nullptr || span_decay == nullptr)
    return -2;
  const int DP = CS * REC_R;
  const int TC = DP > 128 ? REC_TC / 2 : REC_TC;
  if (RV != 1 && RV != 2 && RV != 4) RV = VB % 4 == 0 ? 4 : (VB % 2 == 0 ? 2 : 1);
  if (VB % RV != 0 || CS * (VB / RV) > REC_MAX_THREADS) return -2;
  const int shuffle = (CS & (CS - 1)) == 0;
  const size_t smem = sizeof(float) * ((size_t)3 * TC * DP + 2 * DP + (size_t)TC * VB +
                                       (shuffle ? 0 : (size_t)TC * VB * (CS | 1)));
  if (smem > REC_MAX_LDS) return -2;
  const size_t esz = dtype == ZF_F32 ? 4 : 2;
  const int wide = d % 8 == 0 && dv % 8 == 0 && VB % 8 == 0 && q_stride % 8 == 0 &&
                   k_stride % 8 == 0 && v_stride % 8 == 0 && (uintptr_t)q % 16 == 0 &&
                   (uintptr_t)k % 16 == 0 && (uintptr_t)v % 16 == 0 && (uintptr_t)z % 16 == 0 &&
                   (uintptr_t)z_bias % 16 == 0 && esz > 0;
  const int threads = (CS * (VB / RV) + ZF_WAVE - 1) / ZF_WAVE * ZF_WAVE;
  const dim3 grid(n_seqs * max_spans, H, (dv + VB - 1) / VB), block(threads);
  const long long n = (long long)n_tokens * H * d;
  hipLaunchKernelGGL(decays_in_place_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                     stream, z, z_bias, n, H * d, rule, inv_tau);
  REC_LAUNCH_ANY(1, grid, 2, span, max_spans, span_state, span_decay)
  const long long quads = (long long)H * dv * DP / 4;
  hipLaunchKernelGGL(span_states_kernel, dim3((unsigned)((quads + 255) / 256), n_seqs), dim3(256),
                     0, stream, state, slot_stride, state_slots, q_start, span_state, span_decay,
                     H, dv, DP, span, max_spans);
  REC_LAUNCH_ANY(2, grid, 2, span, max_spans, span_state, span_decay)
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- norm a head, gain, gate
// a wave a (token, head): out[t, h, :] = o / sqrt(mean(o^2) + eps) * gain * silu(g[t, h, :]);
// gain [dv] (one for all heads) or [H dv].  o float32, g and out in the rows' type.
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
    const float* __restrict__ o, const float* __restrict__ gain, int gain_per_head,
    const T* __restrict__ g, long long g_stride, T* __restrict__ out, int n_rows, int H, int dv,
    float eps) {
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int r = blockIdx.x * (blockDim.x / ZF_WAVE) + wave;       // (token, head)
  if (r >= n_rows) return;
  const int t = r / H, hd = r % H;
  const float* row = o + (size_t)r * dv;
  float ss = 0.f;
  for (int i = lane; i < dv; i += ZF_WAVE) ss = fmaf(row[i], row[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)dv + eps);
  const T* gr = g + (size_t)t * g_stride + hd * dv;
  const float* gn = gain + (gain_per_head ? hd * dv : 0);
  for (int i = lane; i < dv; i += ZF_WAVE) {
    const float gv = load_as_float<T>(gr + i);
    const float silu = gv / (1.0f + expf(-gv));
    store_from_float<T>(out + (size_t)r * dv + i, row[i] * inv * gn[i] * silu);
  }
}

extern "C" int zf_head_norm_gate(const float* o, const float* gain, int gain_per_head,
                                 const void* g, long long g_stride, void* out, int dtype, int T,
                                 int H, int dv, float eps, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || dv <= 0) return -2;
  const int rows = T * H;
  const dim3 grid((rows + 3) / 4), block(4 * ZF_WAVE);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, block, 0, stream, o, gain,
                       gain_per_head, (const float*)g, g_stride, (float*)out, rows, H, dv, eps);
  else
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, block, 0, stream, o, gain,
                       gain_per_head, (const bf16_t*)g, g_stride, (bf16_t*)out, rows, H, dv, eps);
  ZF_CHECK_LAUNCH();
}
