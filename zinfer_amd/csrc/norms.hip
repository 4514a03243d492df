// Norms over the rows of a float32 matrix, with a gain and an optional bias, that either
// store their result (float32 or bfloat16) or add it to a float32 destination:
//
//   centred:      n_i = (x_i - mean) / sqrt(mean((x - mean)^2) + eps) * w_i + b_i   (layer norm)
//   not centred:  n_i = x_i / sqrt(mean(x^2) + eps) * w_i (+ b_i)                   (RMS norm)
//
// All arithmetic is 32-bit.  The mean is taken first and the variance from the deviations
// (two passes over a row that is kept in registers), never as mean(x^2) - mean^2.  One
// workgroup per row; its result depends on that row alone.
#include "zf_common.h"

template <typename TO, bool ADD>
__device__ __forceinline__ void norm_store(TO* o, float v) {
  if constexpr (ADD) {
    *o = (TO)(*o + v);      // ADD is only instantiated with TO = float
  } else {
    store_from_float<TO>(o, v);
  }
}

// any width: the row is read three times
template <typename TO, bool ADD>
__global__ __launch_bounds__(256) void norm_rows_kernel(const float* __restrict__ x,
                                                        const float* __restrict__ gain,
                                                        const float* __restrict__ bias,
                                                        TO* __restrict__ out, int W, float eps,
                                                        int centred) {
  __shared__ float red[16];
  const float* row = x + (size_t)blockIdx.x * W;
  TO* o = out + (size_t)blockIdx.x * W;
  float mean = 0.f;
  if (centred) {
    float s = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) s += row[i];
    mean = block_sum(s, red) / (float)W;
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float d = row[i] - mean;
    ss += d * d;
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = (row[i] - mean) * inv * gain[i];
    if (bias != nullptr) v += bias[i];
    norm_store<TO, ADD>(o + i, v);
  }
}

// widths that are a multiple of 4 up to 8192: a thread keeps its part of the row (at most 8
// float4) in registers, so the row is read once
template <typename TO, bool ADD>
__global__ __launch_bounds__(256) void norm_rows_vec_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ gain,
                                                            const float* __restrict__ bias,
                                                            TO* __restrict__ out, int W,
                                                            float eps, int centred) {
  __shared__ float red[16];
  const float4* row = (const float4*)(x + (size_t)blockIdx.x * W);
  TO* o = out + (size_t)blockIdx.x * W;
  const int n4 = W / 4;
  float4 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = c < n4 ? row[c] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float mean = 0.f;
  if (centred) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    mean = block_sum(s, red) / (float)W;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      v[i].x -= mean; v[i].y -= mean; v[i].z -= mean; v[i].w -= mean;
      ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      const float4 g = ((const float4*)gain)[c];
      float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
      if (bias != nullptr) b = ((const float4*)bias)[c];
      norm_store<TO, ADD>(o + 4 * c + 0, v[i].x * inv * g.x + b.x);
      norm_store<TO, ADD>(o + 4 * c + 1, v[i].y * inv * g.y + b.y);
      norm_store<TO, ADD>(o + 4 * c + 2, v[i].z * inv * g.z + b.z);
      norm_store<TO, ADD>(o + 4 * c + 3, v[i].w * inv * g.w + b.w);
    }
  }
}

template <typename TO, bool ADD>
static void launch_norm_rows(const float* x, const float* gain, const float* bias, void* out,
                             int T, int W, float eps, int centred, hipStream_t stream) {
  if (W % 4 == 0 && W <= 8192)
    hipLaunchKernelGGL((norm_rows_vec_kernel<TO, ADD>), dim3(T), dim3(256), 0, stream, x, gain,
                       bias, (TO*)out, W, eps, centred);
  else
    hipLaunchKernelGGL((norm_rows_kernel<TO, ADD>), dim3(T), dim3(256), 0, stream, x, gain, bias,
                       (TO*)out, W, eps, centred);
}

// out = norm(x) (add == 0) or out += norm(x) (add != 0, out float32); bias may be null
extern "C" int zf_norm_rows(const float* x, const float* gain, const float* bias, void* out,
                            int out_dtype, int T, int W, float eps, int centred, int add,
                            hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || (add && out_dtype != ZF_F32)) return -2;
  if (add)
    launch_norm_rows<float, true>(x, gain, bias, out, T, W, eps, centred, stream);
  else if (out_dtype == ZF_F32)
    launch_norm_rows<float, false>(x, gain, bias, out, T, W, eps, centred, stream);
  else
    launch_norm_rows<bf16_t, false>(x, gain, bias, out, T, W, eps, centred, stream);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- a norm behind a sublayer and the one before the next
// x += norm_a(y); out = norm_b(x): the norm that closes a sublayer adds its result into the
// residual stream, and the norm that opens the next sublayer reads the sum while the row is
// still in registers (one kernel and one pass over the stream instead of two).  Widths that
// are a multiple of 4 up to 8192.  Each norm as in norm_rows (32-bit, mean first, variance from
// the deviations): the same numbers as the two kernels one after the other.
template <typename TO>
__global__ __launch_bounds__(256) void norm_add_norm_kernel(
    const float* __restrict__ y, const float* __restrict__ gain_a, const float* __restrict__ bias_a,
    float eps_a, int centred_a, float* __restrict__ x, const float* __restrict__ gain_b,
    const float* __restrict__ bias_b, float eps_b, int centred_b, TO* __restrict__ out, int W) {
  __shared__ float red[16];
  const float4* yrow = (const float4*)(y + (size_t)blockIdx.x * W);
  float4* xrow = (float4*)(x + (size_t)blockIdx.x * W);
  TO* o = out + (size_t)blockIdx.x * W;
  const int n4 = W / 4;
  float4 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = c < n4 ? yrow[c] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // one norm over the row held in v: v = (v - mean) * inv * gain + bias, in place
  auto norm = [&](const float* gain, const float* bias, float eps, int centred) {
    float mean = 0.f;
    if (centred) {
      float s = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
      mean = block_sum(s, red) / (float)W;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = threadIdx.x + i * 256;
      if (c < n4) {
        v[i].x -= mean; v[i].y -= mean; v[i].z -= mean; v[i].w -= mean;
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
      }
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int c = threadIdx.x + i * 256;
      if (c < n4) {
        const float4 g = ((const float4*)gain)[c];
        float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
        if (bias != nullptr) b = ((const float4*)bias)[c];
        v[i].x = v[i].x * inv * g.x + b.x;
        v[i].y = v[i].y * inv * g.y + b.y;
        v[i].z = v[i].z * inv * g.z + b.z;
        v[i].w = v[i].w * inv * g.w + b.w;
      }
    }
  };
  norm(gain_a, bias_a, eps_a, centred_a);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      const float4 r = xrow[c];
      v[i].x = r.x + v[i].x; v[i].y = r.y + v[i].y; v[i].z = r.z + v[i].z; v[i].w = r.w + v[i].w;
      xrow[c] = v[i];
    }
  }
  norm(gain_b, bias_b, eps_b, centred_b);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      store_from_float<TO>(o + 4 * c + 0, v[i].x);
      store_from_float<TO>(o + 4 * c + 1, v[i].y);
      store_from_float<TO>(o + 4 * c + 2, v[i].z);
      store_from_float<TO>(o + 4 * c + 3, v[i].w);
    }
  }
}

extern "C" int zf_norm_add_norm(const float* y, const float* gain_a, const float* bias_a,
                                float eps_a, int centred_a, float* x, const float* gain_b,
                                const float* bias_b, float eps_b, int centred_b, void* out,
                                int out_dtype, int T, int W, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || W % 4 != 0 || W > 8192) return -2;
  if (out_dtype == ZF_F32)
    hipLaunchKernelGGL(norm_add_norm_kernel<float>, dim3(T), dim3(256), 0, stream, y, gain_a,
                       bias_a, eps_a, centred_a, x, gain_b, bias_b, eps_b, centred_b, (float*)out, W);
  else
    hipLaunchKernelGGL(norm_add_norm_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, y, gain_a,
                       bias_a, eps_a, centred_a, x, gain_b, bias_b, eps_b, centred_b,
                       (bf16_t*)out, W);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- a norm behind a sublayer, and the sum as the next one reads it
// x += norm(y); out = x in out's storage type: for blocks whose sublayers read the stream as it
// is (no norm in front of them), the kernel that closes one sublayer leaves the sum in the
// type the next sublayer's products take.  Widths that are a multiple of 4 up to 8192; the
// norm as in norm_rows, the same numbers.
template <typename TO>
__global__ __launch_bounds__(256) void norm_add_store_kernel(
    const float* __restrict__ y, const float* __restrict__ gain, const float* __restrict__ bias,
    float eps, int centred, float* __restrict__ x, TO* __restrict__ out, int W) {
  __shared__ float red[16];
  const float4* yrow = (const float4*)(y + (size_t)blockIdx.x * W);
  float4* xrow = (float4*)(x + (size_t)blockIdx.x * W);
  TO* o = out + (size_t)blockIdx.x * W;
  const int n4 = W / 4;
  float4 v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    v[i] = c < n4 ? yrow[c] : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float mean = 0.f;
  if (centred) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    mean = block_sum(s, red) / (float)W;
  }
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      v[i].x -= mean; v[i].y -= mean; v[i].z -= mean; v[i].w -= mean;
      ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c < n4) {
      const float4 g = ((const float4*)gain)[c];
      float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
      if (bias != nullptr) b = ((const float4*)bias)[c];
      const float4 r = xrow[c];
      float4 s;
      s.x = r.x + (v[i].x * inv * g.x + b.x);
      s.y = r.y + (v[i].y * inv * g.y + b.y);
      s.z = r.z + (v[i].z * inv * g.z + b.z);
      s.w = r.w + (v[i].w * inv * g.w + b.w);
      xrow[c] = s;
      store_from_float<TO>(o + 4 * c + 0, s.x);
      store_from_float<TO>(o + 4 * c + 1, s.y);
      store_from_float<TO>(o + 4 * c + 2, s.z);
      store_from_float<TO>(o + 4 * c + 3, s.w);
    }
  }
}

extern "C" int zf_norm_add_store(const float* y, const float* gain, const float* bias, float eps,
                                 int centred, float* x, void* out, int out_dtype, int T, int W,
                                 hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || W % 4 != 0 || W > 8192) return -2;
  if (out_dtype == ZF_F32)
    hipLaunchKernelGGL(norm_add_store_kernel<float>, dim3(T), dim3(256), 0, stream, y, gain, bias,
                       eps, centred, x, (float*)out, W);
  else
    hipLaunchKernelGGL(norm_add_store_kernel<bf16_t>, dim3(T), dim3(256), 0, stream, y, gain,
                       bias, eps, centred, x, (bf16_t*)out, W);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- embedding plus a learned position
// x[t, :] = E[id[t], :] * scale + P[position[t], :], widened to float32
template <typename TW>
__global__ void embed_position_kernel(const TW* __restrict__ table, const int* __restrict__ ids,
                                      const TW* __restrict__ pos_table,
                                      const int* __restrict__ positions, float* __restrict__ out,
                                      int H, float scale) {
  const int t = blockIdx.x;
  const TW* row = table + (size_t)ids[t] * H;
  const TW* prow = pos_table + (size_t)positions[t] * H;
  float* o = out + (size_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    o[i] = load_as_float<TW>(row + i) * scale + load_as_float<TW>(prow + i);
}

extern "C" int zf_embed_position(const void* table, const void* pos_table, int table_dtype,
                                 const int* ids, const int* positions, float* out, int T, int H,
                                 float scale, hipStream_t stream) {
  if (T <= 0) return 0;
  if (table_dtype == ZF_F32)
    hipLaunchKernelGGL(embed_position_kernel<float>, dim3(T), dim3(256), 0, stream,
                       (const float*)table, ids, (const float*)pos_table, positions, out, H, scale);
  else
    hipLaunchKernelGGL(embed_position_kernel<bf16_t>, dim3(T), dim3(256), 0, stream,
                       (const bf16_t*)table, ids, (const bf16_t*)pos_table, positions, out, H,
                       scale);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- several copies of the residual stream
// The stream is kept in S copies x_1 .. x_S, [S, T, W] floats.  Around a sublayer, row by row
// (a workgroup a row, a thread the same columns of all copies, everything 32-bit):
//
//   write:  x_t <- sum_s M[s, t] x_s + b[t] y   for all t from the old copies,
//           y = c0 y0 (+ c1 y1): the sublayer's output, in one branch or two
//   read:   u = sum_s a[s] x_s (the new copies), then out = u / sqrt(mean(u^2) + eps) * gain in
//           the products' type, or (no gain) out = u as floats
//
// Either half may be left out: the read alone before a layer's first sublayer and for the sum
// of the copies at the end, both between two sublayers.  The sums run over s in ascending order.
#define STREAMS_MAX 8

// V: columns a thread takes side by side (4: 16-byte loads and stores; W a multiple of 4)
template <typename TO, int V>
__global__ __launch_bounds__(256) void streams_step_kernel(
    float* __restrict__ x, long long copy_stride, int S, const float* __restrict__ y0,
    const float* __restrict__ y1, float c0, float c1, const float* __restrict__ M,
    const float* __restrict__ b, const float* __restrict__ a, const float* __restrict__ gain,
    float eps, TO* __restrict__ out, int W, int do_read) {
#pragma clang fp contract(off)
  extern __shared__ float u_row[];
  __shared__ float red[16];
  __shared__ float cm[STREAMS_MAX * STREAMS_MAX], cb[STREAMS_MAX], ca[STREAMS_MAX];
  // the coefficients once a workgroup
  if (threadIdx.x < S * S && M != nullptr) cm[threadIdx.x] = M[threadIdx.x];
  if (threadIdx.x < S) {
    if (b != nullptr) cb[threadIdx.x] = b[threadIdx.x];
    ca[threadIdx.x] = a != nullptr ? a[threadIdx.x] : 1.0f;
  }
  __syncthreads();
  const size_t row = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x * V; i < W; i += blockDim.x * V) {
    float v[STREAMS_MAX][V];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) {
      if (s < S) {
        if constexpr (V == 4) {
          const float4 q = *(const float4*)(x + s * copy_stride + row + i);
          v[s][0] = q.x; v[s][1] = q.y; v[s][2] = q.z; v[s][3] = q.w;
        } else {
          v[s][0] = x[s * copy_stride + row + i];
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) v[s][e] = 0.f;
      }
    }
    if (y0 != nullptr) {
      float y[V];
#pragma unroll
      for (int e = 0; e < V; ++e) {
        y[e] = c0 * y0[row + i + e];
        if (y1 != nullptr) y[e] = y[e] + c1 * y1[row + i + e];
      }
      float n[STREAMS_MAX][V];
#pragma unroll
      for (int t = 0; t < STREAMS_MAX; ++t) {
        if (t >= S) continue;
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) acc = acc + cm[s * S + t] * v[s][e];
          n[t][e] = acc + cb[t] * y[e];
        }
      }
#pragma unroll
      for (int t = 0; t < STREAMS_MAX; ++t)
        if (t < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) v[t][e] = n[t][e];
          if constexpr (V == 4)
            *(float4*)(x + t * copy_stride + row + i) = make_float4(n[t][0], n[t][1], n[t][2], n[t][3]);
          else
            x[t * copy_stride + row + i] = n[t][0];
        }
    }
    if (do_read) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
          if (s < S) u = u + ca[s] * v[s][e];
        if (gain == nullptr) {
          store_from_float<TO>(out + row + i + e, u);
        } else {
          u_row[i + e] = u;
          ss += u * u;
        }
      }
    }
  }
  if (!do_read || gain == nullptr) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  // (a thread reads back the columns it wrote itself)
  for (int i = threadIdx.x * V; i < W; i += blockDim.x * V) {
#pragma unroll
    for (int e = 0; e < V; ++e)
      store_from_float<TO>(out + row + i + e, u_row[i + e] * inv * gain[i + e]);
  }
}

// x [S, T, W] (copy_stride elements from one copy to the next).  y0 null: no write; else y1
// may be null.  do_read 0: no read; else `a` may be null (all ones) and `gain` may be null
// (out float32 = u; out_dtype must then be float32).
extern "C" int zf_streams_step(float* x, long long copy_stride, int S, const float* y0,
                               const float* y1, float c0, float c1, const float* M,
                               const float* b, const float* a, const float* gain, float eps,
                               void* out, int out_dtype, int T, int W, int do_read,
                               hipStream_t stream) {
  if (T <= 0) return 0;
  if (S < 1 || S > STREAMS_MAX || W <= 0 || W > 16384 || (y0 == nullptr && !do_read) ||
      (y0 != nullptr && (M == nullptr || b == nullptr)) || (do_read && out == nullptr) ||
      (do_read && gain == nullptr && out_dtype != ZF_F32))
    return -2;
  const size_t smem = (size_t)W * sizeof(float);
  const bool vec = W % 4 == 0 && copy_stride % 4 == 0 && ((uintptr_t)x % 16) == 0 &&
                   (y0 == nullptr || (uintptr_t)y0 % 16 == 0);
#define STREAMS_LAUNCH(TT, VV)                                                                   \
  hipLaunchKernelGGL((streams_step_kernel<TT, VV>), dim3(T), dim3(256), smem, stream, x,         \
                     copy_stride, S, y0, y1, c0, c1, M, b, a, gain, eps, (TT*)out, W, do_read)
  if (out_dtype == ZF_F32) {
    if (vec) STREAMS_LAUNCH(float, 4); else STREAMS_LAUNCH(float, 1);
  } else {
    if (vec) STREAMS_LAUNCH(bf16_t, 4); else STREAMS_LAUNCH(bf16_t, 1);
  }
  ZF_CHECK_LAUNCH();
}
