// A feed-forward layer made of many small experts, of which every token uses a few.
//
//   router:  z = R h + r            32-bit; the `top` largest z are chosen (the lower index
//            wins a tie), and their weights are the soft-max over the chosen z alone;
//            or (scoring 1) s = sigmoid(z), the choice goes by s + correction among the experts
//            of the best groups (a group of neighbours is marked by its two largest choice
//            scores added), and the weights are the chosen s over their sum (+ 1e-20)
//   expert:  g = min(Wg h, limit), u = clamp(Wu h, -limit, limit)      (limit <= 0: no clamp)
//            y = g * sigmoid(alpha * g) * (u + shift)
//            out = Wd y
//            or, without a gate: y = act(Wu h) with one of the plain activations
//   layer:   out[t] = sum over the chosen experts of weight * expert(h[t])
//
// Expert matrices are stacked: gate_up [E, 2 * ff, W] (an expert's gate rows, then its up
// rows) and down [E, W, ff].  Three kernels that stream the weights of the chosen experts
// token by token; every token's result depends on that token alone and its sums run in a
// fixed order, so a token gives the same bits whatever else is in the batch:
//
//  * moe_route         a workgroup per four tokens
//  * moe_gate_up       grid (token * slot, groups of outputs): y[t, slot, :] of the expert in
//                      that slot, the token's row staged in LDS as 32-bit numbers
//  * moe_down          grid (token, groups of outputs): out[t, n] (=, or += into) the weighted
//                      sum over the slots in slot order, 32-bit
//
// With `ids` null every token uses expert 0 with weight 1 (an expert that all tokens share).
#include "zf_common.h"

#define MOE_MAX_EXPERTS 1024

#define MOE_ROUTE_TOKENS 4     // tokens a workgroup routes: one wave each for the choice
#define MOE_ROUTE_WAVES 16     // waves of the workgroup: the experts' logits are dealt over them

template <typename T> struct Vec4 {};
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *(const uint2*)p;
    v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
};

// A workgroup of 16 waves takes four tokens.  Logits: wave w forms those of the experts w,
// w + 16, ... for all four tokens at once (a piece of the router's row is loaded once and meets
// the four tokens' pieces; every token's sum runs over its own row in a fixed order).  Choice:
// wave w then ranks token w's logits.
template <typename T>
__global__ __launch_bounds__(MOE_ROUTE_WAVES * ZF_WAVE) void moe_route_kernel(
    const T* __restrict__ h, const float* __restrict__ router, const float* __restrict__ bias,
    int* __restrict__ ids, float* __restrict__ weights, int n_tokens, int W, int E, int top,
    int scoring, const float* __restrict__ correction, int n_groups, int keep_groups,
    int mark_top, int normalize, float weight_scale, int n_extra, float* __restrict__ extra) {
  __shared__ float zs[MOE_ROUTE_TOKENS][MOE_MAX_EXPERTS], shares[MOE_ROUTE_TOKENS][MOE_MAX_EXPERTS];
  __shared__ int chosens[MOE_ROUTE_TOKENS][MOE_MAX_EXPERTS];
  __shared__ unsigned char kepts[MOE_ROUTE_TOKENS][MOE_MAX_EXPERTS];
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int t0 = blockIdx.x * MOE_ROUTE_TOKENS;
  const T* rows[MOE_ROUTE_TOKENS];
#pragma unroll
  for (int k = 0; k < MOE_ROUTE_TOKENS; ++k) rows[k] = h + (size_t)min(t0 + k, n_tokens - 1) * W;
  // (rows E .. E + n_extra - 1 of the router are no experts: their sigmoids go to `extra`)
  for (int e = wave; e < E + n_extra; e += MOE_ROUTE_WAVES) {
    const float* r = router + (size_t)e * W;
    float dot[MOE_ROUTE_TOKENS];
#pragma unroll
    for (int k = 0; k < MOE_ROUTE_TOKENS; ++k) dot[k] = 0.f;
    if (W % 4 == 0) {
#pragma unroll 4
      for (int i = lane * 4; i < W; i += ZF_WAVE * 4) {
        const float4 rv = *(const float4*)(r + i);
#pragma unroll
        for (int k = 0; k < MOE_ROUTE_TOKENS; ++k) {
          float x[4];
          Vec4<T>::load(rows[k] + i, x);
          dot[k] = fmaf(x[0], rv.x, dot[k]);
          dot[k] = fmaf(x[1], rv.y, dot[k]);
          dot[k] = fmaf(x[2], rv.z, dot[k]);
          dot[k] = fmaf(x[3], rv.w, dot[k]);
        }
      }
    } else {
      for (int i = lane; i < W; i += ZF_WAVE) {
        const float rv = r[i];
#pragma unroll
        for (int k = 0; k < MOE_ROUTE_TOKENS; ++k)
          dot[k] = fmaf(load_as_float<T>(rows[k] + i), rv, dot[k]);
      }
    }
    const float be = (bias != nullptr && e < E) ? bias[e] : 0.f;
#pragma unroll
    for (int k = 0; k < MOE_ROUTE_TOKENS; ++k) {
      const float z = wave_sum(dot[k]);
      if (lane == 0) {
        if (e < E) zs[k][e] = z + be;
        else if (t0 + k < n_tokens)
          extra[(size_t)(t0 + k) * n_extra + (e - E)] = 1.0f / (1.0f + expf(-z));
      }
    }
  }
  __syncthreads();
  const int t = t0 + wave;
  if (wave >= MOE_ROUTE_TOKENS || t >= n_tokens) return;
  float* z = zs[wave];
  float* share = shares[wave];
  int* chosen = chosens[wave];
  if (scoring != 0) {
    // scores s = sigmoid(z), or the soft-max over all of z (kept in `share`), choice scores
    // s + correction (in `z`)
    float zmax = 0.f, zsum = 1.f;
    if (scoring == 2) {
      zmax = -INFINITY;
      for (int e = lane; e < E; e += ZF_WAVE) zmax = fmaxf(zmax, z[e]);
      zmax = wave_max(zmax);
      zsum = 0.f;
      for (int e = lane; e < E; e += ZF_WAVE) zsum += expf(z[e] - zmax);
      zsum = wave_sum(zsum);
    }
    for (int e = lane; e < E; e += ZF_WAVE) {
      const float sc = scoring == 2 ? expf(z[e] - zmax) / zsum : 1.0f / (1.0f + expf(-z[e]));
      share[e] = sc;
      z[e] = sc + (correction != nullptr ? correction[e] : 0.f);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    if (n_groups > 0 && keep_groups < n_groups) {
      // a group's mark: its two largest choice scores added (its one score, if it has one)
      float* mark = (float*)chosen;
      unsigned char* kept = kepts[wave];
      const int size = E / n_groups;
      for (int g = lane; g < n_groups; g += ZF_WAVE) {
        float a = -INFINITY, b = -INFINITY;
        for (int e = g * size; e < (g + 1) * size; ++e) {
          const float v = z[e];
          if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
        }
        mark[g] = (size > 1 && mark_top > 1) ? a + b : a;
        kept[g] = 0;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
      for (int k = 0; k < keep_groups; ++k) {
        float best = -INFINITY;
        int arg = 0x7fffffff;
        for (int g = lane; g < n_groups; g += ZF_WAVE) {
          const float v = mark[g];
          if (!kept[g] && (v > best || arg == 0x7fffffff)) { best = v; arg = g; }
        }
#pragma unroll
        for (int off = ZF_WAVE / 2; off > 0; off >>= 1) {
          const float ob = __shfl_xor(best, off, ZF_WAVE);
          const int oa = __shfl_xor(arg, off, ZF_WAVE);
          if (oa != 0x7fffffff && (arg == 0x7fffffff || ob > best || (ob == best && oa < arg))) {
            best = ob; arg = oa;
          }
        }
        if (lane == 0 && arg != 0x7fffffff) kept[arg] = 1;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
      }
      // outside the kept groups nothing can be chosen
      for (int e = lane; e < E; e += ZF_WAVE)
        if (!kept[e / size]) z[e] = -INFINITY;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
    }
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
      float best = -INFINITY;
      int arg = 0x7fffffff;
      for (int e = lane; e < E; e += ZF_WAVE) {
        const float v = z[e];
        if (v > best) { best = v; arg = e; }
      }
#pragma unroll
      for (int off = ZF_WAVE / 2; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, ZF_WAVE);
        const int oa = __shfl_xor(arg, off, ZF_WAVE);
        if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
      }
      if (arg == 0x7fffffff) arg = 0;
      sum += share[arg];
      if (lane == 0) {
        chosen[k] = arg;
        z[arg] = -INFINITY;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_wave_barrier();
    }
    for (int k = lane; k < top; k += ZF_WAVE) {
      ids[(size_t)t * top + k] = chosen[k];
      const float sh = share[chosen[k]];
      weights[(size_t)t * top + k] = (normalize ? sh / (sum + 1e-20f) : sh) * weight_scale;
    }
    return;
  }
  // `top` rounds of: the largest remaining logit, the lowest index among equals
  float first = 0.f, sum = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int arg = 0x7fffffff;
    for (int e = lane; e < E; e += ZF_WAVE) {
      const float v = z[e];
      if (v > best) { best = v; arg = e; }
    }
#pragma unroll
    for (int off = ZF_WAVE / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, ZF_WAVE);
      const int oa = __shfl_xor(arg, off, ZF_WAVE);
      if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
    }
    if (arg == 0x7fffffff) arg = 0;            // nothing but NaN or -inf left
    if (k == 0) first = best;
    const float e_k = expf(best - first);       // the first chosen logit is the largest
    sum += e_k;
    if (lane == 0) {
      chosen[k] = arg;
      share[k] = e_k;
      z[arg] = -INFINITY;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
  }
  for (int k = lane; k < top; k += ZF_WAVE) {
    ids[(size_t)t * top + k] = chosen[k];
    weights[(size_t)t * top + k] = share[k] / sum;
  }
}

extern "C" int zf_moe_route(const void* h, int dtype, const float* router, const float* bias,
                            int* ids, float* weights, int T, int W, int E, int top,
                            int scoring, const float* correction, int n_groups, int keep_groups,
                            int mark_top, int normalize, float weight_scale, int n_extra,
                            float* extra, hipStream_t stream) {
  if (T <= 0) return 0;
  if (E <= 0 || E > MOE_MAX_EXPERTS || top <= 0 || top > E || scoring < 0 || scoring > 2 ||
      n_extra < 0 || (n_extra > 0 && extra == nullptr) || mark_top < 1 || mark_top > 2 ||
      n_groups < 0 || (n_groups > 0 && (E % n_groups != 0 || keep_groups < 1 ||
                                        keep_groups > n_groups ||
                                        top > keep_groups * (E / n_groups))))
    return -2;
  const dim3 grid((T + MOE_ROUTE_TOKENS - 1) / MOE_ROUTE_TOKENS), block(MOE_ROUTE_WAVES * ZF_WAVE);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(moe_route_kernel<float>, grid, block, 0, stream, (const float*)h, router,
                       bias, ids, weights, T, W, E, top, scoring, correction, n_groups,
                       keep_groups, mark_top, normalize, weight_scale, n_extra, extra);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)h, router,
                       bias, ids, weights, T, W, E, top, scoring, correction, n_groups,
                       keep_groups, mark_top, normalize, weight_scale, n_extra, extra);
  ZF_CHECK_LAUNCH();
}

// the activation of an expert's two products
__device__ __forceinline__ float gated_unit(float g, float u, float limit, float alpha,
                                            float shift) {
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g * (1.0f / (1.0f + expf(-alpha * g))) * (u + shift);
}

// dot product of a weight row with a vector held in LDS as floats, lanes side by side; a
// bfloat16 row whose length is a multiple of 8 comes as 16-byte loads
template <typename T>
__device__ __forceinline__ float row_dot_lds(const T* __restrict__ w, const float* __restrict__ x,
                                             int n, int lane) {
  float dot = 0.f;
  if constexpr (sizeof(T) == 2) {
    if (n % 8 == 0) {
      for (int i = lane * 8; i < n; i += ZF_WAVE * 8) {
        const uint4 v = *(const uint4*)(w + i);
        const uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          dot = fmaf(__uint_as_float(p[c] << 16), x[i + 2 * c], dot);
          dot = fmaf(__uint_as_float(p[c] & 0xffff0000u), x[i + 2 * c + 1], dot);
        }
      }
      return dot;
    }
  }
  for (int i = lane; i < n; i += ZF_WAVE) dot = fmaf(load_as_float<T>(w + i), x[i], dot);
  return dot;
}

// the same between two rows in global memory
template <typename T>
__device__ __forceinline__ float row_dot(const T* __restrict__ w, const T* __restrict__ y, int n,
                                         int lane) {
  float dot = 0.f;
  if constexpr (sizeof(T) == 2) {
    if (n % 8 == 0) {
      for (int i = lane * 8; i < n; i += ZF_WAVE * 8) {
        const uint4 a = *(const uint4*)(w + i);
        const uint4 b = *(const uint4*)(y + i);
        const uint32_t p[4] = {a.x, a.y, a.z, a.w}, q[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          dot = fmaf(__uint_as_float(p[c] << 16), __uint_as_float(q[c] << 16), dot);
          dot = fmaf(__uint_as_float(p[c] & 0xffff0000u), __uint_as_float(q[c] & 0xffff0000u), dot);
        }
      }
      return dot;
    }
  }
  for (int i = lane; i < n; i += ZF_WAVE)
    dot = fmaf(load_as_float<T>(w + i), load_as_float<T>(y + i), dot);
  return dot;
}

#define MOE_WAVES 4
#define MOE_GU_PER_WAVE 4      // outputs of y a wave computes, one after the other

// GATED: gate_up [E, 2 ff, W] and the gated activation; else `gate_up` holds the up rows alone,
// [E, ff, W], and y = activation_value(up, act) (`act` by the numbers of zf_common.h).
template <typename T, bool GATED>
__global__ __launch_bounds__(MOE_WAVES * ZF_WAVE) void moe_gate_up_kernel(
    const T* __restrict__ h, const T* __restrict__ gate_up, const int* __restrict__ ids,
    T* __restrict__ y, int W, int ff, int slots, float limit, float alpha, float shift, int act,
    int n_experts) {
  extern __shared__ float xs[];                    // the token's row, [W]
  const int ts = blockIdx.x, t = ts / slots;
  const int e = ids != nullptr ? ids[ts] : 0;
  if (e >= n_experts) return;                      // an output of the router without an expert
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const T* row = h + (size_t)t * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) xs[i] = load_as_float<T>(row + i);
  __syncthreads();
  const T* we = gate_up + (size_t)e * (GATED ? 2 : 1) * ff * W;
  const int j0 = (blockIdx.y * MOE_WAVES + wave) * MOE_GU_PER_WAVE;
  if (j0 >= ff) return;
  if constexpr (sizeof(T) == 2) {
    if (W % 8 == 0) {
      // the wave's outputs side by side: eight 16-byte loads in flight for every piece of the
      // token's row (an output beyond the last repeats the last one and is not stored)
      float dg[MOE_GU_PER_WAVE], du[MOE_GU_PER_WAVE];
      const T* gr[MOE_GU_PER_WAVE];
#pragma unroll
      for (int o = 0; o < MOE_GU_PER_WAVE; ++o) {
        dg[o] = du[o] = 0.f;
        gr[o] = we + (size_t)min(j0 + o, ff - 1) * W;
      }
#pragma unroll 2
      for (int i = lane * 8; i < W; i += ZF_WAVE * 8) {
        uint4 a[MOE_GU_PER_WAVE], b[MOE_GU_PER_WAVE];
#pragma unroll
        for (int o = 0; o < MOE_GU_PER_WAVE; ++o) {
          a[o] = *(const uint4*)(gr[o] + i);
          if constexpr (GATED) b[o] = *(const uint4*)(gr[o] + (size_t)ff * W + i);
        }
        const float4 x0 = *(const float4*)(xs + i), x1 = *(const float4*)(xs + i + 4);
        const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
        for (int o = 0; o < MOE_GU_PER_WAVE; ++o) {
          const uint32_t p[4] = {a[o].x, a[o].y, a[o].z, a[o].w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            dg[o] = fmaf(__uint_as_float(p[c] << 16), x[2 * c], dg[o]);
            dg[o] = fmaf(__uint_as_float(p[c] & 0xffff0000u), x[2 * c + 1], dg[o]);
          }
          if constexpr (GATED) {
            const uint32_t q[4] = {b[o].x, b[o].y, b[o].z, b[o].w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
              du[o] = fmaf(__uint_as_float(q[c] << 16), x[2 * c], du[o]);
              du[o] = fmaf(__uint_as_float(q[c] & 0xffff0000u), x[2 * c + 1], du[o]);
            }
          }
        }
      }
#pragma unroll
      for (int o = 0; o < MOE_GU_PER_WAVE; ++o) {
        const float g = wave_sum(dg[o]);
        float r;
        if constexpr (GATED) r = gated_unit(g, wave_sum(du[o]), limit, alpha, shift);
        else r = activation_value(g, act);
        if (lane == 0 && j0 + o < ff) store_from_float<T>(y + (size_t)ts * ff + j0 + o, r);
      }
      return;
    }
  }
  for (int j = j0; j < j0 + MOE_GU_PER_WAVE && j < ff; ++j) {
    const float g = wave_sum(row_dot_lds<T>(we + (size_t)j * W, xs, W, lane));
    float r;
    if constexpr (GATED) {
      const float u = wave_sum(row_dot_lds<T>(we + (size_t)(ff + j) * W, xs, W, lane));
      r = gated_unit(g, u, limit, alpha, shift);
    } else {
      r = activation_value(g, act);
    }
    if (lane == 0) store_from_float<T>(y + (size_t)ts * ff + j, r);
  }
}

// gated != 0: gate_up [E, 2 ff, W]; else [E, ff, W] and the plain activation `act`
extern "C" int zf_moe_gate_up(const void* h, const void* gate_up, int dtype, const int* ids,
                              void* y, int T, int W, int ff, int slots, float limit, float alpha,
                              float shift, int gated, int act, int n_experts,
                              hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || ff <= 0 || slots <= 0 || (size_t)W * sizeof(float) > 64 * 1024 || act < 0 ||
      act > 4)
    return -2;
  const int per_wg = MOE_WAVES * MOE_GU_PER_WAVE;
  dim3 grid(T * slots, (ff + per_wg - 1) / per_wg);
  const size_t smem = (size_t)W * sizeof(float);
#define MOE_GU_LAUNCH(TT, G)                                                                      \
  hipLaunchKernelGGL((moe_gate_up_kernel<TT, G>), grid, dim3(MOE_WAVES * ZF_WAVE), smem, stream, \
                     (const TT*)h, (const TT*)gate_up, ids, (TT*)y, W, ff, slots, limit, alpha,  \
                     shift, act, n_experts)
  if (dtype == ZF_F32) {
    if (gated) MOE_GU_LAUNCH(float, true); else MOE_GU_LAUNCH(float, false);
  } else {
    if (gated) MOE_GU_LAUNCH(bf16_t, true); else MOE_GU_LAUNCH(bf16_t, false);
  }
  ZF_CHECK_LAUNCH();
}

#define MOE_DOWN_PER_WAVE 4

template <typename T>
__global__ __launch_bounds__(MOE_WAVES * ZF_WAVE) void moe_down_kernel(
    const T* __restrict__ y, const T* __restrict__ down, const int* __restrict__ ids,
    const float* __restrict__ weights, float* __restrict__ out, int W, int ff, int slots,
    int add, int n_experts, const T* __restrict__ h) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int n0 = (blockIdx.y * MOE_WAVES + wave) * MOE_DOWN_PER_WAVE;
  if (n0 >= W) return;
  if constexpr (sizeof(T) == 2) {
    if (ff % 8 == 0) {
      // the wave's outputs side by side; a lane adds its pieces over all slots (in slot order)
      // before the lanes are added up, so there is one sum over the wave per output
      float tot[MOE_DOWN_PER_WAVE], same[MOE_DOWN_PER_WAVE];
#pragma unroll
      for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) tot[o] = same[o] = 0.f;
      for (int s = 0; s < slots; ++s) {
        const int ts = t * slots + s;
        const int e = ids != nullptr ? ids[ts] : 0;
        const float c = weights != nullptr ? weights[ts] : 1.0f;
        if (e >= n_experts) {                      // no expert: the token's own row, weighted
#pragma unroll
          for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o)
            same[o] = fmaf(c, load_as_float<T>(h + (size_t)t * W + min(n0 + o, W - 1)), same[o]);
          continue;
        }
        const T* yr = y + (size_t)ts * ff;
        const T* wr[MOE_DOWN_PER_WAVE];
#pragma unroll
        for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o)
          wr[o] = down + ((size_t)e * W + min(n0 + o, W - 1)) * ff;
        float part[MOE_DOWN_PER_WAVE];
#pragma unroll
        for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) part[o] = 0.f;
        for (int i = lane * 8; i < ff; i += ZF_WAVE * 8) {
          uint4 a[MOE_DOWN_PER_WAVE];
#pragma unroll
          for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) a[o] = *(const uint4*)(wr[o] + i);
          const uint4 b = *(const uint4*)(yr + i);
          const uint32_t q[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
          for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) {
            const uint32_t p[4] = {a[o].x, a[o].y, a[o].z, a[o].w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              part[o] = fmaf(__uint_as_float(p[k] << 16), __uint_as_float(q[k] << 16), part[o]);
              part[o] = fmaf(__uint_as_float(p[k] & 0xffff0000u),
                             __uint_as_float(q[k] & 0xffff0000u), part[o]);
            }
          }
        }
#pragma unroll
        for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) tot[o] = fmaf(c, part[o], tot[o]);
      }
#pragma unroll
      for (int o = 0; o < MOE_DOWN_PER_WAVE; ++o) {
        const float total = wave_sum(tot[o]) + same[o];
        if (lane == 0 && n0 + o < W) {
          float* dst = out + (size_t)t * W + n0 + o;
          *dst = add ? *dst + total : total;
        }
      }
      return;
    }
  }
  for (int n = n0; n < n0 + MOE_DOWN_PER_WAVE && n < W; ++n) {
    float total = 0.f;
    for (int s = 0; s < slots; ++s) {
      const int ts = t * slots + s;
      const int e = ids != nullptr ? ids[ts] : 0;
      if (e >= n_experts) {
        total += (weights != nullptr ? weights[ts] : 1.0f) * load_as_float<T>(h + (size_t)t * W + n);
        continue;
      }
      const T* wr = down + ((size_t)e * W + n) * ff;
      const T* yr = y + (size_t)ts * ff;
      const float dot = wave_sum(row_dot<T>(wr, yr, ff, lane));
      total += (weights != nullptr ? weights[ts] : 1.0f) * dot;
    }
    if (lane == 0) {
      float* o = out + (size_t)t * W + n;
      *o = add ? *o + total : total;
    }
  }
}

extern "C" int zf_moe_down(const void* y, const void* down, int dtype, const int* ids,
                           const float* weights, float* out, int T, int W, int ff, int slots,
                           int add, int n_experts, const void* h, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || ff <= 0 || slots <= 0) return -2;
  const int per_wg = MOE_WAVES * MOE_DOWN_PER_WAVE;
  dim3 grid(T, (W + per_wg - 1) / per_wg);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(moe_down_kernel<float>, grid, dim3(MOE_WAVES * ZF_WAVE), 0, stream,
                       (const float*)y, (const float*)down, ids, weights, out, W, ff, slots, add,
                       n_experts, (const float*)h);
  else
    hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, dim3(MOE_WAVES * ZF_WAVE), 0, stream,
                       (const bf16_t*)y, (const bf16_t*)down, ids, weights, out, W, ff, slots,
                       add, n_experts, (const bf16_t*)h);
  ZF_CHECK_LAUNCH();
}

// ---------------------------------------------------------------- the activation alone
// out[t, j] = act(gu[t, j], gu[t, ff + j]) for a gate/up product that a plain matrix kernel
// made (an expert that every token uses)
template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int ff, size_t n,
                                 float limit, float alpha, float shift,
                                 const float* __restrict__ row_factor, int factor_stride) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const size_t t = i / ff, j = i % ff;
  const float g = load_as_float<T>(gu + t * 2 * ff + j);
  const float u = load_as_float<T>(gu + t * 2 * ff + ff + j);
  float r = gated_unit(g, u, limit, alpha, shift);
  if (row_factor != nullptr) r *= row_factor[t * factor_stride];
  store_from_float<T>(out + i, r);
}

extern "C" int zf_gated_act(const void* gu, void* out, int dtype, int T, int ff, float limit,
                            float alpha, float shift, const float* row_factor,
                            int factor_stride, hipStream_t stream) {
  const size_t n = (size_t)T * ff;
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(gated_act_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                       (const float*)gu, (float*)out, ff, n, limit, alpha, shift, row_factor,
                       factor_stride);
  else
    hipLaunchKernelGGL(gated_act_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream,
                       (const bf16_t*)gu, (bf16_t*)out, ff, n, limit, alpha, shift, row_factor,
                       factor_stride);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  Many tokens (bfloat16): the (token, slot) pairs are sorted by expert, and every expert's
//  pairs run through MFMA tiles of 128 pairs against that expert's matrices.
//
//  * moe_sort      one workgroup: counts per expert, the pairs in expert order (`sorted`: the
//                  pair at a place, `place`: the place of a pair), and the list of tiles
//                  (expert, first place, places), their number in n_tiles[0].
//  * moe_grouped   grid (tile, columns): GATED: y[place, j] = act(gate, up) of the pair's token
//                  (rows of h gathered through `sorted`); else o[place, n] = down y[place] in
//                  32-bit.  A row's result depends on that row and the expert's matrix alone
//                  (sums along K in a fixed order), not on the rows beside it in the tile.
//  * moe_combine   out[t] (=, +=) sum over the slots, in slot order, of weight * o[place].
// =====================================================================================
#define MOE_TILE_ROWS 128

__global__ __launch_bounds__(1024) void moe_sort_kernel(
    const int* __restrict__ ids, int P, int E, int* __restrict__ sorted, int* __restrict__ place,
    int* __restrict__ tile_expert, int* __restrict__ tile_row0, int* __restrict__ tile_rows,
    int* __restrict__ n_tiles) {
  __shared__ int count[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
  for (int e = threadIdx.x; e < E; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += blockDim.x) atomicAdd(&count[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      for (int r = 0; r < count[e]; r += MOE_TILE_ROWS) {
        tile_expert[tiles] = e;
        tile_row0[tiles] = at + r;
        tile_rows[tiles] = min(MOE_TILE_ROWS, count[e] - r);
        ++tiles;
      }
      at += count[e];
    }
    n_tiles[0] = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < P; i += blockDim.x) {
    const int e = ids[i];
    const int at = start[e] + atomicAdd(&cursor[e], 1);
    sorted[at] = i;
    place[i] = at;
  }
}

extern "C" int zf_moe_sort(const int* ids, int P, int E, int* sorted, int* place, int* tile_expert,
                           int* tile_row0, int* tile_rows, int* n_tiles, hipStream_t stream) {
  if (P <= 0) return 0;
  if (E <= 0 || E > MOE_MAX_EXPERTS) return -2;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, P, E, sorted, place,
                     tile_expert, tile_row0, tile_rows, n_tiles);
  ZF_CHECK_LAUNCH();
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 moe_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float moe_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t moe_u32x4_t;

#define MOE_BK 64
#define MOE_LD (MOE_BK + 8)      // row stride in LDS (bfloat16): 16-byte reads of 8 lanes cover all banks

// 4 waves as 2 x 2: a wave takes 64 of the tile's 128 rows and 32 of the 64 columns of each of
// the MOE_NB weight tiles (GATED: the gate rows of MOE_NB / 2 groups of 64 outputs, then the up
// rows of the same outputs; else MOE_NB neighbouring groups of 64 outputs).  Two tiles, three
// workgroups to a CU, ran faster than four tiles with one or two, and loads issued one step
// ahead faster than two.  What bounds the loop with a few hundred rows an expert is the
// experts' matrices coming from memory: the tiles of one expert are dealt to workgroups whose
// numbers are equal modulo 8, which share an XCD and so its L2.
// v_mfma_f32_32x32x16_bf16: a lane holds row (or column) lane % 32 and k 8 (lane / 32) .. + 8
// of an operand, and of the result column lane % 32, rows 8 (r / 4) + 4 (lane / 32) + r % 4.
#define MOE_NB 2                 // weight tiles of 64 rows a workgroup holds
#define MOE_HALF (MOE_NB / 2)
// MODE 0: the down pass; 1: gate and up with the gated activation; 2: up alone, w [E, N, K], with
// the plain activation `act`.
template <int MODE>
__global__ __launch_bounds__(256) void moe_grouped_kernel(
    const bf16_t* __restrict__ a, long long lda, const int* __restrict__ sorted, int top,
    const bf16_t* __restrict__ w, const int* __restrict__ tile_expert,
    const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ n_tiles, void* __restrict__ out, int N, int K, float limit,
    float alpha, float shift, int act, int n_experts) {
  constexpr bool GATED = MODE == 1;
  constexpr bool GATHER = MODE != 0;            // rows of h found through the sort
  __shared__ __attribute__((aligned(16))) bf16_t as[MOE_TILE_ROWS * MOE_LD];
  __shared__ __attribute__((aligned(16))) bf16_t bs[MOE_NB * 64 * MOE_LD];
  // gridDim.x is a multiple of 8: workgroup x takes tile (x % 8) * (gridDim.x / 8) + x / 8, so
  // that neighbouring tiles (the same expert's) run on one XCD at about the same time
  const int tile = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile], row0 = tile_row0[tile], nrows = tile_rows[tile];
  if (e >= n_experts) return;                      // an output of the router without an expert
  const int c0 = blockIdx.y * 64 * (GATED ? MOE_HALF : MOE_NB);
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = wave / 2, wn = wave % 2;

  // what this thread stages: rows tid / 8 + 32 i of the pairs' tile (i < 4) and of the
  // weight tiles (i < 2 MOE_NB), 8 values at k0 + 8 (tid % 8)
  const int sr = tid / 8, sk = (tid % 8) * 8;
  const bf16_t* ap[4];
  const bf16_t* bp[2 * MOE_NB];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = sr + 32 * i;
    ap[i] = nullptr;
    if (r < nrows) {
      const int src = GATHER ? sorted[row0 + r] / top : row0 + r;
      ap[i] = a + (size_t)src * lda;
    }
  }
#pragma unroll
  for (int i = 0; i < 2 * MOE_NB; ++i) {
    const int r = sr + 32 * i;
    const int br = r % 64, bt = r / 64;              // row br of weight tile bt
    size_t wrow;
    bool ok;
    if (GATED) {                                     // the first half of the tiles: gate; then up
      const int j = c0 + (bt % MOE_HALF) * 64 + br;
      ok = j < N;
      wrow = (size_t)e * 2 * N + (size_t)(bt / MOE_HALF) * N + j;
    } else {
      const int n = c0 + bt * 64 + br;
      ok = n < N;
      wrow = (size_t)e * N + n;
    }
    bp[i] = ok ? w + wrow * K : nullptr;
  }
  moe_f32x16_t acc[2][MOE_NB];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < MOE_NB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const moe_u32x4_t zero = {0u, 0u, 0u, 0u};
  moe_u32x4_t ra[4], rb[2 * MOE_NB];
  auto fetch = [&](int k0) {
    const bool in_k = k0 + sk < K;                   // K is a multiple of 8
#pragma unroll
    for (int i = 0; i < 4; ++i)
      ra[i] = (ap[i] != nullptr && in_k) ? *(const moe_u32x4_t*)(ap[i] + k0 + sk) : zero;
#pragma unroll
    for (int i = 0; i < 2 * MOE_NB; ++i)
      rb[i] = (bp[i] != nullptr && in_k) ? *(const moe_u32x4_t*)(bp[i] + k0 + sk) : zero;
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += MOE_BK) {
    __syncthreads();                                 // the tiles of the step before are done with
#pragma unroll
    for (int i = 0; i < 4; ++i) *(moe_u32x4_t*)(as + (sr + 32 * i) * MOE_LD + sk) = ra[i];
#pragma unroll
    for (int i = 0; i < 2 * MOE_NB; ++i) *(moe_u32x4_t*)(bs + (sr + 32 * i) * MOE_LD + sk) = rb[i];
    __syncthreads();
    if (k0 + MOE_BK < K) fetch(k0 + MOE_BK);         // in flight while the MFMAs run
#pragma unroll
    for (int ks = 0; ks < MOE_BK; ks += 16) {
      moe_bf16x8_t af[2], bf[MOE_NB];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = *(const moe_bf16x8_t*)(as + (wm * 64 + i * 32 + lane % 32) * MOE_LD + ks + 8 * (lane / 32));
#pragma unroll
      for (int j = 0; j < MOE_NB; ++j)
        bf[j] = *(const moe_bf16x8_t*)(bs + (j * 64 + wn * 32 + lane % 32) * MOE_LD + ks + 8 * (lane / 32));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < MOE_NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
  }
  const int col = wn * 32 + lane % 32;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
      if (row >= nrows) continue;
      if (GATED) {
#pragma unroll
        for (int j = 0; j < MOE_HALF; ++j)
          if (c0 + j * 64 + col < N)
            ((bf16_t*)out)[(size_t)(row0 + row) * N + c0 + j * 64 + col] =
                float_to_bf16(gated_unit(acc[i][j][r], acc[i][MOE_HALF + j][r], limit, alpha, shift));
      } else if (MODE == 2) {
#pragma unroll
        for (int j = 0; j < MOE_NB; ++j)
          if (c0 + j * 64 + col < N)
            ((bf16_t*)out)[(size_t)(row0 + row) * N + c0 + j * 64 + col] =
                float_to_bf16(activation_value(acc[i][j][r], act));
      } else {
#pragma unroll
        for (int j = 0; j < MOE_NB; ++j)
          if (c0 + j * 64 + col < N)
            ((float*)out)[(size_t)(row0 + row) * N + c0 + j * 64 + col] = acc[i][j][r];
      }
    }
}

// mode 1: a = h [T, K] (rows gathered), w = gate_up [E, 2 N, K], out = y bfloat16 [P, N];
// mode 2: the same with w = up [E, N, K] and the plain activation `act`;
// mode 0: a = y [P, K], w = down [E, N, K], out = o float32 [P, N].  K a multiple of 8.
extern "C" int zf_moe_grouped(const void* a, long long lda, const int* sorted, int top,
                              const void* w, const int* tile_expert, const int* tile_row0,
                              const int* tile_rows, const int* n_tiles, void* out, int max_tiles,
                              int N, int K, int mode, float limit, float alpha, float shift,
                              int act, int n_experts, hipStream_t stream) {
  if (max_tiles <= 0) return 0;
  if (N <= 0 || K <= 0 || K % 8 != 0 || top <= 0 || mode < 0 || mode > 2 || act < 0 || act > 4)
    return -2;
  max_tiles = (max_tiles + 7) / 8 * 8;
#define MOE_GROUPED_LAUNCH(MODE, COLS)                                                           \
  hipLaunchKernelGGL(moe_grouped_kernel<MODE>, dim3(max_tiles, (N + (COLS) - 1) / (COLS)),       \
                     dim3(256), 0, stream, (const bf16_t*)a, lda, sorted, top, (const bf16_t*)w, \
                     tile_expert, tile_row0, tile_rows, n_tiles, out, N, K, limit, alpha, shift, \
                     act, n_experts)
  if (mode == 1) MOE_GROUPED_LAUNCH(1, 64 * MOE_HALF);
  else if (mode == 2) MOE_GROUPED_LAUNCH(2, 64 * MOE_NB);
  else MOE_GROUPED_LAUNCH(0, 64 * MOE_NB);
  ZF_CHECK_LAUNCH();
}

__global__ __launch_bounds__(256) void moe_combine_kernel(
    const float* __restrict__ o, const int* __restrict__ place, const float* __restrict__ weights,
    float* __restrict__ out, int W, int slots, int add, const int* __restrict__ ids,
    int n_experts, const bf16_t* __restrict__ h) {
  const int t = blockIdx.x;
  for (int n = blockIdx.y * blockDim.x + threadIdx.x; n < W; n += gridDim.y * blockDim.x) {
    float total = 0.f;
    for (int s = 0; s < slots; ++s) {
      const int ts = t * slots + s;
      // an output of the router without an expert hands the token's own row on
      const float v = (ids != nullptr && ids[ts] >= n_experts)
          ? bf16_to_float(h[(size_t)t * W + n]) : o[(size_t)place[ts] * W + n];
      total += weights[ts] * v;
    }
    float* dst = out + (size_t)t * W + n;
    *dst = add ? *dst + total : total;
  }
}

extern "C" int zf_moe_combine(const float* o, const int* place, const float* weights, float* out,
                              int T, int W, int slots, int add, const int* ids, int n_experts,
                              const void* h, hipStream_t stream) {
  if (T <= 0) return 0;
  if (W <= 0 || slots <= 0) return -2;
  int gy = (W + 255) / 256;
  if (gy > 64) gy = 64;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T, gy), dim3(256), 0, stream, o, place, weights,
                     out, W, slots, add, ids, n_experts, (const bf16_t*)h);
  ZF_CHECK_LAUNCH();
}
