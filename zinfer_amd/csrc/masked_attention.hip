// Causal attention over a paged cache with the pieces that newer decoders add to it, each a
// parameter of its own:
//
//   s_ij = scale * q_i . k_j,  then  s_ij = cap * tanh(s_ij / cap)          (cap 0: not capped)
//   key j is seen by query i when j <= i and
//       i - j < window                         (window 0: no window)
//       floor(i / chunk) == floor(j / chunk)   (chunk 0: no chunks; counted from position 0)
//   a_ij = exp(s_ij) / (exp(sink_h) + sum_j exp(s_ij))   sink: one learned number a head that
//                                                        has no key and no value (null: none)
//   o_i  = sum_j a_ij v_j;  then o_i * sigmoid(gate) with one gate an element or one a head
//
// Keys lie in a pool of blocks [page, kv head] of page_size rows of KW elements; values in a
// pool of their own (rows of VW elements), or (no value pool) they are the first VW columns of
// the key rows: that is what
// attention over a shared latent row looks like once the per-head key and value matrices have
// been moved to the query's and the output's side (one kv head, a key row = the latent and the
// rotated part, the value = the latent).
//
//  * project_rows: the rows of a projection, segment by segment: a bias, an RMS norm over the
//    whole segment or over every head on its own, a rotation of some leading elements of every
//    head by the token's position (angle = position * frequency in 32-bit, pairs (i, i + dims /
//    2) or neighbours (2i, 2i + 1)), then to plain rows or into the pools at slot_mapping.
//  * masked_attention: any sizes, both dtypes, all arithmetic 32-bit; one workgroup a (token,
//    kv head), one wave a query head.  A token's chunks of keys start at the first key it sees,
//    so its result never depends on how the batch was cut.
//  * head_products: out[t, h, :] = W_h a[t, h, :], a matrix a head (the products that move a
//    latent attention's per-head matrices out of the attention), 32-bit sums in ascending k,
//    with an optional gate sigmoid(g) on the output.
#include "zf_common.h"

// Where element d of row r lies in a block of page_size rows of W elements.  When W is a
// multiple of 8 the block is laid out [W / 8][page_size][8]: the 16 bytes that hold 8 elements
// of a row lie beside the same 16 bytes of the next row, so the lanes of a wave that load 16
// bytes of 16 rows each (an MFMA operand) read 256 consecutive bytes.  Else plain rows.
__host__ __device__ __forceinline__ size_t pool_at(int r, int d, int page_size, int W) {
  return (W & 7) == 0 ? ((size_t)(d >> 3) * page_size + r) * 8 + (d & 7) : (size_t)r * W + d;
}

#define PR_MAX_SEGMENTS 4

struct RowSegment {
  int src_off, width;        // columns [src_off, src_off + width) of a source row
  const float* gain;         // [width]: RMS norm over the whole segment; null: none
  const float* bias;         // [width], added to the source's values first; null: none
  int per_head;              // the norm runs over every head alone, gain [hd] for all heads
  int interleaved;           // the rotated pairs are neighbours (2i, 2i + 1), pair i by freq[i]
  float eps;
  int hd;                    // head size inside the segment (width % hd == 0)
  int rot_off, rot_dims;     // elements [rot_off, rot_off + rot_dims) of a head are rotated
  const float* freq;         // [rot_dims / 2]
  float mag;                 // cosine and sine are multiplied by this
  int skip;                  // elements of a head below this are not written
  int to_pool;               // 0: plain rows, 1: pages
  void* dst;
  long long dst_stride;      // plain rows: elements from one row to the next
  int dst_off;               // first column in the destination row (pool: in the key row)
  int dst_hd;                // width a head takes in the destination (pool: of a pool row)
  int pool_heads;            // pool: kv heads
};
struct RowSegments {
  RowSegment s[PR_MAX_SEGMENTS];
  int n;
};

#define PR_MAX_PAIRS 256      // a rotation's cosines and sines are kept in LDS: rot_dims <= 512
#define PR_MAX_HEADS 256      // a norm a head keeps the heads' factors in LDS

template <typename T>
__global__ __launch_bounds__(256) void project_rows_kernel(
    const T* __restrict__ src, long long src_stride, const int* __restrict__ positions,
    const int* __restrict__ slot_mapping, int page_size, RowSegments segs) {
#pragma clang fp contract(off)
  __shared__ float red[16];
  __shared__ float cs_t[PR_MAX_PAIRS], sn_t[PR_MAX_PAIRS];
  __shared__ float inv_h[PR_MAX_HEADS];
  const int t = blockIdx.x;
  const T* row = src + (size_t)t * src_stride;
  const float pos = (float)positions[t];
  const float* have = nullptr;          // the frequencies the tables in LDS were made from
  float have_mag = 0.f;
  for (int si = blockIdx.y; si < segs.n; si += gridDim.y) {
    const RowSegment& g = segs.s[si];
    const T* x = row + g.src_off;
    float inv = 1.f;
    if (g.gain != nullptr && !g.per_head) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < g.width; i += blockDim.x) {
        float v = load_as_float<T>(x + i);
        if (g.bias != nullptr) v = v + g.bias[i];
        ss += v * v;
      }
      ss = block_sum(ss, red);
      inv = 1.0f / sqrtf(ss / (float)g.width + g.eps);
    } else if (g.gain != nullptr) {
      // a wave a head: lanes side by side over its elements, then over the lanes
      __syncthreads();                               // the segment before is done with inv_h
      const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
      for (int head = wave; head < g.width / g.hd; head += blockDim.x / ZF_WAVE) {
        float ss = 0.f;
        for (int d = lane; d < g.hd; d += ZF_WAVE) {
          float v = load_as_float<T>(x + head * g.hd + d);
          if (g.bias != nullptr) v = v + g.bias[head * g.hd + d];
          ss += v * v;
        }
        ss = wave_sum(ss);
        if (lane == 0) inv_h[head] = 1.0f / sqrtf(ss / (float)g.hd + g.eps);
      }
      __syncthreads();
    }
    size_t pool_base = 0;
    int pool_row = 0;
    if (g.to_pool) {
      const int slot = slot_mapping[t];
      if (slot < 0) continue;                       // the same for the whole workgroup
      pool_base = (size_t)(slot / page_size) * g.pool_heads;
      pool_row = slot % page_size;
    }
    const int half = g.rot_dims / 2;
    // the token's cosine and sine a pair, once for all heads (and for the next segment, if it
    // turns by the same frequencies)
    if (half > 0 && (have != g.freq || have_mag != g.mag)) {
      __syncthreads();
      for (int j = threadIdx.x; j < half; j += blockDim.x) {
        float sn, cs;
        sincosf(pos * g.freq[j], &sn, &cs);
        cs_t[j] = cs * g.mag;
        sn_t[j] = sn * g.mag;
      }
      __syncthreads();
      have = g.freq;
      have_mag = g.mag;
    }
    for (int i = threadIdx.x; i < g.width; i += blockDim.x) {
      const int head = i / g.hd, d = i % g.hd;
      if (d < g.skip) continue;
      float a = load_as_float<T>(x + i);
      if (g.bias != nullptr) a = a + g.bias[i];
      const float inv_i = g.per_head ? inv_h[head] : inv;
      if (g.gain != nullptr) a = a * inv_i * g.gain[g.per_head ? d : i];
      const int r = d - g.rot_off;
      if (r >= 0 && r < g.rot_dims) {
        const bool first = g.interleaved ? (r & 1) == 0 : r < half;
        const int step = g.interleaved ? 1 : half;
        const int pi = first ? i + step : i - step;
        float b = load_as_float<T>(x + pi);
        if (g.bias != nullptr) b = b + g.bias[pi];
        if (g.gain != nullptr) b = b * inv_i * g.gain[g.per_head ? pi - head * g.hd : pi];
        const int j = g.interleaved ? r >> 1 : (first ? r : r - half);
        const float cs = cs_t[j], sn = sn_t[j];
        a = first ? a * cs - b * sn : a * cs + b * sn;
      }
      if (g.to_pool) {
        T* o = (T*)g.dst + (pool_base + head) * page_size * (size_t)g.dst_hd
               + pool_at(pool_row, g.dst_off + (d - g.skip), page_size, g.dst_hd);
        store_from_float<T>(o, a);
      } else {
        T* o = (T*)g.dst + (size_t)t * g.dst_stride + g.dst_off + (size_t)head * g.dst_hd
               + (d - g.skip);
        store_from_float<T>(o, a);
      }
    }
  }
}

// The same for bfloat16 rows whose segments are made of whole groups of 8 elements (head
// sizes, rotated ranges and their halves, offsets and strides all multiples of 8): a thread
// takes 8 consecutive elements, 16 bytes in and 16 bytes out (a pool's 8 elements of a row are
// consecutive).  The same arithmetic as the kernel above (the norm's partial sums are added in
// another order).
__device__ __forceinline__ void pr_unpack8(const uint4& v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __uint_as_float(w[i] << 16);
    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}

// 8 elements of a row from column i on, with the bias (if any) added
__device__ __forceinline__ void pr_load8(const bf16_t* x, const float* bias, int i, float (&f)[8]) {
#pragma clang fp contract(off)
  pr_unpack8(*(const uint4*)(x + i), f);
  if (bias != nullptr) {
    const float4 b0 = *(const float4*)(bias + i), b1 = *(const float4*)(bias + i + 4);
    const float bb[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = f[e] + bb[e];
  }
}

__global__ __launch_bounds__(256) void project_rows_vec8_kernel(
    const bf16_t* __restrict__ src, long long src_stride, const int* __restrict__ positions,
    const int* __restrict__ slot_mapping, int page_size, RowSegments segs) {
#pragma clang fp contract(off)
  __shared__ float red[16];
  __shared__ float cs_t[PR_MAX_PAIRS], sn_t[PR_MAX_PAIRS];
  __shared__ float inv_h[PR_MAX_HEADS];
  const int t = blockIdx.x;
  const bf16_t* row = src + (size_t)t * src_stride;
  const float pos = (float)positions[t];
  const float* have = nullptr;
  float have_mag = 0.f;
  for (int si = blockIdx.y; si < segs.n; si += gridDim.y) {
    const RowSegment& g = segs.s[si];
    const bf16_t* x = row + g.src_off;
    const int n8 = g.width / 8;
    float inv = 1.f;
    if (g.gain != nullptr && !g.per_head) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < n8; c += blockDim.x) {
        float f[8];
        pr_load8(x, g.bias, 8 * c, f);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
      }
      ss = block_sum(ss, red);
      inv = 1.0f / sqrtf(ss / (float)g.width + g.eps);
    } else if (g.gain != nullptr) {
      __syncthreads();
      const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
      for (int head = wave; head < g.width / g.hd; head += blockDim.x / ZF_WAVE) {
        float ss = 0.f;
        for (int c = lane; c < g.hd / 8; c += ZF_WAVE) {
          float f[8];
          pr_load8(x, g.bias, head * g.hd + 8 * c, f);
#pragma unroll
          for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
        }
        ss = wave_sum(ss);
        if (lane == 0) inv_h[head] = 1.0f / sqrtf(ss / (float)g.hd + g.eps);
      }
      __syncthreads();
    }
    size_t pool_base = 0;
    int pool_row = 0;
    if (g.to_pool) {
      const int slot = slot_mapping[t];
      if (slot < 0) continue;
      pool_base = (size_t)(slot / page_size) * g.pool_heads;
      pool_row = slot % page_size;
    }
    const int half = g.rot_dims / 2;
    if (half > 0 && (have != g.freq || have_mag != g.mag)) {
      __syncthreads();
      for (int j = threadIdx.x; j < half; j += blockDim.x) {
        float sn, cs;
        sincosf(pos * g.freq[j], &sn, &cs);
        cs_t[j] = cs * g.mag;
        sn_t[j] = sn * g.mag;
      }
      __syncthreads();
      have = g.freq;
      have_mag = g.mag;
    }
    for (int c = threadIdx.x; c < n8; c += blockDim.x) {
      const int i = 8 * c;
      const int head = i / g.hd, d = i % g.hd;
      if (d < g.skip) continue;
      float a[8];
      pr_load8(x, g.bias, i, a);
      const float inv_i = g.per_head ? inv_h[head] : inv;
      if (g.gain != nullptr) {
        const int gi = g.per_head ? d : i;
        const float4 g0 = *(const float4*)(g.gain + gi), g1 = *(const float4*)(g.gain + gi + 4);
        const float gg[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = a[e] * inv_i * gg[e];
      }
      const int r = d - g.rot_off;
      if (r >= 0 && r < g.rot_dims && g.interleaved) {
        // the partner of an element is its neighbour, among the same 8
        float n[8];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const float cs = cs_t[(r + e) >> 1], sn = sn_t[(r + e) >> 1];
          n[e] = a[e] * cs - a[e + 1] * sn;
          n[e + 1] = a[e + 1] * cs + a[e] * sn;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = n[e];
      } else if (r >= 0 && r < g.rot_dims) {
        const bool first = r < half;
        const int pi = first ? i + half : i - half;
        float b[8];
        pr_load8(x, g.bias, pi, b);
        if (g.gain != nullptr) {
          const int gi = g.per_head ? pi - head * g.hd : pi;
          const float4 g0 = *(const float4*)(g.gain + gi), g1 = *(const float4*)(g.gain + gi + 4);
          const float gg[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) b[e] = b[e] * inv_i * gg[e];
        }
        const int j = first ? r : r - half;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float cs = cs_t[j + e], sn = sn_t[j + e];
          a[e] = first ? a[e] * cs - b[e] * sn : a[e] * cs + b[e] * sn;
        }
      }
      bf16_t* o;
      if (g.to_pool)
        o = (bf16_t*)g.dst + (pool_base + head) * page_size * (size_t)g.dst_hd
            + pool_at(pool_row, g.dst_off + (d - g.skip), page_size, g.dst_hd);
      else
        o = (bf16_t*)g.dst + (size_t)t * g.dst_stride + g.dst_off + (size_t)head * g.dst_hd
            + (d - g.skip);
      *(uint4*)o = make_uint4(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]),
                              pack_bf16x2(a[4], a[5]), pack_bf16x2(a[6], a[7]));
    }
  }
}

// ints: 11 a segment (src_off, width, hd, rot_off, rot_dims, skip, to_pool, dst_off, dst_hd,
// pool_heads, flags: 1 = a norm a head, 2 = neighbouring pairs); floats: 2 a segment (eps, mag);
// ptrs: 4 a segment (gain, freq, dst, bias); strides: 1 a segment
extern "C" int zf_project_rows(const void* src, int dtype, long long src_stride,
                               const int* positions, const int* slot_mapping, int T,
                               int page_size, int n_segs, const int* ints, const float* floats,
                               void* const* ptrs, const long long* strides, hipStream_t stream) {
  if (T <= 0 || n_segs <= 0) return 0;
  if (n_segs > PR_MAX_SEGMENTS) return -2;
  RowSegments segs;
  segs.n = n_segs;
  for (int i = 0; i < n_segs; ++i) {
    RowSegment& g = segs.s[i];
    const int* v = ints + 11 * i;
    g.src_off = v[0]; g.width = v[1]; g.hd = v[2]; g.rot_off = v[3]; g.rot_dims = v[4];
    g.skip = v[5]; g.to_pool = v[6]; g.dst_off = v[7]; g.dst_hd = v[8]; g.pool_heads = v[9];
    g.eps = floats[2 * i]; g.mag = floats[2 * i + 1];
    g.per_head = v[10] & 1; g.interleaved = (v[10] >> 1) & 1;
    g.gain = (const float*)ptrs[4 * i]; g.freq = (const float*)ptrs[4 * i + 1];
    g.dst = ptrs[4 * i + 2]; g.bias = (const float*)ptrs[4 * i + 3];
    g.dst_stride = strides[i];
    if (g.per_head && g.gain != nullptr && g.hd > 0 && g.width / g.hd > PR_MAX_HEADS) return -2;
    if (g.width <= 0 || g.hd <= 0 || g.width % g.hd != 0 || g.rot_dims < 0 || g.rot_dims % 2 != 0
        || g.rot_off < 0 || g.rot_off + g.rot_dims > g.hd || g.skip < 0 || g.skip >= g.hd
        || (g.rot_dims > 0 && g.freq == nullptr) || g.rot_dims > 2 * PR_MAX_PAIRS
        || g.dst == nullptr
        || (g.to_pool && (slot_mapping == nullptr || page_size <= 0 || g.pool_heads <= 0)))
      return -2;
  }
  bool vec8 = dtype == ZF_BF16 && src_stride % 8 == 0 && (uintptr_t)src % 16 == 0;
  for (int i = 0; i < n_segs && vec8; ++i) {
    const RowSegment& g = segs.s[i];
    vec8 = g.src_off % 8 == 0 && g.hd % 8 == 0 && g.rot_off % 8 == 0
        && g.rot_dims % (g.interleaved ? 8 : 16) == 0
        && (g.bias == nullptr || (uintptr_t)g.bias % 16 == 0)
        && g.skip % 8 == 0 && g.dst_off % 8 == 0 && g.dst_hd % 8 == 0 && (uintptr_t)g.dst % 16 == 0
        && (g.to_pool || g.dst_stride % 8 == 0) && (g.gain == nullptr || (uintptr_t)g.gain % 16 == 0);
  }
  if (vec8) {
    hipLaunchKernelGGL(project_rows_vec8_kernel, dim3(T, n_segs), dim3(256), 0, stream,
                       (const bf16_t*)src, src_stride, positions, slot_mapping, page_size, segs);
    ZF_CHECK_LAUNCH();
  }
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(project_rows_kernel<float>, dim3(T, n_segs), dim3(256), 0, stream,
                       (const float*)src, src_stride, positions, slot_mapping, page_size, segs);
  else
    hipLaunchKernelGGL(project_rows_kernel<bf16_t>, dim3(T, n_segs), dim3(256), 0, stream,
                       (const bf16_t*)src, src_stride, positions, slot_mapping, page_size, segs);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  masked_attention: the 32-bit kernel for every size
// =====================================================================================
#define MA_MAX_WAVES 16
#define MA_GATE_NONE 0
#define MA_GATE_ELEMENT 1
#define MA_GATE_HEAD 2

struct MaskedAttentionArgs {
  long long q_stride, gate_stride;
  float scale, cap;
  int window, chunk, gate_mode;
  int nH, nKV, KW, VW, page_size, max_pages, KC;
};

template <typename T>
__global__ __launch_bounds__(MA_MAX_WAVES * ZF_WAVE) void masked_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ gate, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const float* __restrict__ sink,
    const int* __restrict__ block_table, const int* __restrict__ q_start,
    const int* __restrict__ ctx_len, const int* __restrict__ seq_index, T* __restrict__ out,
    MaskedAttentionArgs a) {
  extern __shared__ float smem[];
  const int KC = a.KC, KW = a.KW, VW = a.VW;
  const int ldk = KW + 1;                          // odd row stride: a lane a key, no conflicts
  const int ldv = VW + 1;
  const int n_waves = blockDim.x / ZF_WAVE;
  float* ks = smem;                                // [KC][ldk]
  float* vs = ks + KC * ldk;                       // [KC][ldv] when the values have a pool
  float* qs = vs + (v_pool != nullptr ? KC * ldv : 0);   // [n_waves][KW]
  float* ps = qs + n_waves * KW;                   // [n_waves][ZF_WAVE]
  int* rows = (int*)(ps + n_waves * ZF_WAVE);      // [KC]: block of each key in the pools

  const int t = blockIdx.x, kvh = blockIdx.y;
  const int G = a.nH / a.nKV;
  const int wave = threadIdx.x / ZF_WAVE, lane = threadIdx.x % ZF_WAVE;
  const int g = blockIdx.z * n_waves + wave;       // this wave's head within the group
  const bool live = g < G;
  const int h = kvh * G + (live ? g : 0);
  const int s = seq_index[t];
  const int q_len = q_start[s + 1] - q_start[s];
  const int pos = ctx_len[s] - q_len + (t - q_start[s]);
  int lo = 0;
  if (a.window > 0 && pos - a.window + 1 > lo) lo = pos - a.window + 1;
  if (a.chunk > 0 && pos / a.chunk * a.chunk > lo) lo = pos / a.chunk * a.chunk;
  const int* table = block_table + (size_t)s * a.max_pages;

  const T* qrow = q + (size_t)t * a.q_stride + (size_t)h * KW;
  float* qw = qs + wave * KW;
  for (int i = lane; i < KW; i += ZF_WAVE) qw[i] = load_as_float<T>(qrow + i);

  // a lane owns the output elements d = lane, lane + 64, ... (up to 8: VW <= 512)
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // the sink is a key of score sink_h that is there before the first real one
  float m = -INFINITY, l = 0.f;
  if (sink != nullptr) {
    m = sink[h];
    l = 1.f;
  }
  const float* vsrc = v_pool != nullptr ? vs : ks;
  const int ldvs = v_pool != nullptr ? ldv : ldk;

  for (int base = lo; base <= pos; base += KC) {
    const int nk = min(KC, pos - base + 1);
    __syncthreads();                               // the tiles of the chunk before are done with
    if ((int)threadIdx.x < KC) {
      const int key = base + threadIdx.x;
      rows[threadIdx.x] = key <= pos ? table[key / a.page_size] * a.nKV + kvh : -1;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nk * KW; i += blockDim.x) {
      const int j = i / KW, d = i % KW;
      ks[j * ldk + d] = load_as_float<T>(k_pool + (size_t)rows[j] * a.page_size * KW
                                         + pool_at((base + j) % a.page_size, d, a.page_size, KW));
    }
    if (v_pool != nullptr)
      for (int i = threadIdx.x; i < nk * VW; i += blockDim.x) {
        const int j = i / VW, d = i % VW;
        vs[j * ldv + d] = load_as_float<T>(v_pool + (size_t)rows[j] * a.page_size * VW
                                           + pool_at((base + j) % a.page_size, d, a.page_size, VW));
      }
    __syncthreads();
    float sc = -INFINITY;
    if (lane < nk) {
      const float* kr = ks + lane * ldk;
      float dot = 0.f;
      for (int d = 0; d < KW; ++d) dot = fmaf(qw[d], kr[d], dot);
      sc = dot * a.scale;
      if (a.cap > 0.f) sc = a.cap * tanhf(sc / a.cap);
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float corr = expf(m - m_new);            // exp(-inf) = 0 on a first chunk without sink
    const float p = lane < nk ? expf(sc - m_new) : 0.f;
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[wave * ZF_WAVE + lane] = p;                 // read back by this wave only
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] *= corr;
    const float* pw = ps + wave * ZF_WAVE;
    for (int j = 0; j < nk; ++j) {
      const float pj = pw[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int d = lane + i * ZF_WAVE;
        if (d < VW) acc[i] = fmaf(pj, vsrc[j * ldvs + d], acc[i]);
      }
    }
  }
  if (!live) return;
  const float inv = 1.0f / l;
  T* orow = out + ((size_t)t * a.nH + h) * VW;
  float head_gate = 1.f;
  if (a.gate_mode == MA_GATE_HEAD)
    head_gate = 1.0f / (1.0f + expf(-load_as_float<T>(gate + (size_t)t * a.gate_stride + h)));
  const T* grow = a.gate_mode == MA_GATE_ELEMENT
      ? gate + (size_t)t * a.gate_stride + (size_t)h * VW : nullptr;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + i * ZF_WAVE;
    if (d < VW) {
      float v = acc[i] * inv * head_gate;
      if (grow != nullptr) v *= 1.0f / (1.0f + expf(-load_as_float<T>(grow + d)));
      store_from_float<T>(orow + d, v);
    }
  }
}

// floats a key of a chunk takes in LDS, and the chunk that fits 60 KB beside the queries
static int ma_chunk_keys(int KW, int VW, bool v_pool, int n_waves) {
  const long per_key = (KW + 1) + (v_pool ? VW + 1 : 0) + 1;
  const long fixed = (long)n_waves * (KW + ZF_WAVE);
  long kc = (60 * 1024 / 4 - fixed) / per_key;
  if (kc > ZF_WAVE) kc = ZF_WAVE;
  return (int)kc;
}

extern "C" int zf_masked_attention(const void* q, long long q_stride, const void* gate,
                                   long long gate_stride, int gate_mode, const void* k_pool,
                                   const void* v_pool, int dtype, const float* sink,
                                   const int* block_table, const int* q_start,
                                   const int* ctx_len, const int* seq_index, void* out,
                                   float scale, float cap, int window, int chunk, int T, int nH,
                                   int nKV, int KW, int VW, int page_size, int max_pages,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (KW <= 0 || VW <= 0 || VW > 512 || nKV <= 0 || nH % nKV != 0 || page_size <= 0
      || (v_pool == nullptr && VW > KW) || (gate_mode != MA_GATE_NONE && gate == nullptr)
      || gate_mode < 0 || gate_mode > 2 || window < 0 || chunk < 0 || cap < 0.f)
    return -2;
  const int G = nH / nKV;
  // a wave a head, up to 16; fewer where wide rows would leave no room for a chunk of keys
  int n_waves = G < MA_MAX_WAVES ? G : MA_MAX_WAVES;
  while (n_waves > 1 && ma_chunk_keys(KW, VW, v_pool != nullptr, n_waves) < 16) n_waves = (n_waves + 1) / 2;
  const int KC = ma_chunk_keys(KW, VW, v_pool != nullptr, n_waves);
  if (KC < 4) return -3;
  MaskedAttentionArgs a;
  a.q_stride = q_stride; a.gate_stride = gate_stride; a.scale = scale; a.cap = cap;
  a.window = window; a.chunk = chunk; a.gate_mode = gate_mode; a.nH = nH; a.nKV = nKV;
  a.KW = KW; a.VW = VW; a.page_size = page_size; a.max_pages = max_pages; a.KC = KC;
  dim3 grid(T, nKV, (G + n_waves - 1) / n_waves);
  const size_t smem = ((size_t)KC * (KW + 1) + (v_pool != nullptr ? (size_t)KC * (VW + 1) : 0)
                       + (size_t)n_waves * (KW + ZF_WAVE) + KC) * sizeof(float);
  if (dtype == ZF_F32)
    hipLaunchKernelGGL(masked_attention_kernel<float>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const float*)q, (const float*)gate, (const float*)k_pool,
                       (const float*)v_pool, sink, block_table, q_start, ctx_len, seq_index,
                       (float*)out, a);
  else
    hipLaunchKernelGGL(masked_attention_kernel<bf16_t>, grid, dim3(n_waves * ZF_WAVE), smem,
                       stream, (const bf16_t*)q, (const bf16_t*)gate, (const bf16_t*)k_pool,
                       (const bf16_t*)v_pool, sink, block_table, q_start, ctx_len, seq_index,
                       (bf16_t*)out, a);
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  head_products: a matrix a head
// =====================================================================================
// out[t, h, n] = sum_k a[t, h, k] * w[h, n, k]  (n < N, k < K), then times sigmoid(gate[t, h, n])
// if a gate is given.  a: row t at a + t * a_stride, head h at + a_off + h * a_hd; out: row t at
// out + t * out_stride, head h at + out_off + h * out_hd; w [H, N, K]; gate [T, H * N] rows of
// stride gate_stride.  A workgroup takes 16 tokens x 64 outputs of one head; k runs upwards in
// one accumulator an output, so a token's result does not depend on the tokens beside it.
#define HP_TOK 16
#define HP_OUT 64
#define HP_K 64

template <typename T, typename TW>
__global__ __launch_bounds__(256) void head_products_kernel(
    const T* __restrict__ a, long long a_stride, int a_off, int a_hd, const TW* __restrict__ w,
    const T* __restrict__ gate, long long gate_stride, T* __restrict__ out, long long out_stride,
    int out_off, int out_hd, int n_tok, int N, int K) {
  __shared__ float as[HP_TOK][HP_K + 1];
  __shared__ float ws[HP_OUT][HP_K + 1];
  const int t0 = blockIdx.x * HP_TOK, h = blockIdx.y, n0 = blockIdx.z * HP_OUT;
  const int nl = threadIdx.x % HP_OUT, tg = threadIdx.x / HP_OUT;    // 4 groups of 4 tokens
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  const TW* wh = w + (size_t)h * N * K;
  for (int k0 = 0; k0 < K; k0 += HP_K) {
    const int kn = min(HP_K, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < HP_TOK * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      float v = 0.f;
      if (t0 + r < n_tok && c < kn)
        v = load_as_float<T>(a + (size_t)(t0 + r) * a_stride + a_off + (size_t)h * a_hd + k0 + c);
      as[r][c] = v;
    }
    for (int i = threadIdx.x; i < HP_OUT * HP_K; i += 256) {
      const int r = i / HP_K, c = i % HP_K;
      float v = 0.f;
      if (n0 + r < N && c < kn) v = load_as_float<TW>(wh + (size_t)(n0 + r) * K + k0 + c);
      ws[r][c] = v;
    }
    __syncthreads();
    for (int c = 0; c < kn; ++c) {
      const float wv = ws[nl][c];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = fmaf(as[tg * 4 + i][c], wv, acc[i]);
    }
  }
  const int n = n0 + nl;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + tg * 4 + i;
    if (t >= n_tok) continue;
    float v = acc[i];
    if (gate != nullptr)
      v *= 1.0f / (1.0f + expf(-load_as_float<T>(gate + (size_t)t * gate_stride
                                                  + (size_t)h * N + n)));
    store_from_float<T>(out + (size_t)t * out_stride + out_off + (size_t)h * out_hd + n, v);
  }
}

// The same in MFMA tiles for bfloat16 operands (K a multiple of 16, rows aligned to 16 bytes):
// a wave takes 32 outputs x 32 tokens of one head, D = W_h tile (32 x K) times a^T (K x 32), both
// operands straight from memory into v_mfma_f32_32x32x16_bf16, k upwards in one accumulator; a
// lane ends with four runs of four consecutive outputs of one token.  The four waves of a
// workgroup take four tiles of outputs.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hp_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float hp_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t hp_u32x4_t;

__global__ __launch_bounds__(256) void head_products_mfma_kernel(
    const bf16_t* __restrict__ a, long long a_stride, int a_off, int a_hd,
    const bf16_t* __restrict__ w, const bf16_t* __restrict__ gate, long long gate_stride,
    bf16_t* __restrict__ out, long long out_stride, int out_off, int out_hd, int n_tok, int N,
    int K) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int c = lane % 32, hl = lane / 32;
  const int t0 = blockIdx.x * 32, h = blockIdx.y, n0 = (blockIdx.z * 4 + wave) * 32;
  if (n0 >= N) return;
  const int t = t0 + c, n = n0 + c;
  const bool t_ok = t < n_tok, n_ok = n < N;
  const bf16_t* arow = a + (size_t)(t_ok ? t : 0) * a_stride + a_off + (size_t)h * a_hd;
  const bf16_t* wrow = w + ((size_t)h * N + (n_ok ? n : 0)) * K;
  hp_f32x16_t acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  // four k-steps' operands are asked for before the first of their products
  for (int k0 = 0; k0 < K; k0 += 64) {
    hp_u32x4_t av[4], wv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      av[u] = hp_u32x4_t{0u, 0u, 0u, 0u};
      wv[u] = hp_u32x4_t{0u, 0u, 0u, 0u};
      const int k = k0 + 16 * u + 8 * hl;
      if (k < K) {
        if (t_ok) av[u] = *(const hp_u32x4_t*)(arow + k);
        if (n_ok) wv[u] = *(const hp_u32x4_t*)(wrow + k);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (k0 + 16 * u < K)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const hp_bf16x8_t*)&wv[u],
                                                      *(const hp_bf16x8_t*)&av[u], acc, 0, 0, 0);
  }
  if (!t_ok) return;
  // acc[r] is output n0 + 8 (r / 4) + 4 hl + r % 4 of token t
  bf16_t* orow = out + (size_t)t * out_stride + out_off + (size_t)h * out_hd;
  const bf16_t* grow = gate != nullptr ? gate + (size_t)t * gate_stride + (size_t)h * N : nullptr;
  // runs of four outputs as one 8-byte store where the rows allow it
  const bool wide = (N & 3) == 0 && (((size_t)t * out_stride + out_off + (size_t)h * out_hd) & 3) == 0
      && ((uintptr_t)out & 7) == 0;
#pragma unroll
  for (int r4 = 0; r4 < 4; ++r4) {
    const int o = n0 + 8 * r4 + 4 * hl;
    float v[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      v[x] = acc[4 * r4 + x];
      if (grow != nullptr && o + x < N) v[x] *= 1.0f / (1.0f + expf(-bf16_to_float(grow[o + x])));
    }
    if (wide && o < N) {
      *(uint2*)(orow + o) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
    } else {
#pragma unroll
      for (int x = 0; x < 4; ++x)
        if (o + x < N) orow[o + x] = float_to_bf16(v[x]);
    }
  }
}

extern "C" int zf_head_products(const void* a, int dtype, long long a_stride, int a_off, int a_hd,
                                const void* w, int w_dtype, const void* gate,
                                long long gate_stride, void* out, long long out_stride,
                                int out_off, int out_hd, int T, int H, int N, int K,
                                hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || N <= 0 || K <= 0 || a_hd < K || out_hd < N) return -2;
  if (dtype == ZF_BF16 && w_dtype == ZF_BF16 && K % 16 == 0 && a_stride % 8 == 0 && a_off % 8 == 0
      && a_hd % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0) {
    dim3 mgrid((T + 31) / 32, H, (N + 127) / 128);
    hipLaunchKernelGGL(head_products_mfma_kernel, mgrid, dim3(256), 0, stream, (const bf16_t*)a,
                       a_stride, a_off, a_hd, (const bf16_t*)w, (const bf16_t*)gate, gate_stride,
                       (bf16_t*)out, out_stride, out_off, out_hd, T, N, K);
    ZF_CHECK_LAUNCH();
  }
  dim3 grid((T + HP_TOK - 1) / HP_TOK, H, (N + HP_OUT - 1) / HP_OUT);
#define HP_LAUNCH(TA, TWT)                                                                      \
  hipLaunchKernelGGL((head_products_kernel<TA, TWT>), grid, dim3(256), 0, stream, (const TA*)a, \
                     a_stride, a_off, a_hd, (const TWT*)w, (const TA*)gate, gate_stride,        \
                     (TA*)out, out_stride, out_off, out_hd, T, N, K)
  if (dtype == ZF_F32 && w_dtype == ZF_F32) HP_LAUNCH(float, float);
  else if (dtype == ZF_F32) HP_LAUNCH(float, bf16_t);
  else if (w_dtype == ZF_F32) HP_LAUNCH(bf16_t, float);
  else HP_LAUNCH(bf16_t, bf16_t);
#undef HP_LAUNCH
  ZF_CHECK_LAUNCH();
}

// =====================================================================================
//  bfloat16 MFMA kernels: waves on their own
// =====================================================================================
// The same attention in v_mfma_f32_32x32x16_bf16 tiles, for key rows of KD and value rows of VD
// elements (KD a multiple of 16, VD of 32; the pools in the [W / 8][page_size][8] form of
// pool_at) and at most 32 query heads a kv head.  A wave takes
// 32 rows, (position, head of the group) pairs of one sequence, and walks the keys those rows
// see in chunks of 32, on its own: no barrier between waves anywhere.  A lane loads, for its
// key of the chunk, the 8 values that its operand of S^T = K Q^T needs straight from the pool
// (every value of the chunk once in the wave), and the 8 values of that key's value row
// (TIED: of the key row's leading columns) that it writes transposed (permuted against bank
// conflicts) into the wave's own LDS tile for O^T = V^T P^T.  The score tile is transposed so
// that a lane's 16 scores belong to one row: cap, mask and soft-max run in registers in 32-bit
// (base-2 exponentials, the scale folded in; with a sink the running maximum starts at the
// sink and the sum at 1).  Each weight enters the second product as the sum of two bfloat16
// numbers (its rounding and the rounding of what that leaves).  The next chunk's keys are asked
// for as soon as this chunk's score products are issued, its values once this chunk's are in
// the tile.
//   DECODE: grid (sequence, kv head, block); one token a sequence, its G heads the first G rows;
//   the four waves of a workgroup are four splits of the context, wave_keys keys each.
//   else: grid (tile of 128 / G positions, kv head, part); with several parts a wave takes that
//   part of its keys.  Splits and parts leave un-normalised partials (maximum, sum, O) that
//   masked_attention_merge_kernel combines in split order; the sink belongs to the first.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 mw_bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mw_f32x16_t;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t mw_u32x4_t;

#define MW_ROWS 128
#define MW_KEYS 32
#define MW_LOG2E 1.4426950408889634f

__device__ __forceinline__ float mw_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// where key j of value element d lies in the [d][key] tile
__device__ __forceinline__ int mw_swz(int j, int d) { return (((j >> 2) ^ ((d >> 3) & 7)) << 2) | (j & 3); }
// tanh through one exponential: 1 - 2 / (e^(2x) + 1); +-1 where the exponential leaves the range
__device__ __forceinline__ float mw_tanh(float x) {
  const float e = mw_exp2(x * (2.0f * MW_LOG2E));
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

struct MaskedWaveArgs {
  long long q_stride, gate_stride;
  float scale, cap;
  int window, chunk, gate_mode;
  int n_seqs, nH, nKV, page_size, max_pages, QT, wave_keys;
};

template <int KD, int VD, bool TIED, bool DECODE>
__global__ __launch_bounds__(256, 2) void masked_attention_wave_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ gate,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    const float* __restrict__ sink, const int* __restrict__ block_table,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, bf16_t* __restrict__ out,
    float* __restrict__ ws_o, float* __restrict__ ws_ml, MaskedWaveArgs a) {
  constexpr int LDT = MW_KEYS + 4;
  __shared__ __attribute__((aligned(16))) bf16_t vt_all[4 * VD * LDT];
  const int kvh = blockIdx.y;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int c = lane % 32, hl = lane / 32;
  bf16_t* vt = vt_all + wave * VD * LDT;
  const int G = a.nH / a.nKV;
  const int window = a.window, chunk = a.chunk, page_size = a.page_size, nKV = a.nKV;

  // the first key position p sees
  auto first_seen = [&](int p) {
    int lo = 0;
    if (window > 0 && p - window + 1 > lo) lo = p - window + 1;
    if (chunk > 0 && p / chunk * chunk > lo) lo = p / chunk * chunk;
    return lo;
  };

  int s, tok, pos_r, lo_r, h, split = 0, n_splits = 1;
  int k_first, k_end;          // the keys the wave walks: [k_first down to a multiple of 32, k_end)
  bool row_ok;
  if constexpr (DECODE) {
    s = blockIdx.x;
    split = blockIdx.z * 4 + wave;
    n_splits = gridDim.z * 4;
    row_ok = c < G;
    h = kvh * G + (row_ok ? c : 0);
    tok = s;
    pos_r = ctx_len[s] - 1;
    lo_r = first_seen(pos_r);
    k_first = lo_r;
    k_end = pos_r + 1;
  } else {
    split = blockIdx.z;
    n_splits = gridDim.z;
    // the last tiles of a sequence walk the most keys: they are handed out first, so that the
    // grid does not end on its longest workgroups
    s = 0;
    int tile = (int)gridDim.x - 1 - (int)blockIdx.x;
    for (; s < a.n_seqs; ++s) {
      const int n = (q_start[s + 1] - q_start[s] + a.QT - 1) / a.QT;
      if (tile < n) break;
      tile -= n;
    }
    if (s >= a.n_seqs) return;
    const int q_len = q_start[s + 1] - q_start[s];
    const int first = tile * a.QT;
    const int npos = min(a.QT, q_len - first);
    const int nrows = npos * G;
    if (wave * 32 >= nrows) return;                // (no barrier follows: waves are on their own)
    const int pos0 = ctx_len[s] - q_len + first;
    const int row = wave * 32 + c;
    row_ok = row < nrows;
    const int qi = row_ok ? row / G : 0;
    h = kvh * G + (row_ok ? row % G : 0);
    tok = q_start[s] + first + qi;
    pos_r = pos0 + qi;
    lo_r = first_seen(pos_r);
    const int p_lo = pos0 + (wave * 32) / G;                       // the wave's first position
    const int p_hi = pos0 + (min(nrows, wave * 32 + 32) - 1) / G;  // and its last
    k_first = first_seen(p_lo);        // (the first key a position sees never moves back)
    k_end = p_hi + 1;
  }
  const int* table = block_table + (size_t)s * a.max_pages;

  mw_bf16x8_t qf[KD / 16];
  {
    const bf16_t* qrow = q + (size_t)tok * a.q_stride + (size_t)h * KD;
#pragma unroll
    for (int i = 0; i < KD / 16; ++i) {
      mw_u32x4_t v = {0u, 0u, 0u, 0u};
      if (row_ok) v = *(const mw_u32x4_t*)(qrow + 16 * i + 8 * hl);
      qf[i] = *(const mw_bf16x8_t*)&v;
    }
  }
  mw_f32x16_t acc[VD / 32];
#pragma unroll
  for (int i = 0; i < VD / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  // scores are kept times log2(e), so that every weight is one v_exp_f32
  const float scale_log2 = a.scale * MW_LOG2E;
  const float cap_log2 = a.cap * MW_LOG2E;
  const float inv_cap = a.cap > 0.f ? a.scale / a.cap : 0.f;
  const bool capped = a.cap > 0.f;
  const bool has_sink = sink != nullptr && split == 0;
  float m = -INFINITY, l = 0.f;
  if (has_sink) {
    m = sink[h] * MW_LOG2E;
    l = 1.f;
  }

  int k_begin = k_first / MW_KEYS * MW_KEYS;
  if constexpr (DECODE) {
    k_begin += split * a.wave_keys;
    k_end = min(k_end, k_begin + a.wave_keys);
  } else if (n_splits > 1) {
    const int share = (k_end - k_begin + n_splits * MW_KEYS - 1) / (n_splits * MW_KEYS) * MW_KEYS;
    k_begin += split * share;
    k_end = min(k_end, k_begin + share);
  }

  // this lane's key of a chunk: key base + c; of its key row the values 16 i + 8 hl .. + 8 for
  // every i, of its value row the same
  mw_u32x4_t kf[KD / 16];
  mw_u32x4_t vf[TIED ? 1 : VD / 16];
  // the block [page, kv head] of this lane's key, in rows: its row there is key % page_size
  auto row_of = [&](int base, bool& ok) {
    const int key = base + c;
    ok = key >= k_first && key < k_end;          // (pages before k_first may have gone back)
    size_t prow = 0;
    if (ok) prow = ((size_t)table[key / page_size] * nKV + kvh) * page_size;
    return prow;
  };
  auto fetch_k = [&](int base) {
    bool ok;
    const size_t prow = row_of(base, ok);
    const int r = (base + c) % page_size;
#pragma unroll
    for (int i = 0; i < KD / 16; ++i) {
      mw_u32x4_t v = {0u, 0u, 0u, 0u};
      if (ok) v = *(const mw_u32x4_t*)(k_pool + prow * KD + ((size_t)(2 * i + hl) * page_size + r) * 8);
      kf[i] = v;
    }
  };
  auto fetch_v = [&](int base) {
    if constexpr (!TIED) {
      bool ok;
      const size_t prow = row_of(base, ok);
      const int r = (base + c) % page_size;
#pragma unroll
      for (int i = 0; i < VD / 16; ++i) {
        mw_u32x4_t v = {0u, 0u, 0u, 0u};
        if (ok) v = *(const mw_u32x4_t*)(v_pool + prow * VD + ((size_t)(2 * i + hl) * page_size + r) * 8);
        vf[i] = v;
      }
    }
  };
  if (k_begin < k_end) {
    fetch_k(k_begin);
    fetch_v(k_begin);
  }
  for (int base = k_begin; base < k_end; base += MW_KEYS) {
    const bool more = base + MW_KEYS < k_end;
    mw_f32x16_t sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.f;
#pragma unroll
    for (int i = 0; i < KD / 16; ++i)
      sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const mw_bf16x8_t*)&kf[i], qf[i], sc, 0, 0, 0);
    // the chunk's values transposed into the wave's tile
#pragma unroll
    for (int i = 0; i < VD / 16; ++i) {
      const bf16_t* e = TIED ? (const bf16_t*)&kf[i] : (const bf16_t*)&vf[TIED ? 0 : i];
#pragma unroll
      for (int x = 0; x < 8; ++x)
        vt[(16 * i + 8 * hl + x) * LDT + mw_swz(c, 16 * i + 8 * hl)] = e[x];
    }
    if (more) {                                     // in flight while this chunk runs
      fetch_k(base + MW_KEYS);
      fetch_v(base + MW_KEYS);
    }
    float cmax = -INFINITY;
    if (capped) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] = cap_log2 * mw_tanh(sc[r] * inv_cap);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) sc[r] *= scale_log2;
    }
    // a chunk that every row of the wave sees whole needs no mask
    const bool whole = row_ok && base >= lo_r && base + MW_KEYS - 1 <= pos_r &&
                       base >= k_first && base + MW_KEYS <= k_end;
    if (__all(whole)) {
#pragma unroll
      for (int r = 0; r < 16; ++r) cmax = fmaxf(cmax, sc[r]);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int key = base + 8 * (r / 4) + 4 * hl + r % 4;
        const bool seen = row_ok && key >= lo_r && key <= pos_r && key >= k_first && key < k_end;
        sc[r] = seen ? sc[r] : -INFINITY;
        cmax = fmaxf(cmax, sc[r]);
      }
    }
    cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
    const float m_new = fmaxf(m, cmax);
    // nothing seen yet (and no sink): every weight below is exp(-inf) = 0
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = mw_exp2(m - m_use);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      sc[r] = mw_exp2(sc[r] - m_use);
      psum += sc[r];
    }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = m_new;
    if (__any(corr != 1.0f)) {                     // (the maximum of some row moved)
#pragma unroll
      for (int i = 0; i < VD / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] *= corr;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();               // the wave's transposed tile is written
    // O^T += V^T P^T over the chunk's two groups of 16 keys; the registers 8 t .. 8 t + 7 hold
    // the weights of the keys 16 t + {0..3, 8..11} + 4 hl, and V^T is read in that same order
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      mw_bf16x8_t p_hi, p_lo;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float p = sc[8 * t + x];
        const __bf16 hi = (__bf16)p;
        p_hi[x] = hi;
        p_lo[x] = (__bf16)(p - (float)hi);
      }
#pragma unroll
      for (int i = 0; i < VD / 32; ++i) {
        const bf16_t* src = vt + (i * 32 + c) * LDT;
        const uint2 a0 = *(const uint2*)(src + mw_swz(16 * t + 4 * hl, i * 32 + c));
        const uint2 a1 = *(const uint2*)(src + mw_swz(16 * t + 8 + 4 * hl, i * 32 + c));
        mw_u32x4_t av = {a0.x, a0.y, a1.x, a1.y};
        const mw_bf16x8_t vv = *(const mw_bf16x8_t*)&av;
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vv, p_hi, acc[i], 0, 0, 0);
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vv, p_lo, acc[i], 0, 0, 0);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();               // the tile is read before it is written again
  }
  if (!row_ok) return;
  // acc[i][r] is element d = 32 i + 8 (r / 4) + 4 hl + r % 4 of this lane's row
  if (DECODE || n_splits > 1) {
    const size_t slot = ((size_t)tok * a.nH + h) * n_splits + split;
    float* po = ws_o + slot * VD;
#pragma unroll
    for (int i = 0; i < VD / 32; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4)
        *(float4*)(po + 32 * i + 8 * r4 + 4 * hl) = make_float4(acc[i][4 * r4], acc[i][4 * r4 + 1],
                                                                acc[i][4 * r4 + 2], acc[i][4 * r4 + 3]);
    if (hl == 0) {
      ws_ml[2 * slot] = m;
      ws_ml[2 * slot + 1] = l;
    }
  } else {
    float inv = 1.0f / l;
    if (a.gate_mode == MA_GATE_HEAD)
      inv *= 1.0f / (1.0f + expf(-bf16_to_float(gate[(size_t)tok * a.gate_stride + h])));
    bf16_t* orow = out + ((size_t)tok * a.nH + h) * VD;
    const bf16_t* grow = a.gate_mode == MA_GATE_ELEMENT
        ? gate + (size_t)tok * a.gate_stride + (size_t)h * VD : nullptr;
#pragma unroll
    for (int i = 0; i < VD / 32; ++i)
#pragma unroll
      for (int r4 = 0; r4 < 4; ++r4) {
        const int d = 32 * i + 8 * r4 + 4 * hl;
        float v[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          v[x] = acc[i][4 * r4 + x] * inv;
          if (grow != nullptr) v[x] *= 1.0f / (1.0f + expf(-bf16_to_float(grow[d + x])));
        }
        *(uint2*)(orow + d) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      }
  }
}

// one wave per (token, head): the splits' partials in split order (their maxima are scores
// times log2(e)), then the gate
__global__ __launch_bounds__(ZF_WAVE) void masked_attention_merge_kernel(
    const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
    const bf16_t* __restrict__ gate, long long gate_stride, int gate_mode,
    bf16_t* __restrict__ out, int nH, int vd, int n_splits) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t slot0 = ((size_t)t * nH + h) * n_splits;
  // lane z holds split z's maximum and sum (at most 64 splits); a split without keys has the
  // maximum -inf and counts for nothing
  float mz = -INFINITY, lz = 0.f;
  if (lane < n_splits) {
    mz = ws_ml[2 * (slot0 + lane)];
    lz = ws_ml[2 * (slot0 + lane) + 1];
  }
  const float M = wave_max(mz);
  __shared__ float w[ZF_WAVE], lw[ZF_WAVE];
  w[lane] = mz == -INFINITY ? 0.f : exp2f(mz - M);
  lw[lane] = lz * w[lane];
  __syncthreads();
  float L = 0.f;
  for (int z = 0; z < n_splits; ++z) L += lw[z];
  float inv = 1.0f / L;
  if (gate_mode == MA_GATE_HEAD)
    inv *= 1.0f / (1.0f + expf(-bf16_to_float(gate[(size_t)t * gate_stride + h])));
  for (int d = lane; d < vd; d += ZF_WAVE) {
    float o = 0.f;
    for (int z = 0; z < n_splits; ++z) o += ws_o[(slot0 + z) * vd + d] * w[z];
    o *= inv;
    if (gate_mode == MA_GATE_ELEMENT)
      o *= 1.0f / (1.0f + expf(-bf16_to_float(gate[(size_t)t * gate_stride + (size_t)h * vd + d])));
    out[((size_t)t * nH + h) * vd + d] = float_to_bf16(o);
  }
}

#define MW_LAUNCH(KD, VD, TIED, DEC)                                                             \
  hipLaunchKernelGGL((masked_attention_wave_kernel<KD, VD, TIED, DEC>), grid, dim3(256), 0,      \
                     stream, (const bf16_t*)q, (const bf16_t*)gate, (const bf16_t*)k_pool,       \
                     (const bf16_t*)v_pool, sink, block_table, q_start, ctx_len, (bf16_t*)out,   \
                     ws_o, ws_ml, a)

// the shapes that are built: values of their own as wide as the keys; and the keys' leading
// columns as values (a latent and a rotated part behind it, or the latent alone)
#define MW_SHAPES(DEC)                                                                           \
  if (!tied && KD == 64 && VD == 64) MW_LAUNCH(64, 64, false, DEC);                              \
  else if (!tied && KD == 96 && VD == 96) MW_LAUNCH(96, 96, false, DEC);                         \
  else if (!tied && KD == 128 && VD == 128) MW_LAUNCH(128, 128, false, DEC);                     \
  else if (tied && KD == 64 && VD == 64) MW_LAUNCH(64, 64, true, DEC);                           \
  else if (tied && KD == 96 && VD == 96) MW_LAUNCH(96, 96, true, DEC);                           \
  else if (tied && KD == 128 && VD == 128) MW_LAUNCH(128, 128, true, DEC);                       \
  else if (tied && KD == 96 && VD == 64) MW_LAUNCH(96, 64, true, DEC);                           \
  else if (tied && KD == 160 && VD == 128) MW_LAUNCH(160, 128, true, DEC);                       \
  else if (tied && KD == 192 && VD == 128) MW_LAUNCH(192, 128, true, DEC);                       \
  else return -3

// decode == 0: a step's tokens in tiles of 128 / G positions, n_tiles an upper bound of the
// tiles over all sequences (workgroups beyond the real number leave at once), every wave's keys
// in n_splits parts.  decode != 0: token s is sequence s's one token; n_splits workgroups a
// (sequence, kv head), every wave a split of wave_keys keys (a multiple of 32).  With partial
// results: ws_o [T * nH * splits * VD], ws_ml [T * nH * splits * 2] floats, splits = n_splits
// (decode: 4 n_splits), at most 64.
extern "C" int zf_masked_attention_mfma(const void* q, long long q_stride, const void* gate,
                                        long long gate_stride, int gate_mode, const void* k_pool,
                                        const void* v_pool, const float* sink,
                                        const int* block_table, const int* q_start,
                                        const int* ctx_len, void* out, float* ws_o, float* ws_ml,
                                        float scale, float cap, int window, int chunk, int T,
                                        int n_seqs, int n_tiles, int nH, int nKV, int KD, int VD,
                                        int page_size, int max_pages, int decode, int n_splits,
                                        int wave_keys, hipStream_t stream) {
  if (T <= 0) return 0;
  const int splits = decode ? 4 * n_splits : n_splits;
  if (nKV <= 0 || nH % nKV != 0 || nH / nKV > 32 || page_size <= 0 || n_splits < 1 ||
      splits > ZF_WAVE || ((decode || n_splits > 1) && (!ws_o || !ws_ml)) ||
      (decode && (wave_keys <= 0 || wave_keys % MW_KEYS != 0 || T != n_seqs)) ||
      gate_mode < 0 || gate_mode > 2 || (gate_mode != MA_GATE_NONE && gate == nullptr) ||
      window < 0 || chunk < 0 || cap < 0.f)
    return -2;
  const bool tied = v_pool == nullptr;
  MaskedWaveArgs a;
  a.q_stride = q_stride; a.gate_stride = gate_stride; a.scale = scale; a.cap = cap;
  a.window = window; a.chunk = chunk; a.gate_mode = gate_mode; a.n_seqs = n_seqs; a.nH = nH;
  a.nKV = nKV; a.page_size = page_size; a.max_pages = max_pages;
  a.QT = decode ? 1 : MW_ROWS / (nH / nKV);
  a.wave_keys = wave_keys;
  if (decode) {
    dim3 grid(n_seqs, nKV, n_splits);
    MW_SHAPES(true);
  } else {
    if (n_tiles <= 0) return 0;
    dim3 grid(n_tiles, nKV, n_splits);
    MW_SHAPES(false);
  }
  if (decode || n_splits > 1)
    hipLaunchKernelGGL(masked_attention_merge_kernel, dim3(T, nH), dim3(ZF_WAVE), 0, stream, ws_o,
                       ws_ml, (const bf16_t*)gate, gate_stride, gate_mode, (bf16_t*)out, nH, VD,
                       splits);
  ZF_CHECK_LAUNCH();
}
