// Residual stream of a stack whose sublayers all read ONE norm (the mixer and
// the feed-forward run side by side on the same normed input), with an RMS
// norm taken in groups; embedding with a hashed (previous token, token) pair
// table; squared relu; rotation of attention results back by their position.
//
//   group_rmsnorm_add   : x <- x + (y1 + y2) in fp32, then the row is split
//                         into `groups` equal consecutive parts, each divided
//                         by its own sqrt(mean(part^2) + eps), and the whole
//                         multiplied by w -> the next layer's input in the
//                         activation type. One 256-thread workgroup per token;
//                         up to width 4096 the row stays in registers
//                         (16-byte accesses), each thread leaves the sum of
//                         its 4 squares in LDS and one wave per group adds the
//                         group's partial sums in a fixed order.
//   pair_hash_embedding : out = table[id] * scale + pair[r] in fp32, r = (prev
//                         * mul_prev + id * mul_cur) mod buckets, or the pair
//                         table's last row for a token without a predecessor.
//   relu_squared        : max(x, 0)^2 over a strided [rows, I] view.
//   rotate_heads        : x [T, H, D] fp32 -> every head turned over its whole
//                         width by sign * pos * freq[m] (pairs m, m + D/2 or
//                         2m, 2m + 1); the token's cos/sin are worked out once
//                         per workgroup.
#include "seq_common.h"

#define GN_MAXV 4  // 256 threads x 4 elements x GN_MAXV = width 4096 in registers

template <typename T>
DEVINL void gn_load4(const T* p, float* v);
template <>
DEVINL void gn_load4<bf16_t>(const bf16_t* p, float* v) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  v[0] = bf16_bits_to_f32((uint16_t)(raw.x & 0xffff));
  v[1] = bf16_bits_to_f32((uint16_t)(raw.x >> 16));
  v[2] = bf16_bits_to_f32((uint16_t)(raw.y & 0xffff));
  v[3] = bf16_bits_to_f32((uint16_t)(raw.y >> 16));
}
template <>
DEVINL void gn_load4<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
template <typename T>
DEVINL void gn_store4(T* p, const float* v);
template <>
DEVINL void gn_store4<bf16_t>(bf16_t* p, const float* v) {
  uint2 raw;
  raw.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  raw.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}
template <>
DEVINL void gn_store4<float>(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

// LDS: VEC: [GN_MAXV * 256] partial sums | [groups] 1 / rms; else [groups].
// VEC: W % 4 == 0, (W / groups) % 4 == 0, W <= 4096, rows 16-byte aligned
// (8-byte for bf16).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void group_rmsnorm_add_kernel(
    float* __restrict__ x, const T* __restrict__ y1, int64_t y1_stride,
    const T* __restrict__ y2, int64_t y2_stride, const T* __restrict__ w,
    float eps, T* __restrict__ out, int W, int groups) {
  extern __shared__ float lds[];
  const int64_t row = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* xr = x + row * (int64_t)W;
  const T* r1 = y1 ? y1 + row * y1_stride : nullptr;
  const T* r2 = y2 ? y2 + row * y2_stride : nullptr;
  const int gw = W / groups;
  if (VEC) {
    float* rinv = lds + GN_MAXV * 256;
    float v[GN_MAXV][4];
#pragma unroll
    for (int c = 0; c < GN_MAXV; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        gn_load4<float>(xr + i, v[c]);
        if (r1) {
          float a[4], b[4] = {0.f, 0.f, 0.f, 0.f};
          gn_load4<T>(r1 + i, a);
          if (r2) gn_load4<T>(r2 + i, b);
#pragma unroll
          for (int j = 0; j < 4; ++j) v[c][j] += a[j] + b[j];
          gn_store4<float>(xr + i, v[c]);
        }
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) ss = fmaf(v[c][j], v[c][j], ss);
        lds[c * 256 + threadIdx.x] = ss;
      }
    }
    if (w == nullptr) return;
    __syncthreads();
    const int gp = gw / 4;  // partial sums per group, consecutive
    for (int g = wave; g < groups; g += 4) {
      float s = 0.f;
      for (int p = lane; p < gp; p += 64) s += lds[g * gp + p];
      s = wave_reduce_sum(s);
      if (lane == 0) rinv[g] = 1.0f / sqrtf(s / (float)gw + eps);
    }
    __syncthreads();
    T* o = out + row * (int64_t)W;
#pragma unroll
    for (int c = 0; c < GN_MAXV; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        const float r = rinv[i / gw];
        float wv[4], h[4];
        gn_load4<T>(w + i, wv);
#pragma unroll
        for (int j = 0; j < 4; ++j) h[j] = v[c][j] * r * wv[j];
        gn_store4<T>(o + i, h);
      }
    }
  } else {
    if (r1) {
      for (int i = threadIdx.x; i < W; i += 256) {
        float y = ldf(r1 + i);
        if (r2) y += ldf(r2 + i);
        xr[i] += y;
      }
    }
    if (w == nullptr) return;
    __syncthreads();  // the workgroup's own stores to the row are visible
    for (int g = wave; g < groups; g += 4) {
      float s = 0.f;
      for (int i = lane; i < gw; i += 64) {
        const float t = xr[g * gw + i];
        s = fmaf(t, t, s);
      }
      s = wave_reduce_sum(s);
      if (lane == 0) lds[g] = 1.0f / sqrtf(s / (float)gw + eps);
    }
    __syncthreads();
    T* o = out + row * (int64_t)W;
    for (int i = threadIdx.x; i < W; i += 256)
      stf(o + i, xr[i] * lds[i / gw] * ldf(w + i));
  }
}

extern "C" void launch_group_rmsnorm_add(float* x, const void* y1,
                                         int64_t y1_stride, const void* y2,
                                         int64_t y2_stride, const void* w,
                                         float eps, void* out, int rows, int W,
                                         int groups, int kind,
                                         hipStream_t stream) {
  if (rows == 0) return;
  const int esz = kind == 0 ? 2 : 4;
  const bool vec = W % 4 == 0 && (W / groups) % 4 == 0 && W <= 1024 * GN_MAXV &&
                   (y1 == nullptr || (y1_stride % 4 == 0 &&
                                      ((uintptr_t)y1 % (4 * esz)) == 0)) &&
                   (y2 == nullptr || (y2_stride % 4 == 0 &&
                                      ((uintptr_t)y2 % (4 * esz)) == 0));
  const size_t shm = sizeof(float) * ((vec ? GN_MAXV * 256 : 0) + groups);
#define GN_CALL(TT, V)                                                       \
  hipLaunchKernelGGL((group_rmsnorm_add_kernel<TT, V>), dim3(rows), dim3(256), \
                     shm, stream, x, (const TT*)y1, y1_stride, (const TT*)y2, \
                     y2_stride, (const TT*)w, eps, (TT*)out, W, groups)
  if (kind == 0) {
    if (vec) GN_CALL(bf16_t, true);
    else GN_CALL(bf16_t, false);
  } else {
    if (vec) GN_CALL(float, true);
    else GN_CALL(float, false);
  }
#undef GN_CALL
}

// ---- embedding with a hashed pair table -----------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void pair_hash_embedding_kernel(
    float* __restrict__ out, const int64_t* __restrict__ ids,
    const int64_t* __restrict__ prev, const T* __restrict__ table,
    const T* __restrict__ pair, float scale, int64_t buckets, int64_t mul_prev,
    int64_t mul_cur, int64_t vocab, int W) {
  const int64_t t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // never read off the table
  const int64_t pv = prev[t];
  const int64_t r = pv < 0 ? buckets : (pv * mul_prev + id * mul_cur) % buckets;
  const T* e = table + id * (int64_t)W;
  const T* b = pair + r * (int64_t)W;
  float* o = out + t * (int64_t)W;
  for (int i = threadIdx.x; i < W; i += 256)
    o[i] = fmaf(ldf(e + i), scale, ldf(b + i));
}

extern "C" void launch_pair_hash_embedding(float* out, const int64_t* ids,
                                           const int64_t* prev,
                                           const void* table, const void* pair,
                                           float scale, int64_t buckets,
                                           int64_t mul_prev, int64_t mul_cur,
                                           int64_t vocab, int W, int T_,
                                           int kind, hipStream_t stream) {
  if (T_ == 0) return;
  if (kind == 0)
    hipLaunchKernelGGL((pair_hash_embedding_kernel<bf16_t>), dim3(T_), dim3(256),
                       0, stream, out, ids, prev, (const bf16_t*)table,
                       (const bf16_t*)pair, scale, buckets, mul_prev, mul_cur,
                       vocab, W);
  else
    hipLaunchKernelGGL((pair_hash_embedding_kernel<float>), dim3(T_), dim3(256),
                       0, stream, out, ids, prev, (const float*)table,
                       (const float*)pair, scale, buckets, mul_prev, mul_cur,
                       vocab, W);
}

// ---- squared relu --------------------------------------------------------------

DEVINL float relu2_f(float z) {
  z = fmaxf(z, 0.f);
  return z * z;
}

// x [rows, I] (row stride free) -> out [rows, I]
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void relu_squared_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride, int I,
    int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  if (VEC) {
    const int I4 = I / 4;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
      const int64_t row = i / I4;
      const int c = (int)(i % I4) * 4;
      float v[4];
      gn_load4<T>(x + row * x_stride + c, v);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = relu2_f(v[j]);
      gn_store4<T>(out + row * (int64_t)I + c, v);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
      const int64_t row = i / I;
      const int c = (int)(i % I);
      stf(out + i, relu2_f(ldf(x + row * x_stride + c)));
    }
  }
}

extern "C" void launch_relu_squared(void* out, const void* x, int64_t x_stride,
                                    int I, int rows, int kind,
                                    hipStream_t stream) {
  if (rows == 0 || I == 0) return;
  const int esz = kind == 0 ? 2 : 4;
  const bool vec = I % 4 == 0 && x_stride % 4 == 0 &&
                   ((uintptr_t)x % (4 * esz)) == 0;
  const int64_t n = vec ? (int64_t)rows * (I / 4) : (int64_t)rows * I;
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, 256 * 16);
#define R2_CALL(TT, V)                                                        \
  hipLaunchKernelGGL((relu_squared_kernel<TT, V>), dim3(blocks), dim3(256), 0, \
                     stream, (TT*)out, (const TT*)x, x_stride, I, n)
  if (kind == 0) {
    if (vec) R2_CALL(bf16_t, true);
    else R2_CALL(bf16_t, false);
  } else {
    if (vec) R2_CALL(float, true);
    else R2_CALL(float, false);
  }
#undef R2_CALL
}

// ---- rotation of head rows by position -------------------------------------------

// x [T, H, D] fp32 -> out [T, H * D]; LDS: [D / 2][2] cos, sin
template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_kernel(
    T* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ freq, const int* __restrict__ positions, int H,
    int D, int inter, float sign) {
  extern __shared__ float cs[];
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int half = D / 2;
  for (int i = threadIdx.x; i < half; i += 256) {
    float sn, c;
    sincosf(pos * freq[i], &sn, &c);
    cs[2 * i] = c;
    cs[2 * i + 1] = sn * sign;
  }
  __syncthreads();
  const float* xr = x + t * (int64_t)H * D;
  T* o = out + t * (int64_t)H * D;
  const int n = H * half;
  for (int idx = threadIdx.x; idx < n; idx += 256) {
    const int h = idx / half, m = idx % half;
    const int iu = h * D + (inter ? 2 * m : m);
    const int iv = h * D + (inter ? 2 * m + 1 : m + half);
    const float u = xr[iu], v = xr[iv];
    const float c = cs[2 * m], sn = cs[2 * m + 1];
    stf(o + iu, u * c - v * sn);
    stf(o + iv, v * c + u * sn);
  }
}

// the same with the tokens' (cos, sin) pairs given: table [T, D / 2][2]
template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_table_kernel(
    T* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ table, int H, int D, int inter, float sign) {
  const int64_t t = blockIdx.x;
  const int half = D / 2;
  const float* cs = table + t * (int64_t)D;
  const float* xr = x + t * (int64_t)H * D;
  T* o = out + t * (int64_t)H * D;
  const int n = H * half;
  for (int idx = threadIdx.x; idx < n; idx += 256) {
    const int h = idx / half, m = idx % half;
    const int iu = h * D + (inter ? 2 * m : m);
    const int iv = h * D + (inter ? 2 * m + 1 : m + half);
    const float u = xr[iu], v = xr[iv];
    const float c = cs[2 * m], sn = cs[2 * m + 1] * sign;
    stf(o + iu, u * c - v * sn);
    stf(o + iv, v * c + u * sn);
  }
}

extern "C" void launch_rotate_heads_table(void* out, const float* x,
                                          const float* table, int H, int D,
                                          int inter, float sign, int T_,
                                          int kind, hipStream_t stream) {
  if (T_ == 0) return;
  if (kind == 0)
    hipLaunchKernelGGL((rotate_heads_table_kernel<bf16_t>), dim3(T_), dim3(256),
                       0, stream, (bf16_t*)out, x, table, H, D, inter, sign);
  else
    hipLaunchKernelGGL((rotate_heads_table_kernel<float>), dim3(T_), dim3(256),
                       0, stream, (float*)out, x, table, H, D, inter, sign);
}

extern "C" void launch_rotate_heads(void* out, const float* x, const float* freq,
                                    const int* positions, int H, int D,
                                    int inter, float sign, int T_, int kind,
                                    hipStream_t stream) {
  if (T_ == 0) return;
  const size_t shm = sizeof(float) * (size_t)D;
  if (kind == 0)
    hipLaunchKernelGGL((rotate_heads_kernel<bf16_t>), dim3(T_), dim3(256), shm,
                       stream, (bf16_t*)out, x, freq, positions, H, D, inter,
                       sign);
  else
    hipLaunchKernelGGL((rotate_heads_kernel<float>), dim3(T_), dim3(256), shm,
                       stream, (float*)out, x, freq, positions, H, D, inter,
                       sign);
}
