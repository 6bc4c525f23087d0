// Post-norm residual step, clamped gated linear unit, minGRU scan.
//
//   branch_rmsnorm_add : one residual step of a stack that norms a sublayer's
//                        OUTPUT: y = a y1 (+ b y2), x <- x + y / rms(y) * w,
//                        and the stream rounded to the activation type as
//                        the next sublayer's input. One 256-thread workgroup
//                        per token; up to width 4096 the row stays in
//                        registers (16-byte accesses when the width is a
//                        multiple of 4), so every operand is read once. The
//                        stream is fp32; y1 has the activation type or fp32
//                        (fp32 expert sums), y2 the activation type.
//   clamped_glu        : [gate | up] -> a sigma(alpha a) (1 + b), a = gate cut
//                        off above at `limit`, b = up cut off at +-limit.
//   mingru_scan        : S_t = S_(t-1) + f_t (c_t - S_(t-1)) per channel, a
//                        thread per (sequence, channel), token-serial. The
//                        gate pre-activations of 8 tokens are loaded and
//                        turned into (f, c, silu(g)) off the dependent chain;
//                        the chain itself is one fused multiply-add per
//                        token.
//   mingru_chunk_*     : the same recurrence for long prompt portions, cut
//                        into chunks of L tokens that run side by side: the
//                        recurrence is affine in the state, so a first
//                        kernel reduces every chunk to (A, B) with S_out =
//                        A S_in + B (A = prod(1 - f), B = the chunk run from
//                        zero), and a second one folds the (A, B) of the
//                        chunks before its own into S_in and runs its chunk
//                        for the outputs. Everything fp32; the result
//                        differs from the serial order by rounding only.
#include "seq_common.h"

#define PN_MAXV 4  // 256 threads x 4 elements x PN_MAXV = width 4096 in registers

template <typename T>
DEVINL void pn_load4(const T* p, float* v);
template <>
DEVINL void pn_load4<bf16_t>(const bf16_t* p, float* v) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  v[0] = bf16_bits_to_f32((uint16_t)(raw.x & 0xffff));
  v[1] = bf16_bits_to_f32((uint16_t)(raw.x >> 16));
  v[2] = bf16_bits_to_f32((uint16_t)(raw.y & 0xffff));
  v[3] = bf16_bits_to_f32((uint16_t)(raw.y >> 16));
}
template <>
DEVINL void pn_load4<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}
template <typename T>
DEVINL void pn_store4(T* p, const float* v);
template <>
DEVINL void pn_store4<bf16_t>(bf16_t* p, const float* v) {
  uint2 raw;
  raw.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  raw.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}
template <>
DEVINL void pn_store4<float>(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

// VEC: W % 4 == 0, W <= 4096 and all rows 16-byte aligned (8-byte for bf16)
template <typename T, typename Y1, bool VEC>
__global__ __launch_bounds__(256) void branch_rmsnorm_add_kernel(
    const float* __restrict__ x_in, float* __restrict__ x_out,
    const Y1* __restrict__ y1, int64_t y1_stride, const T* __restrict__ y2,
    int64_t y2_stride, float a, float b, const T* __restrict__ w, float eps,
    T* __restrict__ out, int W) {
  __shared__ float scratch[8];
  const int64_t row = blockIdx.x;
  const Y1* r1 = y1 + row * y1_stride;
  const T* r2 = y2 ? y2 + row * y2_stride : nullptr;
  const float* xi = x_in ? x_in + row * (int64_t)W : nullptr;
  float* xo = x_out ? x_out + row * (int64_t)W : nullptr;
  T* o = out + row * (int64_t)W;
  if (VEC) {
    float v[PN_MAXV][4];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < PN_MAXV; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        pn_load4<Y1>(r1 + i, v[c]);
        float t2[4] = {0.f, 0.f, 0.f, 0.f};
        if (r2) pn_load4<T>(r2 + i, t2);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[c][j] = r2 ? fmaf(b, t2[j], a * v[c][j]) : a * v[c][j];
          ss = fmaf(v[c][j], v[c][j], ss);
        }
      }
    }
    ss = block256_sum(ss, scratch);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int c = 0; c < PN_MAXV; ++c) {
      const int i = (c * 256 + threadIdx.x) * 4;
      if (i < W) {
        float wv[4], xv[4] = {0.f, 0.f, 0.f, 0.f};
        pn_load4<T>(w + i, wv);
        if (xi) pn_load4<float>(xi + i, xv);
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] += v[c][j] * r * wv[j];
        if (xo) pn_store4<float>(xo + i, xv);
        pn_store4<T>(o + i, xv);
      }
    }
  } else {
    float ss = 0.f;
    for (int i = threadIdx.x; i < W; i += 256) {
      float y = a * ldf(r1 + i);
      if (r2) y = fmaf(b, ldf(r2 + i), y);
      ss = fmaf(y, y, ss);
    }
    ss = block256_sum(ss, scratch);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += 256) {
      float y = a * ldf(r1 + i);
      if (r2) y = fmaf(b, ldf(r2 + i), y);
      float n = y * r * ldf(w + i);
      if (xi) n += xi[i];
      if (xo) xo[i] = n;
      stf(o + i, n);
    }
  }
}

// kind: activation type (0 bf16, 1 float); y1_kind: type of y1
extern "C" void launch_branch_rmsnorm_add(
    const float* x_in, float* x_out, const void* y1, int64_t y1_stride,
    int y1_kind, const void* y2, int64_t y2_stride, float a, float b,
    const void* w, float eps, void* out, int rows, int W, int kind,
    hipStream_t stream) {
  if (rows == 0) return;
  const int esz = kind == 0 ? 2 : 4, e1 = y1_kind == 0 ? 2 : 4;
  const bool vec = W % 4 == 0 && W <= 1024 * PN_MAXV &&
                   (y1_stride * e1) % (4 * e1) == 0 &&
                   (y2 == nullptr || (y2_stride * esz) % (4 * esz) == 0) &&
                   ((uintptr_t)y1 % (4 * e1)) == 0 &&
                   (y2 == nullptr || ((uintptr_t)y2 % (4 * esz)) == 0);
#define PN_CALL(TT, YY, V)                                                     \
  hipLaunchKernelGGL((branch_rmsnorm_add_kernel<TT, YY, V>), dim3(rows),      \
                     dim3(256), 0, stream, x_in, x_out, (const YY*)y1,        \
                     y1_stride, (const TT*)y2, y2_stride, a, b, (const TT*)w, \
                     eps, (TT*)out, W)
  if (kind == 0) {
    if (y1_kind == 0) {
      if (vec) PN_CALL(bf16_t, bf16_t, true);
      else PN_CALL(bf16_t, bf16_t, false);
    } else {
      if (vec) PN_CALL(bf16_t, float, true);
      else PN_CALL(bf16_t, float, false);
    }
  } else {
    if (vec) PN_CALL(float, float, true);
    else PN_CALL(float, float, false);
  }
#undef PN_CALL
}

// ---- clamped gated linear unit ----------------------------------------------

DEVINL float pn_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

DEVINL float clamped_glu_f(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * pn_sigmoid(alpha * g) * (u + 1.0f);
}

// x [rows, 2 I] (row stride free) -> out [rows, I]
template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride, int I,
    int64_t n, float limit, float alpha) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
    const int64_t row = i / I;
    const int c = (int)(i % I);
    const T* xr = x + row * x_stride;
    stf(out + i, clamped_glu_f(ldf(xr + c), ldf(xr + I + c), limit, alpha));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_vec_kernel(
    T* __restrict__ out, const T* __restrict__ x, int64_t x_stride, int I,
    int64_t n4, float limit, float alpha) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int I4 = I / 4;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
    const int64_t row = i / I4;
    const int c = (int)(i % I4) * 4;
    const T* xr = x + row * x_stride;
    float g[4], u[4], r[4];
    pn_load4<T>(xr + c, g);
    pn_load4<T>(xr + I + c, u);
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = clamped_glu_f(g[j], u[j], limit, alpha);
    pn_store4<T>(out + row * (int64_t)I + c, r);
  }
}

extern "C" void launch_clamped_glu(void* out, const void* x, int64_t x_stride,
                                   int rows, int I, float limit, float alpha,
                                   int kind, hipStream_t stream) {
  const int64_t n = (int64_t)rows * I;
  if (n == 0) return;
  const int esz = kind == 0 ? 2 : 4;
  const bool vec = I % 4 == 0 && x_stride % 4 == 0 &&
                   ((uintptr_t)x % (4 * esz)) == 0;
  const int64_t items = vec ? n / 4 : n;
  const int64_t want = (items + 255) / 256;
  const int blocks = (int)(want < 8192 ? want : 8192);
#define CG_CALL(K, TT, N)                                                     \
  hipLaunchKernelGGL((K<TT>), dim3(blocks), dim3(256), 0, stream, (TT*)out,   \
                     (const TT*)x, x_stride, I, N, limit, alpha)
  if (kind == 0) {
    if (vec) CG_CALL(clamped_glu_vec_kernel, bf16_t, items);
    else CG_CALL(clamped_glu_kernel, bf16_t, items);
  } else {
    if (vec) CG_CALL(clamped_glu_vec_kernel, float, items);
    else CG_CALL(clamped_glu_kernel, float, items);
  }
#undef CG_CALL
}

// ---- minGRU scan --------------------------------------------------------------

#define MG_CHUNK 8

// one chunk [t0, t1) of one channel from state S; OUT: write S_t silu(g_t).
// Returns the final state; *decay (when given) gets prod(1 - z_t).
template <typename T, bool OUT>
DEVINL float mingru_run(T* __restrict__ out, const T* __restrict__ zug,
                        int64_t stride, int t0, int t1, int c, int width,
                        float zb, float ub, float S, float* decay) {
  float A = 1.0f;
  for (int t = t0; t < t1; t += MG_CHUNK) {
    float z[MG_CHUNK], cand[MG_CHUNK], g[MG_CHUNK];
#pragma unroll
    for (int i = 0; i < MG_CHUNK; ++i) {
      const int tt = min(t + i, t1 - 1);
      const T* r = zug + (int64_t)tt * stride + c;
      z[i] = ldf(r);
      cand[i] = ldf(r + width);
      if (OUT) g[i] = ldf(r + 2 * width);
    }
#pragma unroll
    for (int i = 0; i < MG_CHUNK; ++i) {
      z[i] = pn_sigmoid(z[i] + zb);
      const float u = cand[i] + ub;
      cand[i] = u >= 0.f ? u + 0.5f : pn_sigmoid(u);
      if (OUT) g[i] = g[i] * pn_sigmoid(g[i]);
    }
#pragma unroll
    for (int i = 0; i < MG_CHUNK; ++i) {
      if (t + i < t1) {
        S = fmaf(z[i], cand[i] - S, S);
        A *= 1.0f - z[i];
        if (OUT) stf(out + (int64_t)(t + i) * width + c, S * g[i]);
      }
    }
  }
  if (decay) *decay = A;
  return S;
}

// zug [T, 3 width] (row stride free): z | u | g pre-activations. grid
// (sequences, ceil(width / 256)); cu == nullptr: sequence b is token b.
template <typename T>
__global__ __launch_bounds__(256) void mingru_scan_kernel(
    T* __restrict__ out, const T* __restrict__ zug, int64_t stride,
    const float* __restrict__ z_bias, const float* __restrict__ u_bias,
    float* __restrict__ state, const int64_t* __restrict__ slots,
    const int* __restrict__ cu, const int* __restrict__ positions, int width) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int t0 = cu ? cu[b] : b, t1 = cu ? cu[b + 1] : b + 1;
  if (t0 >= t1 || c >= width) return;
  float* sp = state + slots[b] * (int64_t)width + c;
  const float S = positions[t0] == 0 ? 0.f : *sp;
  *sp = mingru_run<T, true>(out, zug, stride, t0, t1, c, width, z_bias[c],
                            u_bias[c], S, nullptr);
}

// which (sequence, chunk) a tile is; false past the last one. base: index of
// the sequence's first tile.
DEVINL bool mingru_tile(const int* __restrict__ cu, int B, int L, int tile,
                        int* b_out, int* chunk, int* base) {
  int b = 0, first = 0;
  for (; b < B; ++b) {
    const int nt = (cu[b + 1] - cu[b] + L - 1) / L;
    if (tile < first + nt) break;
    first += nt;
  }
  if (b == B) return false;
  *b_out = b;
  *chunk = tile - first;
  *base = first;
  return true;
}

// carry [tiles][2][width]: (A, B) per chunk; init [B][width]: the state every
// sequence starts this step from (copied here so that no chunk reads the slot
// after the last chunk has written it)
template <typename T>
__global__ __launch_bounds__(256) void mingru_chunk_reduce_kernel(
    float* __restrict__ carry, float* __restrict__ init,
    const T* __restrict__ zug, int64_t stride, const float* __restrict__ z_bias,
    const float* __restrict__ u_bias, const float* __restrict__ state,
    const int64_t* __restrict__ slots, const int* __restrict__ cu,
    const int* __restrict__ positions, int B, int L, int width) {
  int b, chunk, base;
  if (!mingru_tile(cu, B, L, blockIdx.x, &b, &chunk, &base)) return;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = cu[b] + chunk * L, t1 = min(t0 + L, cu[b + 1]);
  if (chunk == 0)
    init[(int64_t)b * width + c] =
        positions[t0] == 0 ? 0.f : state[slots[b] * (int64_t)width + c];
  float A;
  const float Bv = mingru_run<T, false>(nullptr, zug, stride, t0, t1, c, width,
                                        z_bias[c], u_bias[c], 0.f, &A);
  float* dst = carry + (int64_t)blockIdx.x * 2 * width;
  dst[c] = A;
  dst[width + c] = Bv;
}

template <typename T>
__global__ __launch_bounds__(256) void mingru_chunk_apply_kernel(
    T* __restrict__ out, const float* __restrict__ carry,
    const float* __restrict__ init, const T* __restrict__ zug, int64_t stride,
    const float* __restrict__ z_bias, const float* __restrict__ u_bias,
    float* __restrict__ state, const int64_t* __restrict__ slots,
    const int* __restrict__ cu, int B, int L, int width) {
  int b, chunk, base;
  if (!mingru_tile(cu, B, L, blockIdx.x, &b, &chunk, &base)) return;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const int t0 = cu[b] + chunk * L, t1 = min(t0 + L, cu[b + 1]);
  float S = init[(int64_t)b * width + c];
  const float* cr = carry + (int64_t)base * 2 * width + c;
#pragma unroll 4
  for (int k = 0; k < chunk; ++k)
    S = fmaf(cr[(int64_t)k * 2 * width], S, cr[(int64_t)k * 2 * width + width]);
  S = mingru_run<T, true>(out, zug, stride, t0, t1, c, width, z_bias[c],
                          u_bias[c], S, nullptr);
  if (t1 == cu[b + 1]) state[slots[b] * (int64_t)width + c] = S;
}

// tiles: an upper bound on the number of chunks (ceil(T / L) + B); carry
// [tiles, 2, width] and init [B, width] fp32 scratch
extern "C" void launch_mingru_chunked(void* out, float* carry, float* init,
                                      const void* zug, int64_t stride,
                                      const float* z_bias, const float* u_bias,
                                      float* state, const int64_t* slots,
                                      const int* cu, const int* positions,
                                      int B, int L, int tiles, int width,
                                      int kind, hipStream_t stream) {
  if (B == 0 || width == 0 || tiles == 0) return;
  const dim3 grid(tiles, (width + 255) / 256);
  if (kind == 0) {
    hipLaunchKernelGGL((mingru_chunk_reduce_kernel<bf16_t>), grid, dim3(256), 0,
                       stream, carry, init, (const bf16_t*)zug, stride, z_bias,
                       u_bias, state, slots, cu, positions, B, L, width);
    hipLaunchKernelGGL((mingru_chunk_apply_kernel<bf16_t>), grid, dim3(256), 0,
                       stream, (bf16_t*)out, carry, init, (const bf16_t*)zug,
                       stride, z_bias, u_bias, state, slots, cu, B, L, width);
  } else {
    hipLaunchKernelGGL((mingru_chunk_reduce_kernel<float>), grid, dim3(256), 0,
                       stream, carry, init, (const float*)zug, stride, z_bias,
                       u_bias, state, slots, cu, positions, B, L, width);
    hipLaunchKernelGGL((mingru_chunk_apply_kernel<float>), grid, dim3(256), 0,
                       stream, (float*)out, carry, init, (const float*)zug,
                       stride, z_bias, u_bias, state, slots, cu, B, L, width);
  }
}

extern "C" void launch_mingru_scan(void* out, const void* zug, int64_t stride,
                                   const float* z_bias, const float* u_bias,
                                   float* state, const int64_t* slots,
                                   const int* cu, const int* positions, int B,
                                   int width, int kind, hipStream_t stream) {
  if (B == 0 || width == 0) return;
  const dim3 grid(B, (width + 255) / 256);
  if (kind == 0)
    hipLaunchKernelGGL((mingru_scan_kernel<bf16_t>), grid, dim3(256), 0, stream,
                       (bf16_t*)out, (const bf16_t*)zug, stride, z_bias, u_bias,
                       state, slots, cu, positions, width);
  else
    hipLaunchKernelGGL((mingru_scan_kernel<float>), grid, dim3(256), 0, stream,
                       (float*)out, (const float*)zug, stride, z_bias, u_bias,
                       state, slots, cu, positions, width);
}
