// Grouped-head attention over a row-per-token paged cache: softmax weights,
// or sigmoid(score + per-head bias) weights that are not normalised over the
// keys; optionally a per-head sigmoid gate on the result.
//
// A cache row holds, for one token, the keys of all kv heads and then the
// values of all kv heads: [G x M x d | G x dv], M = score maps per head (1, or
// 2 for differential attention, where both maps weight the same values).
// Queries arrive in fp32 (qkv_store prepares them); scores, softmax, the
// accumulation and the per-head post-processing are fp32; only the cache rows
// and the result have the activation type.
//
//   qkv_store         : queries -> fp32 (optional per-segment RMS norm with an
//                       optional weight, optional rotation by position of the
//                       segment's first dimensions, optional
//                       position-dependent temperature); keys (normed,
//                       weighted and rotated alike) and values scattered into
//                       the token's cache row. With no value tensor the
//                       values are the keys BEFORE the norm.
//   pool_cache_update : a token that completes a block of P positions writes
//                       the fp32 mean of the block's P cache rows to the
//                       sequence's pooled rows.
//   row_attention     : a workgroup per (token, kv head, group of HB query
//                       heads, share of the keys). The key list of a token at
//                       position p is [pooled blocks 0 .. nb) ++ [tokens lo ..
//                       p]: window 0 -> lo = 0, nb = 0 (full causal); window w
//                       -> lo = max(0, p - w + 1), nb = floor((p - w + 1) / P)
//                       blocks that lie wholly before the window. 64 keys per
//                       wave and pass, online softmax per (head, map). Score
//                       pass: a lane owns a key. Value pass: a lane owns 4
//                       value features and the wave's lanes split into 64 / FL
//                       key subgroups (FL lanes cover the value width).
//                       Prompt portions and decode rows are the same code;
//                       few tokens (decode) split their keys over several
//                       workgroups, sized from host-known numbers only, and
//                       row_attention_reduce joins the partial results.
//   epilogue          : o = a1 - lam * a2 (M = 2) or a1; optional division by
//                       the RMS over the value width, times out_mult;
//                       optional sigmoid(gate[t, h]) multiplier.
//   sigmoid weights   : with head_bias a visible key weighs sigmoid(score +
//                       head_bias[h]); the running maximum is pinned at 0
//                       and the denominator at 1, so partial results of
//                       waves and key shares simply add up.
#include "seq_common.h"

#define RA_WAVES 4

// ---- qkv_store -------------------------------------------------------------

// What a segment passes after its norm: a weight per dimension (shared by the
// segments) and a rotation of its first rot_dims dimensions by the token's
// position, dimension i paired with i + rot_dims / 2 at angle pos * freq[i]
// (fp32), cos and sin times rot_mult: the token's (cos, sin) pairs are worked
// out once per workgroup, in LDS, for all heads.
struct RaSegOps {
  const float* w;       // [seg] (or the whole row's width when w_full) or null
  const float* cs;      // LDS [rot_dims / 2][2]: cos, sin (scaled), or null
  int rot_dims;
  bool inter;           // pairs (2i, 2i + 1) instead of (i, i + rot_dims / 2)
  bool w_full;          // the weight has one entry per element of the row
  float r_whole;        // > 0: the row's 1 / RMS, used for every segment
};

// 1 / RMS over all n elements of a row; every thread of the workgroup gets it
template <typename TI>
DEVINL float ra_row_rrms(const TI* __restrict__ src, int n, float eps,
                         float* scratch) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += 64 * RA_WAVES) {
    const float t = ldf(src + i);
    ss += t * t;
  }
  ss = block256_sum(ss, scratch);
  return 1.0f / sqrtf(ss / (float)n + eps);
}

// n elements in segments of `seg`; NORM: every segment divided by its RMS
// (wave per segment), or by the row's when so.r_whole is set; then times mult.
template <typename TI, typename TO, bool NORM>
DEVINL void ra_segments(const TI* __restrict__ src, TO* __restrict__ dst, int n,
                        int seg, float eps, float mult, const RaSegOps& so) {
  if (NORM || so.w != nullptr || so.cs != nullptr) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int half = so.cs ? so.rot_dims / 2 : 0;
    for (int s0 = wave * seg; s0 < n; s0 += RA_WAVES * seg) {
      float r = mult;
      if (NORM) {
        if (so.r_whole > 0.f) {
          r = mult * so.r_whole;
        } else {
          float ss = 0.f;
          for (int i = lane; i < seg; i += 64) {
            const float t = ldf(src + s0 + i);
            ss += t * t;
          }
          ss = wave_reduce_sum(ss);
          r = mult / sqrtf(ss / (float)seg + eps);
        }
      }
      const float* w = so.w ? (so.w_full ? so.w + s0 : so.w) : nullptr;
      for (int i = lane; i < seg; i += 64) {
        if (i < half) {
          const int iu = so.inter ? 2 * i : i;
          const int iv = so.inter ? 2 * i + 1 : i + half;
          float u = ldf(src + s0 + iu) * r, v = ldf(src + s0 + iv) * r;
          if (w) {
            u *= w[iu];
            v *= w[iv];
          }
          const float cs = so.cs[2 * i], sn = so.cs[2 * i + 1];
          stf(dst + s0 + iu, u * cs - v * sn);
          stf(dst + s0 + iv, v * cs + u * sn);
        } else if (i >= 2 * half) {
          float t = ldf(src + s0 + i) * r;
          if (w) t *= w[i];
          stf(dst + s0 + i, t);
        }
      }
    }
  } else {
    for (int i = threadIdx.x; i < n; i += 64 * RA_WAVES)
      stf(dst + i, ldf(src + i) * mult);
  }
}

// n elements of a token's row into LDS as floats; vec: 16-byte loads (the row
// starts 16-byte aligned and n is a multiple of 8)
template <typename T>
DEVINL void ra_stage(const T* __restrict__ src, float* __restrict__ dst, int n,
                     bool vec) {
  if (vec) {
    for (int i = threadIdx.x * 8; i < n; i += 64 * RA_WAVES * 8) {
      float v[8];
      if (sizeof(T) == 2) {
        const bf16x8 raw = load_bf16x8(src + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = bf16x8_get(raw, j);
      } else {
        const float4 a = *reinterpret_cast<const float4*>(src + i);
        const float4 b = *reinterpret_cast<const float4*>(src + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
      }
      *reinterpret_cast<float4*>(dst + i) = make_float4(v[0], v[1], v[2], v[3]);
      *reinterpret_cast<float4*>(dst + i + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
  } else {
    for (int i = threadIdx.x; i < n; i += 64 * RA_WAVES) dst[i] = ldf(src + i);
  }
}

// LDS: [rot_dims] cos/sin pairs | [v_seg] cos/sin pairs of the value rotation
// | [wq + wk] the token's queries and keys as floats when `staged` (they
// fit): one pass of wide loads, then the segment work runs out of LDS
// instead of re-reading global memory per segment.
// whole: the RMS of NORM runs over the whole query row and the whole key row
// (weights as wide as the rows) instead of per segment. inter: rotation pairs
// (2i, 2i + 1). v_freq: every v_seg-wide segment of the values is rotated
// over its whole width by pos * v_freq[m] before it is stored.
template <typename T, bool NORM>
__global__ __launch_bounds__(256) void qkv_store_kernel(
    float* __restrict__ q_out, const T* __restrict__ q, int64_t q_stride,
    const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const int* __restrict__ positions,
    const int64_t* __restrict__ slots, T* __restrict__ cache, int wq, int wk,
    int wv, int seg, float eps, float temp_coef, int temp_every,
    const float* __restrict__ q_weight, const float* __restrict__ k_weight,
    const float* __restrict__ rot_freq, float rot_mult, int rot_dims,
    int staged, int vec, int whole, int inter,
    const float* __restrict__ v_freq, int v_seg, float* __restrict__ v_cs_out) {
  __shared__ float red[8];
  const int64_t t = blockIdx.x;
  float temp = 1.0f;
  if (temp_every > 0)
    temp = 1.0f + temp_coef * logf((float)((positions[t] + 1) / temp_every) + 1.0f);
  extern __shared__ float rot_cs[];  // [rot_dims / 2][2]
  float* v_cs = rot_cs + ((rot_freq ? rot_dims : 0) + 3) / 4 * 4;
  float* stage = v_cs + ((v_freq ? v_seg : 0) + 3) / 4 * 4;
  if (staged) {
    ra_stage<T>(q + t * q_stride, stage, wq, vec);
    if (k != nullptr) ra_stage<T>(k + t * k_stride, stage + wq, wk, vec);
  }
  const float pos = (float)positions[t];
  if (rot_freq != nullptr) {
    for (int i = threadIdx.x; i < rot_dims / 2; i += 64 * RA_WAVES) {
      float sn, cs;
      sincosf(pos * rot_freq[i], &sn, &cs);
      rot_cs[2 * i] = cs * rot_mult;
      rot_cs[2 * i + 1] = sn * rot_mult;
    }
  }
  if (v_freq != nullptr) {
    for (int i = threadIdx.x; i < v_seg / 2; i += 64 * RA_WAVES) {
      float sn, cs;
      sincosf(pos * v_freq[i], &sn, &cs);
      v_cs[2 * i] = cs;
      v_cs[2 * i + 1] = sn;
    }
  }
  __syncthreads();
  // the token's (cos, sin) pairs of the value rotation, for the attention
  // kernels that turn their results back
  if (v_cs_out != nullptr)
    for (int i = threadIdx.x; i < v_seg; i += 64 * RA_WAVES)
      v_cs_out[t * v_seg + i] = v_cs[i];
  const bool full = NORM && whole;
  RaSegOps so{q_weight, rot_freq ? rot_cs : nullptr, rot_dims, inter != 0,
              full, 0.f};
  if (staged) {
    if (full) so.r_whole = ra_row_rrms<float>(stage, wq, eps, red);
    ra_segments<float, float, NORM>(stage, q_out + t * wq, wq, seg, eps, temp, so);
  } else {
    if (full) so.r_whole = ra_row_rrms<T>(q + t * q_stride, wq, eps, red);
    ra_segments<T, float, NORM>(q + t * q_stride, q_out + t * wq, wq, seg, eps,
                                temp, so);
  }
  if (k == nullptr) return;
  const int64_t slot = slots[t];
  if (slot < 0) return;  // pad row of a captured graph
  T* row = cache + slot * (int64_t)(wk + wv);
  so.w = k_weight;
  if (staged) {
    if (full) so.r_whole = ra_row_rrms<float>(stage + wq, wk, eps, red);
    ra_segments<float, T, NORM>(stage + wq, row, wk, seg, eps, 1.0f, so);
  } else {
    if (full) so.r_whole = ra_row_rrms<T>(k + t * k_stride, wk, eps, red);
    ra_segments<T, T, NORM>(k + t * k_stride, row, wk, seg, eps, 1.0f, so);
  }
  const T* vals = v ? v + t * v_stride : k + t * k_stride;
  if (v_freq != nullptr) {
    const RaSegOps sv{nullptr, v_cs, v_seg, inter != 0, false, 0.f};
    ra_segments<T, T, false>(vals, row + wk, wv, v_seg, eps, 1.0f, sv);
  } else {
    for (int i = threadIdx.x; i < wv; i += 64 * RA_WAVES) row[wk + i] = vals[i];
  }
}

extern "C" void launch_qkv_store(float* q_out, const void* q, int64_t q_stride,
                                 const void* k, int64_t k_stride, const void* v,
                                 int64_t v_stride, const int* positions,
                                 const int64_t* slots, void* cache, int wq,
                                 int wk, int wv, int seg, float eps,
                                 float temp_coef, int temp_every,
                                 const float* q_weight, const float* k_weight,
                                 const float* rot_freq, float rot_mult,
                                 int rot_dims, int whole, int inter,
                                 const float* v_freq, int v_seg,
                                 float* v_cs_out, int T_, int kind,
                                 hipStream_t stream) {
  if (T_ == 0) return;
#define QS_ARGS(TT)                                                          \
  q_out, (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v,       \
      v_stride, positions, slots, (TT*)cache, wq, wk, wv, seg, eps,          \
      temp_coef, temp_every, q_weight, k_weight, rot_freq, rot_mult, rot_dims,  \
      staged, vec, whole, inter, v_freq, v_seg, v_cs_out
  const bool norm = eps >= 0.f;
  // stage the token's queries and keys in LDS when they fit in 48 KB
  const int rot_floats = ((rot_freq ? rot_dims : 0) + 3) / 4 * 4 +
                         ((v_freq ? v_seg : 0) + 3) / 4 * 4;
  const int staged = (rot_floats + wq + wk) <= 12 * 1024;
  const int vec = wq % 8 == 0 && wk % 8 == 0 && q_stride % 8 == 0 &&
                  k_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 &&
                  (k == nullptr || ((uintptr_t)k % 16) == 0);
  const size_t shm = sizeof(float) * (rot_floats + (staged ? wq + wk : 0));
  if (kind == 0) {
    if (norm)
      hipLaunchKernelGGL((qkv_store_kernel<bf16_t, true>), dim3(T_), dim3(256),
                         shm, stream, QS_ARGS(bf16_t));
    else
      hipLaunchKernelGGL((qkv_store_kernel<bf16_t, false>), dim3(T_), dim3(256),
                         shm, stream, QS_ARGS(bf16_t));
  } else {
    if (norm)
      hipLaunchKernelGGL((qkv_store_kernel<float, true>), dim3(T_), dim3(256),
                         shm, stream, QS_ARGS(float));
    else
      hipLaunchKernelGGL((qkv_store_kernel<float, false>), dim3(T_), dim3(256),
                         shm, stream, QS_ARGS(float));
  }
#undef QS_ARGS
}

// ---- pool_cache_update -----------------------------------------------------

// grid (tokens, column chunks of 256): a thread owns one column and adds the
// block's rows in position order; the rows' offsets are looked up once per
// workgroup (LDS) so that the loads of a column do not wait on table reads.
template <typename T>
__global__ __launch_bounds__(256) void pool_cache_update_kernel(
    const T* __restrict__ cache, float* __restrict__ pool,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ token_seq, const int* __restrict__ positions,
    const int64_t* __restrict__ slots, int E, int block_size, int per_page,
    int P) {
  __shared__ int64_t roff[256];
  const int64_t t = blockIdx.x;
  if (slots[t] < 0) return;
  const int pos = positions[t];
  if ((pos + 1) % P != 0) return;
  const int b = token_seq ? token_seq[t] : (int)t;
  const int* bt = block_tables + (int64_t)b * bt_stride;
  const int blk = pos / P;
  const int c = blockIdx.y * 256 + threadIdx.x;
  float acc = 0.f;
  for (int j0 = pos - P + 1; j0 <= pos; j0 += 256) {
    __syncthreads();
    const int j = j0 + threadIdx.x;
    if (j <= pos)
      roff[threadIdx.x] = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
    __syncthreads();
    const int nr = min(256, pos - j0 + 1);
    if (c < E) {
#pragma unroll 8
      for (int r = 0; r < nr; ++r) acc += ldf(cache + roff[r] + c);
    }
  }
  if (c < E)
    pool[((int64_t)bt[blk / per_page] * per_page + blk % per_page) * E + c] =
        acc / (float)P;
}

extern "C" void launch_pool_cache_update(const void* cache, float* pool,
                                         const int* block_tables, int bt_stride,
                                         const int* token_seq,
                                         const int* positions,
                                         const int64_t* slots, int E,
                                         int block_size, int per_page, int P,
                                         int T_, int kind, hipStream_t stream) {
  if (T_ == 0) return;
  if (kind == 0)
    hipLaunchKernelGGL((pool_cache_update_kernel<bf16_t>),
                       dim3(T_, (E + 255) / 256), dim3(256), 0, stream, (const bf16_t*)cache, pool, block_tables,
                       bt_stride, token_seq, positions, slots, E, block_size,
                       per_page, P);
  else
    hipLaunchKernelGGL((pool_cache_update_kernel<float>),
                       dim3(T_, (E + 255) / 256), dim3(256), 0, stream, (const float*)cache, pool, block_tables,
                       bt_stride, token_seq, positions, slots, E, block_size,
                       per_page, P);
}

// ---- row_attention ---------------------------------------------------------

template <typename T>
DEVINL void ra_load8(const T* p, float* v);
template <>
DEVINL void ra_load8<bf16_t>(const bf16_t* p, float* v) {
  const bf16x8 raw = load_bf16x8(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = bf16x8_get(raw, i);
}
template <>
DEVINL void ra_load8<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

template <typename T>
DEVINL void ra_load4(const T* p, float* v);
template <>
DEVINL void ra_load4<bf16_t>(const bf16_t* p, float* v) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  v[0] = bf16_bits_to_f32((uint16_t)(raw.x & 0xffff));
  v[1] = bf16_bits_to_f32((uint16_t)(raw.x >> 16));
  v[2] = bf16_bits_to_f32((uint16_t)(raw.y & 0xffff));
  v[3] = bf16_bits_to_f32((uint16_t)(raw.y >> 16));
}
template <>
DEVINL void ra_load4<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
}

// s[n] += q[n] . key for NQ queries in LDS that lie `dp` floats apart at
// `qs`; key = d elements at `key`.
template <typename TK, int NQ, bool VEC>
DEVINL void ra_dot(const TK* __restrict__ key, const float* __restrict__ qs,
                   int dp, int d, float* s) {
  if (VEC) {
#pragma unroll 4
    for (int f = 0; f < d; f += 8) {
      float kv[8];
      ra_load8<TK>(key + f, kv);
#pragma unroll
      for (int n = 0; n < NQ; ++n) {
        const float4 qa = *reinterpret_cast<const float4*>(qs + n * dp + f);
        const float4 qb = *reinterpret_cast<const float4*>(qs + n * dp + f + 4);
        float a = s[n];
        a = fmaf(qa.x, kv[0], a);
        a = fmaf(qa.y, kv[1], a);
        a = fmaf(qa.z, kv[2], a);
        a = fmaf(qa.w, kv[3], a);
        a = fmaf(qb.x, kv[4], a);
        a = fmaf(qb.y, kv[5], a);
        a = fmaf(qb.z, kv[6], a);
        a = fmaf(qb.w, kv[7], a);
        s[n] = a;
      }
    }
  } else {
    for (int f = 0; f < d; ++f) {
      const float kv = ldf(key + f);
#pragma unroll
      for (int n = 0; n < NQ; ++n) s[n] = fmaf(qs[n * dp + f], kv, s[n]);
    }
  }
}

// The shared end of the main kernel and the reduce kernel: one wave turns the
// unnormalised sums of one head (M maps, acc[m * acc_stride + f], softmax
// denominators l[m]) into the head's output row.
template <typename T, int M>
DEVINL void ra_epilogue(T* __restrict__ dst, float* __restrict__ dst32,
                        const float* __restrict__ acc,
                        int acc_stride, const float* l, int dv, float lam,
                        float norm_eps, float out_mult, float post,
                        const float* __restrict__ rcs, int rot_inter) {
  const int lane = threadIdx.x & 63;
  const float i0 = 1.0f / l[0];
  const float i1 = M == 2 ? lam / l[1] : 0.f;
  float o[4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int f = lane + 64 * c;
    float v = 0.f;
    if (f < dv) {
      v = acc[f] * i0;
      if (M == 2) v -= acc[acc_stride + f] * i1;
      if (rcs != nullptr) {
        // rcs: the token's [dv / 2][2] cos, sin; the result turns BACK by its
        // angle: pair (u, w) -> (u cos + w sin, w cos - u sin)
        const int hv = dv >> 1;
        const bool first = rot_inter ? !(f & 1) : f < hv;
        const int fp = rot_inter ? (f ^ 1) : (first ? f + hv : f - hv);
        const int m = rot_inter ? (f >> 1) : (first ? f : f - hv);
        float w = acc[fp] * i0;
        if (M == 2) w -= acc[acc_stride + fp] * i1;
        const float cs = rcs[2 * m], sn = rcs[2 * m + 1];
        v = first ? fmaf(w, sn, v * cs) : fmaf(-w, sn, v * cs);
      }
    }
    o[c] = v;
    ss += v * v;
  }
  float r = post;
  if (norm_eps >= 0.f) {
    ss = wave_reduce_sum(ss);
    r = post * out_mult / sqrtf(ss / (float)dv + norm_eps);
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int f = lane + 64 * c;
    if (f < dv) {
      if (dst32) dst32[f] = o[c] * r;
      else stf(dst + f, o[c] * r);
    }
  }
}

DEVINL float ra_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// sigmoid(gate[t, h]) or 1
template <typename T>
DEVINL float ra_gate(const T* __restrict__ gate, int64_t gate_stride, int64_t t,
                     int h) {
  return gate ? ra_sigmoid(ldf(gate + t * gate_stride + h)) : 1.0f;
}

// part layout: [T, H, splits, M, 2 + dv]: running max, denominator, sums
// POOL false: no pooled rows exist, so the value loop has no per-key branch
// and its loads of several keys are in flight together.
template <typename T, int M, int HB, bool VEC, bool POOL>
__global__ __launch_bounds__(256) void row_attention_kernel(
    T* __restrict__ out, float* __restrict__ out32, float* __restrict__ part,
    const float* __restrict__ q,
    const T* __restrict__ cache, const float* __restrict__ pool,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ token_seq, const int* __restrict__ positions, int H,
    int G, int d, int dv, int block_size, int per_page, int window, int P,
    float scale, float softcap, float lam, float norm_eps, float out_mult,
    int splits, int FL, const float* __restrict__ head_bias,
    const T* __restrict__ gate, int64_t gate_stride, int vbase,
    const float* __restrict__ rot_cs, int rot_inter) {
  constexpr int NQ = HB * M;
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t t = blockIdx.x;
  const int rep = H / G;
  const int nhb = (rep + HB - 1) / HB;
  const int g = blockIdx.y / nhb;
  const int r0 = (blockIdx.y % nhb) * HB;  // first head of the group, within g
  const int split = blockIdx.z;
  // vbase: the column where a row's values start (0: the values are the keys)
  const int wkeys = G * M * d;
  const int E = max(wkeys, vbase + G * dv);
  const int kcol = g * M * d, vcol = vbase + g * dv;
  const int dp = (d + 7) & ~7;
  const int dvp = (dv + 3) & ~3;
  // LDS: q [NQ][dp] | per wave: p [NQ][64], row offsets [64] (int64)
  float* qs = lds;
  float* ps = qs + NQ * dp + wave * (NQ * 64 + 128);
  int64_t* rows = reinterpret_cast<int64_t*>(ps + NQ * 64);

  for (int idx = threadIdx.x; idx < NQ * dp; idx += 256) {
    const int n = idx / dp, f = idx % dp;
    const int hh = n / M, m = n % M;
    const int h = g * rep + min(r0 + hh, rep - 1);
    qs[idx] = f < d ? q[((t * H + h) * M + m) * (int64_t)d + f] : 0.f;
  }

  const int b = token_seq ? token_seq[t] : (int)t;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int nb = (POOL && window > 0 && P > 0 && pos - window + 1 >= P) ? (pos - window + 1) / P : 0;
  const int nk = nb + (pos - lo + 1);
  const int* bt = block_tables + (int64_t)b * bt_stride;

  const bool sig = head_bias != nullptr;
  float mx[NQ], l[NQ], acc[NQ][4], hb[NQ];
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    hb[n] = sig ? head_bias[g * rep + min(r0 + n / M, rep - 1)] : 0.f;
    mx[n] = sig ? 0.f : -INFINITY;
    l[n] = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[n][i] = 0.f;
  }
  // value pass geometry: VEC: lane = (key subgroup, 4 features); else a lane
  // owns features lane + 64 c and every lane walks every key
  const int ks = VEC ? lane / FL : 0;
  const int kp = VEC ? 64 / FL : 1;
  const int fl = VEC ? (lane % FL) * 4 : lane;
  __syncthreads();

  const int stride = 64 * RA_WAVES * splits;
  for (int u0 = 64 * (split * RA_WAVES + wave); u0 < nk; u0 += stride) {
    const int u = u0 + lane;
    const bool valid = u < nk;
    int64_t off = 0;
    bool pooled = false;
    float s[NQ];
#pragma unroll
    for (int n = 0; n < NQ; ++n) s[n] = 0.f;
    if (valid) {
      pooled = POOL && u < nb;
      if (pooled) {
        off = ((int64_t)bt[u / per_page] * per_page + u % per_page) * E;
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float sm[HB];
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) sm[hh] = 0.f;
          // queries of map m sit at rows hh * M + m: stride M * dp
          ra_dot<float, HB, VEC>(pool + off + kcol + m * d, qs + m * dp, M * dp,
                                 d, sm);
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) s[hh * M + m] = sm[hh];
        }
      } else {
        const int j = lo + (u - nb);
        off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
#pragma unroll
        for (int m = 0; m < M; ++m) {
          float sm[HB];
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) sm[hh] = 0.f;
          ra_dot<T, HB, VEC>(cache + off + kcol + m * d, qs + m * dp, M * dp, d,
                             sm);
#pragma unroll
          for (int hh = 0; hh < HB; ++hh) s[hh * M + m] = sm[hh];
        }
      }
    }
    float corr[NQ];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
      float sc = s[n] * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
      float p;
      if (sig) {
        p = valid ? ra_sigmoid(sc + hb[n]) : 0.f;
        corr[n] = 1.0f;
      } else {
        if (!valid) sc = -INFINITY;
        const float m_new = fmaxf(mx[n], wave_reduce_max(sc));  // finite: key u0 is valid
        p = valid ? expf(sc - m_new) : 0.f;
        corr[n] = expf(mx[n] - m_new);  // exp(-inf) = 0 on the first tile
        l[n] = l[n] * corr[n] + wave_reduce_sum(p);
        mx[n] = m_new;
      }
      ps[n * 64 + lane] = p;
    }
    rows[lane] = pooled ? -(off + 1) : off;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int n = 0; n < NQ; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[n][i] *= corr[n];
    const int cnt = min(64, nk - u0);
#pragma unroll 8
    for (int jj = ks; jj < cnt; jj += kp) {
      const int64_t r = rows[jj];
      float vv[4];
      if (VEC) {
        if (fl < dv) {
          if (POOL && r < 0) ra_load4<float>(pool + (-r - 1) + vcol + fl, vv);
          else ra_load4<T>(cache + r + vcol + fl, vv);
        } else {
          vv[0] = vv[1] = vv[2] = vv[3] = 0.f;
        }
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int f = fl + 64 * c;
          vv[c] = f < dv ? ((POOL && r < 0) ? pool[(-r - 1) + vcol + f]
                                            : ldf(cache + r + vcol + f))
                         : 0.f;
        }
      }
#pragma unroll
      for (int n = 0; n < NQ; ++n) {
        const float pj = ps[n * 64 + jj];
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[n][i] = fmaf(pj, vv[i], acc[n][i]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (VEC) {
    // key subgroups of the wave add up; afterwards subgroup 0 holds the sums
    for (int o = FL; o < 64; o <<= 1) {
#pragma unroll
      for (int n = 0; n < NQ; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[n][i] += __shfl_xor(acc[n][i], o, 64);
    }
  }

  // ---- merge the 4 waves: common max, rescale, add up through LDS -------------
  __syncthreads();  // q and the per-wave regions are free from here on
  float* wm = lds;                      // [4][NQ]
  float* wl = wm + RA_WAVES * NQ;       // [4][NQ]
  float* oacc = wl + RA_WAVES * NQ;     // [NQ][dvp]
  if (lane == 0) {
#pragma unroll
    for (int n = 0; n < NQ; ++n) wm[wave * NQ + n] = mx[n];
  }
  __syncthreads();
  float sc_w[NQ];
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    float x = wm[n];
    for (int w = 1; w < RA_WAVES; ++w) x = fmaxf(x, wm[w * NQ + n]);
    sc_w[n] = (mx[n] == -INFINITY) ? 0.f : expf(mx[n] - x);
  }
  if (lane == 0) {
#pragma unroll
    for (int n = 0; n < NQ; ++n) wl[wave * NQ + n] = l[n] * sc_w[n];
  }
  for (int w = 0; w < RA_WAVES; ++w) {
    if (wave == w && ks == 0) {
#pragma unroll
      for (int n = 0; n < NQ; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int f = VEC ? fl + i : fl + 64 * i;
          if (f < dv) {
            float* dst = oacc + n * dvp + f;
            const float v = acc[n][i] * sc_w[n];
            *dst = (w == 0) ? v : *dst + v;
          }
        }
    }
    __syncthreads();
  }
  // one wave per head of the group
  for (int hh = wave; hh < HB; hh += RA_WAVES) {
    if (r0 + hh >= rep) continue;
    const int h = g * rep + r0 + hh;
    float lg[M], mg[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int n = hh * M + m;
      float a = 0.f, x = wm[n];
      for (int w = 0; w < RA_WAVES; ++w) a += wl[w * NQ + n];
      for (int w = 1; w < RA_WAVES; ++w) x = fmaxf(x, wm[w * NQ + n]);
      lg[m] = sig ? 1.0f : a;
      mg[m] = x;
    }
    if (splits == 1) {
      ra_epilogue<T, M>(out + (t * H + h) * (int64_t)dv,
                        out32 ? out32 + (t * H + h) * (int64_t)dv : nullptr,
                        oacc + hh * M * dvp, dvp,
                        lg, dv, lam, norm_eps, out_mult,
                        ra_gate<T>(gate, gate_stride, t, h),
                        rot_cs ? rot_cs + t * dv : nullptr, rot_inter);
    } else {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float* pr = part + ((((t * H + h) * (int64_t)splits + split) * M + m) * (dv + 2));
        for (int f = lane; f < dv; f += 64) pr[2 + f] = oacc[(hh * M + m) * dvp + f];
        if (lane == 0) {
          pr[0] = mg[m];
          pr[1] = lg[m];
        }
      }
    }
  }
}

// one wave per (token, head): joins `splits` (at most 64) partial results, then
// the epilogue. Lane s weighs split s once; every lane then adds up its value
// features over the splits.
template <typename T, int M>
__global__ __launch_bounds__(64) void row_attention_reduce_kernel(
    T* __restrict__ out, float* __restrict__ out32,
    const float* __restrict__ part, int dv, int splits,
    float lam, float norm_eps, float out_mult, int H, int sig,
    const T* __restrict__ gate, int64_t gate_stride,
    const float* __restrict__ rot_cs, int rot_inter) {
  extern __shared__ float lds[];  // [M][dvp] sums | [M][64] weights
  const int64_t th = blockIdx.x;
  const int lane = threadIdx.x;
  const int dvp = (dv + 3) & ~3;
  float* wts = lds + M * dvp;
  const int64_t step = (int64_t)M * (dv + 2);
  float lg[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const float* pr = part + (th * splits * M + m) * (int64_t)(dv + 2);
    const float ms = lane < splits ? pr[lane * step] : -INFINITY;
    const float ls = lane < splits ? pr[lane * step + 1] : 0.f;
    const float mg = wave_reduce_max(ms);
    const float w = (ms == -INFINITY) ? 0.f : expf(ms - mg);
    lg[m] = wave_reduce_sum(ls * w);
    if (sig) lg[m] = 1.0f;  // sigmoid weights: the shares' sums add up as they are
    wts[m * 64 + lane] = w;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int m = 0; m < M; ++m) {
    const float* pr = part + (th * splits * M + m) * (int64_t)(dv + 2) + 2;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int s = 0; s < splits; ++s) {
      const float w = wts[m * 64 + s];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int f = lane + 64 * c;
        if (f < dv) v[c] = fmaf(w, pr[s * step + f], v[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int f = lane + 64 * c;
      if (f < dv) lds[m * dvp + f] = v[c];
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  ra_epilogue<T, M>(out + th * (int64_t)dv,
                    out32 ? out32 + th * (int64_t)dv : nullptr, lds, dvp, lg,
                    dv, lam, norm_eps,
                    out_mult, ra_gate<T>(gate, gate_stride, th / H, (int)(th % H)),
                    rot_cs ? rot_cs + (th / H) * dv : nullptr, rot_inter);
}

struct RaArgs {
  void* out;
  float* out32;
  float* part;
  const float* q;
  const void* cache;
  const float* pool;
  const int* block_tables;
  int bt_stride;
  const int* token_seq;
  const int* positions;
  int T_, H, G, d, dv, block_size, per_page, window, P;
  float scale, softcap, lam, norm_eps, out_mult;
  int splits;
  const float* head_bias;
  const void* gate;
  int64_t gate_stride;
  int vbase;
  const float* rot_cs;
  int rot_inter;
  hipStream_t stream;
};

template <typename T, int M, int HB>
static void launch_ra_hb(const RaArgs& a) {
  constexpr int NQ = HB * M;
  const int rep = a.H / a.G;
  const int nhb = (rep + HB - 1) / HB;
  const int dp = (a.d + 7) & ~7, dvp = (a.dv + 3) & ~3;
  const size_t run = (size_t)NQ * dp + RA_WAVES * (NQ * 64 + 128);
  const size_t merge = 2 * RA_WAVES * NQ + (size_t)NQ * dvp;
  const size_t shm = sizeof(float) * (run > merge ? run : merge);
  const dim3 grid(a.T_, a.G * nhb, a.splits);
  // 16-byte key loads and 8/16-byte value loads need aligned columns
  const bool vec = (a.d % 8 == 0) && (a.dv % 8 == 0);
  int FL = 1;
  while (FL * 4 < a.dv) FL <<= 1;  // dv <= 256 -> FL <= 64
#define RA_CALL(V, PL)                                                        \
  hipLaunchKernelGGL((row_attention_kernel<T, M, HB, V, PL>), grid, dim3(256), shm, \
                     a.stream, (T*)a.out, a.out32, a.part, a.q,               \
                     (const T*)a.cache,                                       \
                     a.pool, a.block_tables, a.bt_stride, a.token_seq,        \
                     a.positions, a.H, a.G, a.d, a.dv, a.block_size,          \
                     a.per_page, a.window, a.P, a.scale, a.softcap, a.lam,    \
                     a.norm_eps, a.out_mult, a.splits, FL, a.head_bias,       \
                     (const T*)a.gate, a.gate_stride, a.vbase, a.rot_cs,      \
                     a.rot_inter)
  const bool pooled = a.pool != nullptr && a.window > 0 && a.P > 0;
  if (vec) {
    if (pooled) RA_CALL(true, true);
    else RA_CALL(true, false);
  } else {
    if (pooled) RA_CALL(false, true);
    else RA_CALL(false, false);
  }
#undef RA_CALL
  if (a.splits > 1)
    hipLaunchKernelGGL((row_attention_reduce_kernel<T, M>),
                       dim3(a.T_ * a.H), dim3(64), sizeof(float) * M * (dvp + 64),
                       a.stream, (T*)a.out, a.out32, a.part, a.dv, a.splits,
                       a.lam,
                       a.norm_eps, a.out_mult, a.H, a.head_bias != nullptr,
                       (const T*)a.gate, a.gate_stride, a.rot_cs, a.rot_inter);
}

template <typename T, int M>
static void launch_ra_m(const RaArgs& a) {
  const int rep = a.H / a.G;
  if (rep >= 4) launch_ra_hb<T, M, 4>(a);
  else if (rep >= 2) launch_ra_hb<T, M, 2>(a);
  else launch_ra_hb<T, M, 1>(a);
}

// heads per workgroup for a given group size (the host sizes `splits` with it)
extern "C" int row_attention_heads_per_group(int rep) {
  return rep >= 4 ? 4 : (rep >= 2 ? 2 : 1);
}

extern "C" void launch_row_attention(
    void* out, float* out32, float* part, const float* q, const void* cache, const float* pool,
    const int* block_tables, int bt_stride, const int* token_seq,
    const int* positions, int T_, int H, int G, int M, int d, int dv,
    int block_size, int per_page, int window, int P, float scale, float softcap,
    float lam, float norm_eps, float out_mult, int splits,
    const float* head_bias, const void* gate, int64_t gate_stride, int vbase,
    const float* rot_cs, int rot_inter, int kind, hipStream_t stream) {
  if (T_ == 0) return;
  const RaArgs a{out, out32, part, q, cache, pool, block_tables, bt_stride, token_seq,
                 positions, T_, H, G, d, dv, block_size, per_page, window, P,
                 scale, softcap, lam, norm_eps, out_mult, splits, head_bias,
                 gate, gate_stride, vbase, rot_cs, rot_inter, stream};
  if (kind == 0) {
    if (M == 1) launch_ra_m<bf16_t, 1>(a);
    else launch_ra_m<bf16_t, 2>(a);
  } else {
    if (M == 1) launch_ra_m<float, 1>(a);
    else launch_ra_m<float, 2>(a);
  }
}
