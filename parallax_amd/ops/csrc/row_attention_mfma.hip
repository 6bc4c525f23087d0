// Prompt-portion path of the row-cache attention on the fp32 matrix cores.
//
// Same arithmetic as row_attention.hip (fp32 scores, soft cap, softmax and
// value sums over paged [keys | values] rows, pooled blocks beyond a sliding
// window, one or two score maps per head), tiled for portions of many tokens:
// a workgroup takes 32 consecutive tokens of ONE sequence, one kv head and 4
// (head, map) streams of it, one per wave. Per step 32 keys (pooled rows
// first, then tokens) are gathered through the block table, converted to fp32
// and staged in LDS once for the 4 waves. Each wave then computes
//
//     S^T (32 keys x 32 queries) = K_tile (32 x D) . Q^T (D x 32)
//
// with v_mfma_f32_32x32x2_f32 (its 32 queries' features stay in registers for
// the whole kernel). In the accumulator layout a lane holds 16 keys of ONE
// query (column lane % 32; rows 8 i + 4 (lane / 32) + j), so mask, soft cap,
// running max and sum are in-lane work plus one exchange with lane ^ 32, and
// the softmax weights are already laid out as the B operand of
//
//     O^T (DV x 32 queries) += V_tile^T (DV x 32 keys) . P^T (32 keys x 32 queries)
//
// when step (i, j) of that product contracts over the key pair {8 i + j,
// 8 i + 4 + j}: no data moves between the two products. The contraction order
// of the first product is permuted likewise (lane half h walks features
// h D/2 ...) so that a lane reads its key features from LDS in 16-byte pieces.
// Key and value widths are padded with zeros to D and DV (template sizes).
//
// The epilogue (a1 - lam a2 for two maps, exchanged through LDS; optional RMS
// norm over the value width; division by the softmax sum; optional sigmoid
// gate per (token, head)) works on columns, i.e. per lane pair, too.
//
// SIG instantiations replace the softmax by sigmoid(score + head_bias[h])
// weights that are not normalised over the keys: no running maximum, no
// rescaling of the accumulators, masked keys weigh 0.
#include <cstdlib>
#include <type_traits>

#include "seq_common.h"

typedef float f32x16v __attribute__((ext_vector_type(16)));

#define RM_Q 32     // queries per workgroup
#define RM_K 32     // keys per step
#define RM_PAD 4    // LDS row padding (floats)

template <typename T>
DEVINL void rm_load8(const T* p, float* v);
template <>
DEVINL void rm_load8<bf16_t>(const bf16_t* p, float* v) {
  const bf16x8 raw = load_bf16x8(p);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = bf16x8_get(raw, i);
}
template <>
DEVINL void rm_load8<float>(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// 8 cache elements as they are loaded (converted only when they go to LDS, so
// that a prefetched tile costs few registers while the loads are in flight)
template <typename T>
struct rm_raw8;
template <>
struct rm_raw8<bf16_t> {
  int4 v;
  DEVINL void fetch(const bf16_t* p) { v = *reinterpret_cast<const int4*>(p); }
  DEVINL void zero() { v = make_int4(0, 0, 0, 0); }
  DEVINL void unpack(float* o) const {
    bf16x8 r;
    r.raw = v;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i] = bf16x8_get(r, i);
  }
};
template <>
struct rm_raw8<float> {
  float4 a, b;
  DEVINL void fetch(const float* p) {
    a = *reinterpret_cast<const float4*>(p);
    b = *reinterpret_cast<const float4*>(p + 4);
  }
  DEVINL void zero() { a = b = make_float4(0.f, 0.f, 0.f, 0.f); }
  DEVINL void unpack(float* o) const {
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
};

// tanh through one exponential and one reciprocal (both hardware
// approximations, relative error about 1e-6; +-1 at the ends)
DEVINL float rm_tanh(float x) {
  return 1.0f - 2.0f * __frcp_rn(__expf(2.0f * x) + 1.0f);
}

// sigmoid through the same two hardware approximations
DEVINL float rm_sigmoid(float x) { return __frcp_rn(1.0f + __expf(-x)); }
// once per (token, head): the library exponential
DEVINL float rm_sigmoid_exact(float x) { return 1.0f / (1.0f + expf(-x)); }

// D: padded key width (64 | 128), DVB: 32-wide blocks of the padded value width
template <typename T, int M, int D, int DVB, bool SIG>
__global__ __launch_bounds__(256, 2) void row_attention_prefill_kernel(
    T* __restrict__ out, float* __restrict__ out32, const float* __restrict__ q, const T* __restrict__ cache,
    const float* __restrict__ pool, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ cu, int B,
    const int* __restrict__ positions, int H, int G, int d, int dv,
    int block_size, int per_page, int window, int P, float scale, float softcap,
    float lam, float norm_eps, float out_mult,
    const float* __restrict__ head_bias, const T* __restrict__ gate,
    int64_t gate_stride, int vbase, const float* __restrict__ rot_cs,
    int rot_inter) {
  constexpr int DV = DVB * 32;
  constexpr int KS = D + RM_PAD, VS = DV + RM_PAD;
  constexpr int HW = 4 / M;  // heads per workgroup
  extern __shared__ float lds[];
  float* Ks = lds;                    // [M][32][KS]
  float* Vs = lds + M * RM_K * KS;    // [32][VS]

  // ---- which 32 tokens: tiles never straddle two sequences ---------------------
  // Workgroups start in index order and a sequence's later tiles see more
  // keys, so the tiles are dealt from the back: the longest run first and
  // the short ones fill the tail of the launch.
  int tile = gridDim.x - 1 - blockIdx.x, b = 0;
  for (; b < B; ++b) {
    const int nt = (cu[b + 1] - cu[b] + RM_Q - 1) / RM_Q;
    if (tile < nt) break;
    tile -= nt;
  }
  if (b == B) return;
  const int t0 = cu[b] + tile * RM_Q;
  const int nq = min(RM_Q, cu[b + 1] - t0);
  const int p0 = positions[t0], p_last = p0 + nq - 1;
  const int* bt = block_tables + (int64_t)b * bt_stride;

  const int rep = H / G;
  const int nhw = (rep + HW - 1) / HW;
  const int g = blockIdx.y / nhw;
  const int r0 = (blockIdx.y % nhw) * HW;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int half = lane >> 5, col = lane & 31;
  const int hh = wave / M, m = wave % M;   // this wave's stream
  const bool stream_on = r0 + hh < rep;
  const int h = g * rep + min(r0 + hh, rep - 1);
  // vbase: the column where a row's values start (0: the values are the keys)
  const int wkeys = G * M * d;
  const int E = max(wkeys, vbase + G * dv);
  const int kcol = g * M * d, vcol = vbase + g * dv;

  // key list of the tile: pooled blocks [0, nb) then tokens [lo, p_last]
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int nb = (window > 0 && P > 0 && p_last - window + 1 >= P) ? (p_last - window + 1) / P : 0;
  const int nk = nb + (p_last - lo + 1);

  // the lane's query (column col): features half * D/2 + s, s < D/2
  float qr[D / 2];
  {
    const bool on = stream_on && col < nq;
    const float* src = q + (((int64_t)(t0 + min(col, nq - 1)) * H + h) * M + m) * d;
#pragma unroll
    for (int s = 0; s < D / 2; ++s) {
      const int f = half * (D / 2) + s;
      qr[s] = (on && f < d) ? src[f] : 0.f;
    }
  }
  const int pq = p0 + col;
  const bool qvalid = col < nq;

  f32x16v acc[DVB];
#pragma unroll
  for (int k = 0; k < DVB; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  float mx = -INFINITY, l = 0.f;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const float hbias = SIG ? head_bias[h] : 0.f;

  // staging role: 8 threads per key row, 8 features each at a time
  const int srow = threadIdx.x >> 3, ssub = threadIdx.x & 7;

  // steps whose 32 keys are all token rows (every step after the pooled rows)
  // are prefetched: their global loads are issued before the previous step's
  // products and land in LDS after them
  constexpr int KC = D / 64, VC = (DV + 63) / 64;
  rm_raw8<T> kraw[M][KC], vraw[VC];
  auto fetch = [&](int u0) {
    const int u = u0 + srow;
    const bool on = u < nk;
    int64_t off = 0;
    if (on) {
      const int j = lo + (u - nb);
      off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
    }
#pragma unroll
    for (int mm = 0; mm < M; ++mm)
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const int f = ssub * 8 + 64 * c;
        if (on && f < d) kraw[mm][c].fetch(cache + off + kcol + mm * d + f);
        else kraw[mm][c].zero();
      }
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int f = ssub * 8 + 64 * c;
      if (on && f < dv) vraw[c].fetch(cache + off + vcol + f);
      else vraw[c].zero();
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int mm = 0; mm < M; ++mm)
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        float v[8];
        kraw[mm][c].unpack(v);
        float* dst = Ks + (mm * RM_K + srow) * KS + ssub * 8 + 64 * c;
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
      }
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int f = ssub * 8 + 64 * c;
      if (f < DV) {
        float v[8];
        vraw[c].unpack(v);
        float* dst = Vs + srow * VS + f;
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
      }
    }
  };

  // the widest value tile leaves no registers for a tile in flight
  constexpr bool PREFETCH = DVB <= 4;
  bool fetched = false;
  for (int u0 = 0; u0 < nk; u0 += RM_K) {
    __syncthreads();  // the previous step's reads are done
    if (u0 >= nb) {
      if (!fetched) fetch(u0);
      stash();
    } else {
      const int u = u0 + srow;
      const bool on = u < nk;
      const bool pooled = on && u < nb;
      int64_t off = 0;
      if (pooled) {
        off = ((int64_t)bt[u / per_page] * per_page + u % per_page) * E;
      } else if (on) {
        const int j = lo + (u - nb);
        off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
      }
#pragma unroll
      for (int mm = 0; mm < M; ++mm)
#pragma unroll
        for (int c = 0; c < D / 64; ++c) {
          const int f = ssub * 8 + 64 * c;
          float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if (on && f < d) {
            if (pooled) rm_load8<float>(pool + off + kcol + mm * d + f, v);
            else rm_load8<T>(cache + off + kcol + mm * d + f, v);
          }
          float* dst = Ks + (mm * RM_K + srow) * KS + f;
          *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
#pragma unroll
      for (int c = 0; c < (DV + 63) / 64; ++c) {
        const int f = ssub * 8 + 64 * c;
        if (f < DV) {
          float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          if (on && f < dv) {
            if (pooled) rm_load8<float>(pool + off + vcol + f, v);
            else rm_load8<T>(cache + off + vcol + f, v);
          }
          float* dst = Vs + srow * VS + f;
          *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
      }
    }
    __syncthreads();
    fetched = PREFETCH && u0 + RM_K < nk && u0 + RM_K >= nb;
    if (fetched) fetch(u0 + RM_K);

    // ---- S^T = K_tile . Q^T ---------------------------------------------------
    f32x16v S;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = 0.f;
    {
      const float* krow = Ks + (m * RM_K + col) * KS + half * (D / 2);
#pragma unroll
      for (int s = 0; s < D / 2; s += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(krow + s);
        S = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.x, qr[s], S, 0, 0, 0);
        S = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.y, qr[s + 1], S, 0, 0, 0);
        S = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.z, qr[s + 2], S, 0, 0, 0);
        S = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.w, qr[s + 3], S, 0, 0, 0);
      }
    }
    // ---- mask, soft cap, online softmax (column = query, 16 keys in-lane) -------
    // a step whose 32 keys are tokens that every one of the 32 queries sees
    // needs no mask (most steps of a long portion)
    const int jt0 = lo + (u0 - nb);
    const bool interior = nq == RM_Q && u0 >= nb && u0 + RM_K <= nk &&
                          jt0 + RM_K - 1 <= p0 && (window == 0 || p_last - jt0 < window);
    float tmax = -INFINITY;
    float corr = 1.f;
    if (SIG) {
      if (interior) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          float sc = S[i] * scale;
          if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
          S[i] = rm_sigmoid(sc + hbias);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int u = u0 + 8 * i + 4 * half + j;
            bool vis;
            if (u < nb) {
              vis = u * P + P - 1 <= pq - window;
            } else {
              const int jt = lo + (u - nb);
              vis = jt <= pq && (window == 0 || pq - jt < window);
            }
            float sc = S[4 * i + j] * scale;
            if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
            S[4 * i + j] = (vis && qvalid && u < nk) ? rm_sigmoid(sc + hbias) : 0.f;
          }
      }
    } else {
    if (interior) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        float sc = S[i] * scale;
        if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
        S[i] = sc;
        tmax = fmaxf(tmax, sc);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = u0 + 8 * i + 4 * half + j;
          bool vis;
          if (u < nb) {
            vis = u * P + P - 1 <= pq - window;
          } else {
            const int jt = lo + (u - nb);
            vis = jt <= pq && (window == 0 || pq - jt < window);
          }
          float sc = S[4 * i + j] * scale;
          if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
          sc = (vis && qvalid && u < nk) ? sc : -INFINITY;
          S[4 * i + j] = sc;
          tmax = fmaxf(tmax, sc);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(mx, tmax);
    float psum = 0.f;
    if (m_new == -INFINITY) {
#pragma unroll
      for (int i = 0; i < 16; ++i) S[i] = 0.f;
    } else {
      corr = __expf(mx - m_new);  // exp(-inf) = 0 the first time a key is seen
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = __expf(S[i] - m_new);  // exp(-inf) = 0 for masked keys
        S[i] = p;
        psum += p;
      }
    }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    mx = m_new;
    }  // !SIG
    // ---- O^T += V_tile^T . P^T ------------------------------------------------
#pragma unroll
    for (int k = 0; k < DVB; ++k) {
      if (!SIG) {
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[k][i] *= corr;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float a = Vs[(8 * i + 4 * half + j) * VS + 32 * k + col];
          acc[k] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, S[4 * i + j], acc[k], 0, 0, 0);
        }
    }
  }

  // ---- epilogue: lane holds O[query col][feature 32 k + 8 i + 4 half + j] --------
  __syncthreads();  // staging area free
  const float inv = SIG ? (qvalid ? 1.0f : 0.f)
                        : ((qvalid && l > 0.f) ? 1.0f / l : 0.f);
  if (M == 2) {
    // the second map's wave parks a2 (times lam) in LDS for its head's first wave
    float* X = lds + hh * (DV * (RM_Q + 1));
    if (m == 1) {
#pragma unroll
      for (int k = 0; k < DVB; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
          X[f * (RM_Q + 1) + col] = acc[k][i] * inv * lam;
        }
    }
    __syncthreads();
    if (m == 1) return;
#pragma unroll
    for (int k = 0; k < DVB; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
        acc[k][i] = acc[k][i] * inv - X[f * (RM_Q + 1) + col];
      }
  } else {
#pragma unroll
    for (int k = 0; k < DVB; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[k][i] *= inv;
  }
  if (rot_cs != nullptr) {
    // the result turns BACK by the query's angle: rot_cs holds [dv / 2][2]
    // cos, sin per token; pair (u, w) -> (u cos + w sin, w cos - u sin).
    // Neighbouring pairs sit in one lane (i, i + 1); halves pair block k with
    // block k + DVB / 2 when the value width fills the tile (the host sends
    // other widths through a separate pass).
    const float* rc = rot_cs + (int64_t)(t0 + min(col, nq - 1)) * dv;
    if (rot_inter) {
#pragma unroll
      for (int k = 0; k < DVB; ++k)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
          if (f < dv) {
            const float2 cs = *reinterpret_cast<const float2*>(rc + f);
            const float u = acc[k][i], w = acc[k][i + 1];
            acc[k][i] = fmaf(w, cs.y, u * cs.x);
            acc[k][i + 1] = fmaf(-u, cs.y, w * cs.x);
          }
        }
    } else {
#pragma unroll
      for (int k = 0; k < DVB / 2; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
          const float2 cs = *reinterpret_cast<const float2*>(rc + 2 * f);
          const float u = acc[k][i], w = acc[k + DVB / 2][i];
          acc[k][i] = fmaf(w, cs.y, u * cs.x);
          acc[k + DVB / 2][i] = fmaf(-u, cs.y, w * cs.x);
        }
    }
  }
  float r = 1.0f;
  if (norm_eps >= 0.f) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < DVB; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) ss += acc[k][i] * acc[k][i];
    ss += __shfl_xor(ss, 32, 64);
    r = out_mult / sqrtf(ss / (float)dv + norm_eps);
  }
  if (!stream_on || !qvalid) return;
  if (gate != nullptr)
    r *= rm_sigmoid_exact(ldf(gate + (int64_t)(t0 + col) * gate_stride + h));
  const int64_t o0 = ((int64_t)(t0 + col) * H + h) * dv;
  if (out32 != nullptr) {
#pragma unroll
    for (int k = 0; k < DVB; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
        if (f < dv) out32[o0 + f] = acc[k][i] * r;
      }
    return;
  }
  T* dst = out + o0;
#pragma unroll
  for (int k = 0; k < DVB; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
      if (f < dv) stf(dst + f, acc[k][i] * r);
    }
}

// ---- bf16 cache rows: the same products on the bf16 matrix cores, exactly ----
//
// With bf16 cache rows a key or value element IS a bf16 number, and an fp32
// query element (or key weight) x is exactly the sum of three bf16 numbers:
// its top 8 mantissa bits, the top 8 of what is left, and the rest. So
//     q . k = q_hi . k + q_mid . k + q_lo . k
// holds term by term in fp32 (a product of two bf16 numbers is exact in fp32,
// the sums run in the fp32 accumulator), and likewise sum_j p_j v_j with p
// split. Three v_mfma_f32_32x32x16_bf16 per 16 contracted elements do the
// work of eight v_mfma_f32_32x32x2_f32 at one sixteenth of their cost each.
// Same tiling, masks, softmax, accumulator layout and epilogue as the kernel
// above; one score map, no pooled rows. K rows go to LDS as they are (no
// conversion), V goes in transposed ([feature][key]) so that a lane reads the
// 8 keys of its slots in two 8-byte pieces.
//
// Operand slots: lane (col = lane % 32, half = lane / 32) supplies 8 of the
// 16 contracted elements of an instruction. Both operands put the SAME
// element into the same slot, which is all the instruction asks for:
//   scores, step s:  slot e <-> feature 16 s + 8 half + e
//   values, step s:  slot e <-> key 16 s + 4 half + e (e < 4),
//                               key 16 s + 8 + 4 half + e - 4 (e >= 4)
// (the keys whose weights the lane's score registers 8 s .. 8 s + 7 hold).

DEVINL void rb_split3(float x, short& hi, short& mid, short& lo) {
  const uint32_t b0 = __float_as_uint(x) & 0xffff0000u;
  const float r1 = x - __uint_as_float(b0);          // exact
  const uint32_t b1 = __float_as_uint(r1) & 0xffff0000u;
  const float r2 = r1 - __uint_as_float(b1);         // exact, at most 8 bits left
  hi = (short)(b0 >> 16);
  mid = (short)(b1 >> 16);
  lo = (short)(__float_as_uint(r2) >> 16);
}

#define RB_KPAD 8   // bf16 elements of padding per K row (16 bytes)
#define RB_VS 36    // bf16 elements per transposed V row: 32 keys + 4 (72 bytes)

template <int D, int DVB, bool SIG>
__global__ __launch_bounds__(256, 2) void row_attention_prefill_bf16_kernel(
    bf16_t* __restrict__ out, float* __restrict__ out32, const float* __restrict__ q,
    const bf16_t* __restrict__ cache, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ cu, int B,
    const int* __restrict__ positions, int H, int G, int d, int dv,
    int block_size, int window, float scale, float softcap, float norm_eps,
    float out_mult, const float* __restrict__ head_bias,
    const bf16_t* __restrict__ gate, int64_t gate_stride, int vbase,
    const float* __restrict__ rot_cs, int rot_inter) {
  constexpr int DV = DVB * 32;
  constexpr int KS = D + RB_KPAD;
  constexpr int HW = 4;  // heads per workgroup
  extern __shared__ float lds[];
  bf16_t* Ks = reinterpret_cast<bf16_t*>(lds);   // [32][KS]
  bf16_t* Vt = Ks + RM_K * KS;                    // [DV][RB_VS]

  int tile = gridDim.x - 1 - blockIdx.x, b = 0;
  for (; b < B; ++b) {
    const int nt = (cu[b + 1] - cu[b] + RM_Q - 1) / RM_Q;
    if (tile < nt) break;
    tile -= nt;
  }
  if (b == B) return;
  const int t0 = cu[b] + tile * RM_Q;
  const int nq = min(RM_Q, cu[b + 1] - t0);
  const int p0 = positions[t0], p_last = p0 + nq - 1;
  const int* bt = block_tables + (int64_t)b * bt_stride;

  const int rep = H / G;
  const int nhw = (rep + HW - 1) / HW;
  const int g = blockIdx.y / nhw;
  const int r0 = (blockIdx.y % nhw) * HW;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int half = lane >> 5, col = lane & 31;
  const bool stream_on = r0 + wave < rep;
  const int h = g * rep + min(r0 + wave, rep - 1);
  const int wkeys = G * d;
  const int E = max(wkeys, vbase + G * dv);
  const int kcol = g * d, vcol = vbase + g * dv;

  const int lo = window > 0 ? max(0, p0 - window + 1) : 0;
  const int nk = p_last - lo + 1;

  // the lane's query (column col) in three bf16 parts, slot order
  bf16x8v qh[D / 16], qm[D / 16], ql[D / 16];
  {
    const bool on = stream_on && col < nq;
    const float* src = q + ((int64_t)(t0 + min(col, nq - 1)) * H + h) * d;
#pragma unroll
    for (int s = 0; s < D / 16; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int f = 16 * s + 8 * half + e;
        const float x = (on && f < d) ? src[f] : 0.f;
        short a, m, l;
        rb_split3(x, a, m, l);
        qh[s][e] = a;
        qm[s][e] = m;
        ql[s][e] = l;
      }
  }
  const int pq = p0 + col;
  const bool qvalid = col < nq;

  f32x16v acc[DVB];
#pragma unroll
  for (int k = 0; k < DVB; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
  float mx = -INFINITY, l = 0.f;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const float hbias = SIG ? head_bias[h] : 0.f;

  // staging role: 8 threads per key row, 8 elements each at a time
  const int srow = threadIdx.x >> 3, ssub = threadIdx.x & 7;
  constexpr int KC = D / 64, VC = (DV + 63) / 64;
  int4 kraw[KC], vraw[VC];
  auto fetch = [&](int u0) {
    const int u = u0 + srow;
    const bool on = u < nk;
    int64_t off = 0;
    if (on) {
      const int j = lo + u;
      off = ((int64_t)bt[j / block_size] * block_size + j % block_size) * E;
    }
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int f = ssub * 8 + 64 * c;
      kraw[c] = (on && f < d) ? *reinterpret_cast<const int4*>(cache + off + kcol + f)
                              : make_int4(0, 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int f = ssub * 8 + 64 * c;
      vraw[c] = (on && f < dv) ? *reinterpret_cast<const int4*>(cache + off + vcol + f)
                               : make_int4(0, 0, 0, 0);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int c = 0; c < KC; ++c)
      *reinterpret_cast<int4*>(Ks + srow * KS + ssub * 8 + 64 * c) = kraw[c];
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int f = ssub * 8 + 64 * c;
      if (f < DV) {
        const uint32_t w[4] = {(uint32_t)vraw[c].x, (uint32_t)vraw[c].y,
                               (uint32_t)vraw[c].z, (uint32_t)vraw[c].w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
          Vt[(f + e) * RB_VS + srow] =
              (bf16_t)((e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu));
      }
    }
  };

  bool fetched = false;
  for (int u0 = 0; u0 < nk; u0 += RM_K) {
    __syncthreads();  // the previous step's reads are done
    if (!fetched) fetch(u0);
    stash();
    __syncthreads();
    fetched = u0 + RM_K < nk;
    if (fetched) fetch(u0 + RM_K);

    // ---- S^T = K_tile . Q^T, three parts of q ------------------------------------
    f32x16v S;
#pragma unroll
    for (int i = 0; i < 16; ++i) S[i] = 0.f;
    {
      const bf16_t* krow = Ks + col * KS + 8 * half;
#pragma unroll
      for (int s = 0; s < D / 16; ++s) {
        const bf16x8v a = *reinterpret_cast<const bf16x8v*>(krow + 16 * s);
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qh[s], S, 0, 0, 0);
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qm[s], S, 0, 0, 0);
        S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, ql[s], S, 0, 0, 0);
      }
    }
    // ---- mask, soft cap, weights (column = query, 16 keys in-lane) ---------------
    const int jt0 = lo + u0;
    const bool interior = nq == RM_Q && u0 + RM_K <= nk && jt0 + RM_K - 1 <= p0 &&
                          (window == 0 || p_last - jt0 < window);
    float corr = 1.f;
    if (SIG) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = u0 + 8 * i + 4 * half + j;
          const int jt = lo + u;
          const bool vis = interior || (jt <= pq && (window == 0 || pq - jt < window) &&
                                        qvalid && u < nk);
          float sc = S[4 * i + j] * scale;
          if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
          S[4 * i + j] = vis ? rm_sigmoid(sc + hbias) : 0.f;
        }
    } else {
      float tmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int u = u0 + 8 * i + 4 * half + j;
          const int jt = lo + u;
          const bool vis = interior || (jt <= pq && (window == 0 || pq - jt < window) &&
                                        qvalid && u < nk);
          float sc = S[4 * i + j] * scale;
          if (softcap > 0.f) sc = softcap * rm_tanh(sc * inv_cap);
          sc = vis ? sc : -INFINITY;
          S[4 * i + j] = sc;
          tmax = fmaxf(tmax, sc);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(mx, tmax);
      float psum = 0.f;
      if (m_new == -INFINITY) {
#pragma unroll
        for (int i = 0; i < 16; ++i) S[i] = 0.f;
      } else {
        corr = __expf(mx - m_new);  // exp(-inf) = 0 the first time a key is seen
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float p = __expf(S[i] - m_new);  // exp(-inf) = 0 for masked keys
          S[i] = p;
          psum += p;
        }
      }
      psum += __shfl_xor(psum, 32, 64);
      l = l * corr + psum;
      mx = m_new;
#pragma unroll
      for (int k = 0; k < DVB; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[k][i] *= corr;
    }
    // ---- O^T += V_tile^T . P^T, three parts of p ---------------------------------
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      bf16x8v ph, pm, pl;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        short a, m, lw;
        rb_split3(S[8 * s + e], a, m, lw);
        ph[e] = a;
        pm[e] = m;
        pl[e] = lw;
      }
#pragma unroll
      for (int k = 0; k < DVB; ++k) {
        const bf16_t* vrow = Vt + (32 * k + col) * RB_VS + 16 * s + 4 * half;
        const int2 v0 = *reinterpret_cast<const int2*>(vrow);
        const int2 v1 = *reinterpret_cast<const int2*>(vrow + 8);
        const int4 packed = make_int4(v0.x, v0.y, v1.x, v1.y);
        const bf16x8v a = *reinterpret_cast<const bf16x8v*>(&packed);
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, ph, acc[k], 0, 0, 0);
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pm, acc[k], 0, 0, 0);
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pl, acc[k], 0, 0, 0);
      }
    }
  }

  // ---- epilogue: lane holds O[query col][feature 32 k + 8 i + 4 half + j] --------
  const float inv = SIG ? (qvalid ? 1.0f : 0.f)
                        : ((qvalid && l > 0.f) ? 1.0f / l : 0.f);
#pragma unroll
  for (int k = 0; k < DVB; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[k][i] *= inv;
  if (rot_cs != nullptr) {
    const float* rc = rot_cs + (int64_t)(t0 + min(col, nq - 1)) * dv;
    if (rot_inter) {
#pragma unroll
      for (int k = 0; k < DVB; ++k)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
          if (f < dv) {
            const float2 cs = *reinterpret_cast<const float2*>(rc + f);
            const float u = acc[k][i], w = acc[k][i + 1];
            acc[k][i] = fmaf(w, cs.y, u * cs.x);
            acc[k][i + 1] = fmaf(-u, cs.y, w * cs.x);
          }
        }
    } else {
#pragma unroll
      for (int k = 0; k < DVB / 2; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
          const float2 cs = *reinterpret_cast<const float2*>(rc + 2 * f);
          const float u = acc[k][i], w = acc[k + DVB / 2][i];
          acc[k][i] = fmaf(w, cs.y, u * cs.x);
          acc[k + DVB / 2][i] = fmaf(-u, cs.y, w * cs.x);
        }
    }
  }
  float r = 1.0f;
  if (norm_eps >= 0.f) {
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < DVB; ++k)
#pragma unroll
      for (int i = 0; i < 16; ++i) ss += acc[k][i] * acc[k][i];
    ss += __shfl_xor(ss, 32, 64);
    r = out_mult / sqrtf(ss / (float)dv + norm_eps);
  }
  if (!stream_on || !qvalid) return;
  if (gate != nullptr)
    r *= rm_sigmoid_exact(ldf(gate + (int64_t)(t0 + col) * gate_stride + h));
  const int64_t o0 = ((int64_t)(t0 + col) * H + h) * dv;
#pragma unroll
  for (int k = 0; k < DVB; ++k)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int f = 32 * k + 8 * (i >> 2) + 4 * half + (i & 3);
      if (f < dv) {
        if (out32 != nullptr) out32[o0 + f] = acc[k][i] * r;
        else stf(out + o0 + f, acc[k][i] * r);
      }
    }
}

struct RmArgs {
  void* out;
  float* out32;
  const float* q;
  const void* cache;
  const float* pool;
  const int* block_tables;
  int bt_stride;
  const int* cu;
  int B;
  const int* positions;
  int tiles, H, G, d, dv, block_size, per_page, window, P;
  float scale, softcap, lam, norm_eps, out_mult;
  const float* head_bias;
  const void* gate;
  int64_t gate_stride;
  int vbase;
  const float* rot_cs;
  int rot_inter;
  hipStream_t stream;
};

// PARALLAX_ROW_ATTN_FP32=1 keeps bf16 rows on the fp32 matrix cores too
static bool rm_split_bf16() {
  static const bool on = []() {
    const char* e = getenv("PARALLAX_ROW_ATTN_FP32");
    return !(e && e[0] == '1');
  }();
  return on;
}

template <int D, int DVB, bool SIG>
static void launch_rb(const RmArgs& a) {
  constexpr int DV = DVB * 32;
  const int rep = a.H / a.G;
  const size_t shm = sizeof(bf16_t) * ((size_t)RM_K * (D + RB_KPAD) + (size_t)DV * RB_VS);
  const dim3 grid(a.tiles, a.G * ((rep + 3) / 4));
  hipLaunchKernelGGL((row_attention_prefill_bf16_kernel<D, DVB, SIG>), grid,
                     dim3(256), shm, a.stream, (bf16_t*)a.out, a.out32, a.q,
                     (const bf16_t*)a.cache, a.block_tables, a.bt_stride, a.cu,
                     a.B, a.positions, a.H, a.G, a.d, a.dv, a.block_size,
                     a.window, a.scale, a.softcap, a.norm_eps, a.out_mult,
                     a.head_bias, (const bf16_t*)a.gate, a.gate_stride, a.vbase,
                     a.rot_cs, a.rot_inter);
}

template <typename T, int M, int D, int DVB, bool SIG>
static void launch_rm_k(const RmArgs& a) {
  constexpr int DV = DVB * 32;
  // bf16 rows, one score map, no pooled rows, value tiles up to 128: the
  // exact three-part products on the bf16 matrix cores
  if constexpr (std::is_same<T, bf16_t>::value && M == 1 && DVB <= 4) {
    if (a.P == 0 && rm_split_bf16()) {
      launch_rb<D, DVB, SIG>(a);
      return;
    }
  }
  const int rep = a.H / a.G;
  const int hw = 4 / M;
  const size_t stage = (size_t)M * RM_K * (D + RM_PAD) + RM_K * (DV + RM_PAD);
  const size_t xchg = M == 2 ? (size_t)hw * DV * (RM_Q + 1) : 0;
  const size_t shm = sizeof(float) * (stage > xchg ? stage : xchg);
  const dim3 grid(a.tiles, a.G * ((rep + hw - 1) / hw));
  if (shm > 64 * 1024) {
    // gfx950 has 160 KB of LDS per CU; more than 64 KB per workgroup is opt-in
    static bool raised = false;
    if (!raised) {
      (void)hipFuncSetAttribute(
          reinterpret_cast<const void*>(&row_attention_prefill_kernel<T, M, D, DVB, SIG>),
          hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
      raised = true;
    }
  }
  hipLaunchKernelGGL((row_attention_prefill_kernel<T, M, D, DVB, SIG>), grid,
                     dim3(256), shm, a.stream, (T*)a.out, a.out32, a.q,
                     (const T*)a.cache, a.pool, a.block_tables, a.bt_stride,
                     a.cu, a.B, a.positions, a.H, a.G, a.d, a.dv, a.block_size,
                     a.per_page, a.window, a.P, a.scale, a.softcap, a.lam,
                     a.norm_eps, a.out_mult, a.head_bias, (const T*)a.gate,
                     a.gate_stride, a.vbase, a.rot_cs, a.rot_inter);
}

// sigmoid weights come with one score map only
template <typename T, int M, int D, int DVB>
static void launch_rm(const RmArgs& a) {
  if (M == 1 && a.head_bias != nullptr) launch_rm_k<T, 1, D, DVB, true>(a);
  else launch_rm_k<T, M, D, DVB, false>(a);
}

template <typename T, int M, int D>
static void launch_rm_d(const RmArgs& a) {
  if (a.dv <= 64) launch_rm<T, M, D, 2>(a);
  else if (a.dv <= 128) launch_rm<T, M, D, 4>(a);
  else launch_rm<T, M, D, 8>(a);
}

template <typename T, int M>
static void launch_rm_m(const RmArgs& a) {
  if (a.d <= 64) launch_rm_d<T, M, 64>(a);
  else launch_rm_d<T, M, 128>(a);
}

// what the matrix-core path takes: 16-byte aligned columns, widths within the
// template sizes
extern "C" int row_attention_prefill_supported(int d, int dv) {
  return d % 8 == 0 && dv % 8 == 0 && d <= 128 && dv <= 256;
}

// whether the matrix-core kernel can turn its results back in registers:
// neighbouring pairs always; halves when the value width fills its tile
extern "C" int row_attention_prefill_rotates(int dv, int inter) {
  const int tile = dv <= 64 ? 64 : (dv <= 128 ? 128 : 256);
  return inter || dv == tile;
}

// tiles: an upper bound on the number of 32-token tiles (ceil(T / 32) + B)
extern "C" void launch_row_attention_prefill(
    void* out, float* out32, const float* q, const void* cache, const float* pool,
    const int* block_tables, int bt_stride, const int* cu, int B,
    const int* positions, int tiles, int H, int G, int M, int d, int dv,
    int block_size, int per_page, int window, int P, float scale, float softcap,
    float lam, float norm_eps, float out_mult, const float* head_bias,
    const void* gate, int64_t gate_stride, int vbase, const float* rot_cs,
    int rot_inter, int kind, hipStream_t stream) {
  if (tiles == 0) return;
  const RmArgs a{out, out32, q, cache, pool, block_tables, bt_stride, cu, B, positions,
                 tiles, H, G, d, dv, block_size, per_page, window, P, scale,
                 softcap, lam, norm_eps, out_mult, head_bias, gate, gate_stride,
                 vbase, rot_cs, rot_inter, stream};
  if (kind == 0) {
    if (M == 1) launch_rm_m<bf16_t, 1>(a);
    else launch_rm_m<bf16_t, 2>(a);
  } else {
    if (M == 1) launch_rm_m<float, 1>(a);
    else launch_rm_m<float, 2>(a);
  }
}
