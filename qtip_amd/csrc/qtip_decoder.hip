// Single-token decode attention for the end-to-end decode loop: rotary
// embedding of q and k, KV-cache write and attention over the cache in one
// launch (the reference runs these as a dozen framework kernels:
// model/llama.py:264-295 RoPE, model/cache_utils.py:1173-1193 cache update,
// model/llama.py:866-880 scaled-dot-product attention).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qtip_hip.h"
#include "qtip_wht.h"

namespace {

constexpr int kAttnThreads = 1024;
constexpr int kMaxHeadDim = 256;

// Cross-lane exchanges go through qtip_wht::lane_xor (DPP, ds_swizzle, v_permlane32_swap: a few
// cycles each); a generic shuffle is a ds_bpermute with an LDS round trip per step, which these
// latency-bound kernels feel.
__device__ __forceinline__ int lane_xor_i(int v, int b) {
  return __builtin_bit_cast(int, qtip_wht::lane_xor(__builtin_bit_cast(float, v), b));
}
__device__ __forceinline__ float wave_reduce_max(float v) {
#pragma unroll
  for (int b = 5; b >= 0; --b) v = fmaxf(v, qtip_wht::lane_xor(v, b));
  return v;
}
__device__ __forceinline__ float wave_reduce_sum(float v) {
#pragma unroll
  for (int b = 5; b >= 0; --b) v += qtip_wht::lane_xor(v, b);
  return v;
}

// The qkv projection's output transform, for the XF form of the kernel: the new token's
// [q | k | v] vector (n = order * 2^logp2 elements) is
//   post * scale * (H_order (x) H_{2^logp2}) (sum of the in_parts partial sums),
// and a workgroup needs three D-long slices of it.  A slice (table row iK, block b of the
// power-of-two part) is the D-point Walsh-Hadamard transform of
//   u[c] = sum_{jK, b'} (-1)^(bits[jK][iK] + popcount(b & b')) v[(jK * 2^logp2) + b' * D + c],
// n additions per slice instead of a launch of its own for the whole vector.
// XF = 1: q, k and v are slices of one transformed vector [q | k | v] (fused projection; entry 0
// of the arrays below describes it).  XF = 2: three vectors with a transform each (separate
// projections): q of heads * D elements, k and v of kv_heads * D.
struct AttnXf {
  const float* parts[3];
  const float* post[3];
  const uint32_t* had_bits[3];
  size_t part_stride;
  float scale[3];
  int order[3], logp2[3], n[3];
  int in_parts;
};

typedef float float4a __attribute__((ext_vector_type(4)));

// One workgroup per query head and key range.  qkv: [H*D | Hkv*D | Hkv*D] fp16 of the new
// token; k_cache / v_cache: [Hkv][max_len][D] fp16; pos_ptr: position of the
// new token (device memory, so that a recorded graph follows the position).
// nsplit > 1 (long contexts): workgroup blockIdx.z takes the keys
// [z * keys_per_split, (z + 1) * keys_per_split) and leaves its share - the D unnormalised output
// sums, its score maximum and its sum of exponentials - in split_ws[head][z][D + 2] for
// attn_combine_kernel; every workgroup repeats the prologue (transform, rotary embedding), the
// one of range 0 writes the cache.
template <int D, int XF>
__global__ __launch_bounds__(kAttnThreads) void decode_attn_kernel(
    _Float16* __restrict__ out, const _Float16* __restrict__ qkv, _Float16* __restrict__ k_cache,
    _Float16* __restrict__ v_cache, const long* __restrict__ pos_ptr,
    const float* __restrict__ inv_freq, int H, int Hkv, int max_len, const AttnXf X, int nsplit,
    int keys_per_split, float* __restrict__ split_ws) {
  extern __shared__ __align__(16) uint8_t smem[];
  float* q_s = reinterpret_cast<float*>(smem);   // [D] rotated query (as fp16 values)
  float* k_s = q_s + kMaxHeadDim;                // [D] rotated new key
  float* v_s = k_s + kMaxHeadDim;                // [D] new value
  float* red = v_s + kMaxHeadDim;                // [32] reductions
  float* acc = red + 32;                         // [TG][D] partial outputs, TG*D = 8192
  float* p_s = acc + 8192;                       // [max_len] scores / probabilities
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // grid = (query heads per kv head, kv heads): no integer division on the way to the loads
  const int rep = gridDim.x, kvh = blockIdx.y, h = kvh * rep + blockIdx.x;
  const int pos = (int)pos_ptr[0];
  constexpr int half = D >> 1;
  const _Float16* q_in = qkv + (size_t)h * D;
  const _Float16* k_in = qkv + (size_t)H * D + (size_t)kvh * D;
  const _Float16* v_in = qkv + (size_t)(H + Hkv) * D + (size_t)kvh * D;
  _Float16* kc = k_cache + (size_t)kvh * max_len * D;
  _Float16* vc = v_cache + (size_t)kvh * max_len * D;

  // rotary angle of this thread's dimension, requested before anything else: the angle is the fp32
  // product the reference forms; its reduction to a fraction of a turn is done in fp64 (exact to
  // 2^-29 of a turn at position 4096), the hardware cos / sin take turns.  (cosf / sinf with their
  // large-argument paths cost ~0.5 us on this kernel's critical path.)
  _Float16 rc = (_Float16)1.f, rs = (_Float16)0.f;
  if (tid < D) {
    const float ang = (float)pos * inv_freq[tid < half ? tid : tid - half];
    const double turns = (double)ang * 0.15915494309189535;
    const float fr = (float)(turns - __builtin_floor(turns));
    rc = (_Float16)__builtin_amdgcn_cosf(fr);
    rs = (_Float16)__builtin_amdgcn_sinf(fr);
  }

  if constexpr (XF) {
    static_assert(D == 64 || D == 128, "the transform prologue holds 3 x 16 x D partial sums in LDS");
    constexpr int LOGD = D == 64 ? 6 : 7;
    constexpr int G = D / 4, R = kAttnThreads / G;  // float4 column groups, chunk rows per pass
    constexpr int QP = 4, WP = 2;                   // chunk rows and partial sums in flight per thread
    constexpr bool SEP = XF == 2;
    const int g = tid & (G - 1), r = tid >> (LOGD - 2);
    // slices: q of head h, k and v of its kv head - of the one vector, or each of its own
    const int off[3] = {h * D, SEP ? kvh * D : (H + kvh) * D, SEP ? kvh * D : (H + Hkv + kvh) * D};
    int iK[3], bb[3], lgb[3];
#pragma unroll
    for (int s3 = 0; s3 < 3; ++s3) {
      const int lp = X.logp2[SEP ? s3 : 0];
      lgb[s3] = lp - LOGD;
      iK[s3] = off[s3] >> lp;
      bb[s3] = (off[s3] >> LOGD) & ((1 << lgb[s3]) - 1);
    }
    // the epilogue's operands, requested with everything else
    const int s3 = tid >> LOGD, c = tid & (D - 1);
    const int sx = SEP ? (s3 < 3 ? s3 : 0) : 0;  // descriptor of this thread's slice
    float postv = 1.f;
    const float* postp = sx == 0 ? X.post[0] : (sx == 1 ? X.post[1] : X.post[2]);
    if (tid < 3 * D && postp) postv = postp[off[s3 < 3 ? s3 : 0] + c];
    const float scalev = sx == 0 ? X.scale[0] : (sx == 1 ? X.scale[1] : X.scale[2]);
    float a[3][4];  // (plain arrays: element-wise bit operations on vector-typed values went wrong in the compiler)
#pragma unroll
    for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
      for (int e = 0; e < 4; ++e) a[s3][e] = 0.f;
    if constexpr (SEP) {
      // three vectors: the rows of all three are requested in one go, one chunk row and two
      // partial sums per slice in flight (more would spill)
      constexpr int Q2 = 1, W2 = 2;
      int nrows[3], maxrows = 0;
#pragma unroll
      for (int s3 = 0; s3 < 3; ++s3) {
        nrows[s3] = X.n[s3] >> LOGD;
        maxrows = nrows[s3] > maxrows ? nrows[s3] : maxrows;
      }
      for (int j0 = 0; j0 < maxrows; j0 += Q2 * R) {
        float v[3][Q2][4];
        uint32_t hw[3][Q2];
#pragma unroll
        for (int s3 = 0; s3 < 3; ++s3) {
          // table words: with order 1 the index is 0 and the word is masked out (any readable address does)
          const uint32_t* hb = X.order[s3] > 1 ? X.had_bits[s3] : reinterpret_cast<const uint32_t*>(X.parts[s3]);
#pragma unroll
          for (int q = 0; q < Q2; ++q) {
            const int j = j0 + r + q * R;
            const int jc = j < nrows[s3] ? j : 0;
            const unsigned bit = (unsigned)(jc >> lgb[s3]) * X.order[s3] + iK[s3];
            hw[s3][q] = hb[bit >> 5] >> (bit & 31);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[s3][q][e] = 0.f;
          }
        }
        for (int w0 = 0; w0 < X.in_parts; w0 += W2) {
          float4a raw[3][Q2][W2];
#pragma unroll
          for (int u = 0; u < W2; ++u) {
            if (w0 + u < X.in_parts) {
#pragma unroll
              for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
                for (int q = 0; q < Q2; ++q) {
                  const int j = j0 + r + q * R;
                  const int jc = j < nrows[s3] ? j : 0;
                  raw[s3][q][u] = *reinterpret_cast<const float4a*>(
                      X.parts[s3] + (size_t)(w0 + u) * X.part_stride + ((size_t)jc << LOGD) + 4 * g);
                }
            } else {
#pragma unroll
              for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
                for (int q = 0; q < Q2; ++q) raw[s3][q][u] = float4a{0.f, 0.f, 0.f, 0.f};
            }
          }
#pragma unroll
          for (int u = 0; u < W2; ++u)
#pragma unroll
            for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
              for (int q = 0; q < Q2; ++q) {
                v[s3][q][0] += raw[s3][q][u].x;
                v[s3][q][1] += raw[s3][q][u].y;
                v[s3][q][2] += raw[s3][q][u].z;
                v[s3][q][3] += raw[s3][q][u].w;
              }
        }
#pragma unroll
        for (int s3 = 0; s3 < 3; ++s3) {
          const uint32_t omask = X.order[s3] > 1 ? 1u : 0u;
          const int bmask = (1 << lgb[s3]) - 1;
#pragma unroll
          for (int q = 0; q < Q2; ++q) {
            const int j = j0 + r + q * R;
            if (j < nrows[s3]) {
              const uint32_t sg = (((hw[s3][q] & omask) ^ (uint32_t)__builtin_popcount(bb[s3] & j & bmask)) & 1u) << 31;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                a[s3][e] += __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v[s3][q][e]) ^ sg);
            }
          }
        }
      }
    } else {
    const int logb = lgb[0], bmask = (1 << logb) - 1;
    const int nrows = X.n[0] >> LOGD;
    // table words: with order 1 the index is 0 and the word is masked out (any readable address does)
    const uint32_t* hb = X.order[0] > 1 ? X.had_bits[0] : reinterpret_cast<const uint32_t*>(X.parts[0]);
    const uint32_t omask = X.order[0] > 1 ? 1u : 0u;
    for (int j0 = 0; j0 < nrows; j0 += QP * R) {
      float v[QP][4];
      uint32_t hw[QP][3];
#pragma unroll
      for (int q = 0; q < QP; ++q) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[q][e] = 0.f;
        const int j = j0 + r + q * R;
        const int jc = j < nrows ? j : 0;
#pragma unroll
        for (int s3 = 0; s3 < 3; ++s3) {
          const unsigned bit = (unsigned)(jc >> logb) * X.order[0] + iK[s3];
          hw[q][s3] = hb[bit >> 5] >> (bit & 31);
        }
      }
      for (int w0 = 0; w0 < X.in_parts; w0 += WP) {
        float4a raw[QP][WP];
#pragma unroll
        for (int u = 0; u < WP; ++u) {
          if (w0 + u < X.in_parts) {
#pragma unroll
            for (int q = 0; q < QP; ++q) {
              const int j = j0 + r + q * R;
              const int jc = j < nrows ? j : 0;
              raw[q][u] = *reinterpret_cast<const float4a*>(X.parts[0] + (size_t)(w0 + u) * X.part_stride +
                                                            ((size_t)jc << LOGD) + 4 * g);
            }
          } else {
#pragma unroll
            for (int q = 0; q < QP; ++q) raw[q][u] = float4a{0.f, 0.f, 0.f, 0.f};
          }
        }
#pragma unroll
        for (int u = 0; u < WP; ++u)
#pragma unroll
          for (int q = 0; q < QP; ++q) {
            v[q][0] += raw[q][u].x;
            v[q][1] += raw[q][u].y;
            v[q][2] += raw[q][u].z;
            v[q][3] += raw[q][u].w;
          }
      }
#pragma unroll
      for (int q = 0; q < QP; ++q) {
        const int j = j0 + r + q * R;
        if (j < nrows) {
#pragma unroll
          for (int s3 = 0; s3 < 3; ++s3) {
            const uint32_t sg = (((hw[q][s3] & omask) ^ (uint32_t)__builtin_popcount(bb[s3] & j & bmask)) & 1u) << 31;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              a[s3][e] += __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v[q][e]) ^ sg);
          }
        }
      }
    }
    }
    // rows that share a wave, then one partial slice per wave
#pragma unroll
    for (int b = 5; (1 << b) >= G; --b)
#pragma unroll
      for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
        for (int e = 0; e < 4; ++e) a[s3][e] += qtip_wht::lane_xor(a[s3][e], b);
    if (lane < G) {
#pragma unroll
      for (int s3 = 0; s3 < 3; ++s3)
        *reinterpret_cast<float4a*>(acc + (s3 * 16 + wave) * D + 4 * g) =
            float4a{a[s3][0], a[s3][1], a[s3][2], a[s3][3]};
    }
    __syncthreads();
    float y = 0.f;
    if (tid < 3 * D) {
#pragma unroll
      for (int w = 0; w < 16; ++w) y += acc[(s3 * 16 + w) * D + c];
      y = qtip_wht::wht_lanes(y, 6, lane);
      if (D > 64) q_s[s3 * kMaxHeadDim + c] = y;
    }
    __syncthreads();  // the partial slices are consumed: their space takes the fp16 result
    _Float16* h_s = reinterpret_cast<_Float16*>(acc);
    if (tid < 3 * D) {
      if (D > 64) {
        const float other = q_s[s3 * kMaxHeadDim + (c ^ 64)];
        y = (c & 64) ? other - y : y + other;
      }
      h_s[s3 * D + c] = (_Float16)(y * scalev * postv);
    }
    __syncthreads();
  }
  const _Float16* h_s = reinterpret_cast<const _Float16*>(acc);
  auto QV = [&](int i) -> _Float16 { return XF ? h_s[i] : q_in[i]; };
  auto KV = [&](int i) -> _Float16 { return XF ? h_s[D + i] : k_in[i]; };
  auto VV = [&](int i) -> _Float16 { return XF ? h_s[2 * D + i] : v_in[i]; };

  // ---- rotary embedding in fp16 arithmetic: x*cos + rotate_half(x)*sin
  if (tid < D) {
    const _Float16 c = rc, s = rs;
    const _Float16 q0 = QV(tid), k0 = KV(tid), v0 = VV(tid);
    const _Float16 qr = tid < half ? (_Float16)(-(float)QV(tid + half)) : QV(tid - half);
    const _Float16 kr = tid < half ? (_Float16)(-(float)KV(tid + half)) : KV(tid - half);
    const _Float16 qe = (_Float16)((float)(_Float16)((float)q0 * (float)c) + (float)(_Float16)((float)qr * (float)s));
    const _Float16 ke = (_Float16)((float)(_Float16)((float)k0 * (float)c) + (float)(_Float16)((float)kr * (float)s));
    q_s[tid] = (float)qe;
    k_s[tid] = (float)ke;
    v_s[tid] = (float)v0;
    if (blockIdx.x == 0 && blockIdx.z == 0 && pos < max_len) {
      kc[(size_t)pos * D + tid] = ke;
      vc[(size_t)pos * D + tid] = v0;
    }
  }
  __syncthreads();

  // ---- scores: 8 lanes per key (16 dims each), 128 keys per pass
  const float sm_scale = rsqrtf((float)D);
  const int nkeys = pos + 1 < max_len ? pos + 1 : max_len;
  const int k0 = (int)blockIdx.z * keys_per_split;                       // this workgroup's keys: [k0, k1)
  const int k1 = k0 + keys_per_split < nkeys ? k0 + keys_per_split : nkeys;
  const int sub = tid & 7, kq = tid >> 3;
  constexpr int dper = D >> 3;  // dims per lane (multiple of 8: D % 64 == 0)
  float mx = -INFINITY;
  // four keys per thread group and round, all of their loads issued before the first use
  constexpr int KU = 4;
  for (int t0 = k0; t0 < k1; t0 += KU * (kAttnThreads / 8)) {
    uint4 raw[KU][dper / 8];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int t = t0 + kq + u * (kAttnThreads / 8);
      const int tc = (t < k1 && t != pos) ? t : 0;  // clamped: the new key comes from LDS
      const uint4* kr = reinterpret_cast<const uint4*>(kc + (size_t)tc * D + sub * dper);
#pragma unroll
      for (int d8 = 0; d8 < dper / 8; ++d8) raw[u][d8] = kr[d8];
    }
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int t = t0 + kq + u * (kAttnThreads / 8);
      float s = 0.f;
      if (t == pos) {
        for (int d = 0; d < dper; ++d) s += q_s[sub * dper + d] * k_s[sub * dper + d];
      } else {
#pragma unroll
        for (int d8 = 0; d8 < dper / 8; ++d8) {
          const _Float16* hv = reinterpret_cast<const _Float16*>(&raw[u][d8]);
#pragma unroll
          for (int e = 0; e < 8; ++e) s += q_s[sub * dper + d8 * 8 + e] * (float)hv[e];
        }
      }
      s += qtip_wht::lane_xor(s, 0);
      s += qtip_wht::lane_xor(s, 1);
      s += qtip_wht::lane_xor(s, 2);
      s *= sm_scale;
      if (t < k1) {
        if (sub == 0) p_s[t - k0] = s;
        mx = fmaxf(mx, s);
      }
    }
  }
  // the values of the first round (keys tg, tg + TG, ...: all of them up to 512 keys) are requested
  // here, before the softmax reductions: their addresses do not depend on the scores.  (Requesting
  // the first round of keys ahead of the rotary embedding in the same way measured slower.)
  constexpr int DG = D >> 3, TG = kAttnThreads / DG;  // 16 dim groups, 64 key groups for D = 128
  constexpr int VU = 8;  // values per thread and round, loaded before the first use
  const int dg = tid % DG, tg = tid / DG;
  uint4 vfirst[VU];
#pragma unroll
  for (int u = 0; u < VU; ++u) {
    const int t = k0 + tg + u * TG;
    const int tc = (t < k1 && t != pos) ? t : 0;
    vfirst[u] = *reinterpret_cast<const uint4*>(vc + (size_t)tc * D + dg * 8);
  }
  mx = wave_reduce_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) mx = fmaxf(mx, red[w]);
  float sum = 0.f;
  for (int t = tid; t < k1 - k0; t += kAttnThreads) {
    const float e = __expf(p_s[t] - mx);
    p_s[t] = e;
    sum += e;
  }
  sum = wave_reduce_sum(sum);
  __syncthreads();  // everyone has read red[] (max) and written p_s
  if (lane == 0) red[16 + wave] = sum;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) tot += red[16 + w];
  const float inv = 1.f / tot;

  // ---- output: thread (tg, dg) sums keys tg, tg+TG, ... for dims 8*dg .. 8*dg+7
  float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int t0 = k0 + tg; t0 < k1; t0 += VU * TG) {
    uint4 raw[VU];
    if (t0 == k0 + tg) {
#pragma unroll
      for (int u = 0; u < VU; ++u) raw[u] = vfirst[u];
    } else {
#pragma unroll
      for (int u = 0; u < VU; ++u) {
        const int t = t0 + u * TG;
        const int tc = (t < k1 && t != pos) ? t : 0;
        raw[u] = *reinterpret_cast<const uint4*>(vc + (size_t)tc * D + dg * 8);
      }
    }
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int t = t0 + u * TG;
      if (t < k1) {
        const float pt = p_s[t - k0];
        if (t == pos) {
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] += pt * v_s[dg * 8 + e];
        } else {
          const _Float16* hv = reinterpret_cast<const _Float16*>(&raw[u]);
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] += pt * (float)hv[e];
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[tg * D + dg * 8 + e] = o[e];
  __syncthreads();
  // two-level sum over the TG partial rows: thread (part, d) adds TG/PARTS rows, then PARTS rows
  {
    constexpr int PARTS = kAttnThreads / D;  // 8 for D = 128 (TG = 64 rows)
    const int d = tid % D, part = tid / D;
    constexpr int per = TG / PARTS;
    float sum = 0.f;
    for (int r = 0; r < per; ++r) sum += acc[(part * per + r) * D + d];
    __syncthreads();
    acc[part * D + d] = sum;
    __syncthreads();
    if (tid < D) {
      float tot2 = 0.f;
      for (int r = 0; r < PARTS; ++r) tot2 += acc[r * D + tid];
      acc[tid] = tot2;  // only read by this thread below
    }
  }
  if (nsplit == 1) {
    if (tid < D) out[(size_t)h * D + tid] = (_Float16)(acc[tid] * inv);
  } else if (tid < D) {
    float* w = split_ws + ((size_t)h * nsplit + blockIdx.z) * (D + 2);
    w[tid] = acc[tid];  // 0 for a range past the last key
    if (tid == 0) {
      w[D] = mx;        // -inf for an empty range
      w[D + 1] = tot;
    }
  }
}

// out[head] = sum_z exp(m_z - M) o_z / sum_z exp(m_z - M) l_z over the key ranges of a head
// (M = max_z m_z): the softmax of the whole context from the shares of its ranges.
__global__ __launch_bounds__(kMaxHeadDim) void attn_combine_kernel(_Float16* __restrict__ out,
                                                                  const float* __restrict__ split_ws,
                                                                  int nsplit, int D) {
  const int h = blockIdx.x, d = threadIdx.x;
  const float* w = split_ws + (size_t)h * nsplit * (D + 2);
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, w[z * (D + 2) + D]);
  float num = 0.f, den = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float mz = w[z * (D + 2) + D];
    const float e = mz == -INFINITY ? 0.f : __expf(mz - M);
    num += e * w[z * (D + 2) + d];
    den += e * w[z * (D + 2) + D + 1];
  }
  out[(size_t)h * D + d] = (_Float16)(num / den);
}

}  // namespace

static int launch_attention(void* out_f16, const void* qkv_f16, const AttnXf* xf, int xf_mode, void* k_cache_f16,
                            void* v_cache_f16, const void* pos_i64, const float* inv_freq, int heads,
                            int kv_heads, int head_dim, int max_len, int key_splits, float* split_ws,
                            void* stream) {
  if (!out_f16 || !k_cache_f16 || !v_cache_f16 || !pos_i64 || !inv_freq) return QTIP_E_NULL;
  if (key_splits < 1 || key_splits > 16) return QTIP_E_SHAPE;
  if (key_splits > 1 && !split_ws) return QTIP_E_NULL;
  if (key_splits > 1 && (reinterpret_cast<uintptr_t>(split_ws) & 15)) return QTIP_E_ALIGN;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || head_dim < 64 || head_dim > kMaxHeadDim ||
      (head_dim & (head_dim - 1)) || max_len < 1 || max_len > 4096)
    return QTIP_E_SHAPE;
  const size_t lds = (size_t)(3 * kMaxHeadDim + 32 + 8192 + max_len) * sizeof(float);
  const dim3 grid((unsigned)(heads / kv_heads), (unsigned)kv_heads, (unsigned)key_splits);
  const int kps = (max_len + key_splits - 1) / key_splits;  // keys per range
#define QTIP_ATTN(DD, XX, ARG)                                                                      \
  decode_attn_kernel<DD, XX><<<grid, kAttnThreads, lds, (hipStream_t)stream>>>(                      \
      (_Float16*)out_f16, (const _Float16*)qkv_f16, (_Float16*)k_cache_f16, (_Float16*)v_cache_f16,  \
      (const long*)pos_i64, inv_freq, heads, kv_heads, max_len, ARG, key_splits, kps, split_ws)
  if (xf) {
    if (head_dim != 64 && head_dim != 128) return QTIP_E_SHAPE;
    if (xf_mode == 1) {
      if (head_dim == 64) QTIP_ATTN(64, 1, *xf); else QTIP_ATTN(128, 1, *xf);
    } else {
      if (head_dim == 64) QTIP_ATTN(64, 2, *xf); else QTIP_ATTN(128, 2, *xf);
    }
  } else {
    switch (head_dim) {
      case 64: QTIP_ATTN(64, 0, AttnXf{}); break;
      case 128: QTIP_ATTN(128, 0, AttnXf{}); break;
      default: QTIP_ATTN(256, 0, AttnXf{}); break;
    }
  }
#undef QTIP_ATTN
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || key_splits == 1) return (int)e;
  attn_combine_kernel<<<heads, head_dim, 0, (hipStream_t)stream>>>((_Float16*)out_f16, split_ws, key_splits,
                                                                   head_dim);
  return (int)hipGetLastError();
}

// one transformed vector of n elements: table order and log2 of the power-of-two part
static int fill_xf_slot(AttnXf& x, int slot, const float* parts, const float* post, const uint32_t* had_bits,
                        float scale, int order, long n, int head_dim) {
  if (!parts || (order > 1 && !had_bits)) return QTIP_E_NULL;
  if (order < 1 || order > 256 || n % order) return QTIP_E_SHAPE;
  const long p2 = n / order;
  if ((p2 & (p2 - 1)) || p2 < head_dim || n > (1 << 20)) return QTIP_E_SHAPE;
  if (reinterpret_cast<uintptr_t>(parts) & 15) return QTIP_E_ALIGN;
  x.parts[slot] = parts;
  x.post[slot] = post;
  x.had_bits[slot] = had_bits;
  x.scale[slot] = scale;
  x.order[slot] = order;
  x.logp2[slot] = 0;
  while ((1L << x.logp2[slot]) < p2) ++x.logp2[slot];
  x.n[slot] = (int)n;
  return QTIP_OK;
}

extern "C" int qtip_decode_attention(void* out_f16, const void* qkv_f16, void* k_cache_f16,
                                     void* v_cache_f16, const void* pos_i64, const float* inv_freq,
                                     int heads, int kv_heads, int head_dim, int max_len, int key_splits,
                                     float* split_workspace, void* stream) {
  if (!qkv_f16) return QTIP_E_NULL;
  return launch_attention(out_f16, qkv_f16, nullptr, 0, k_cache_f16, v_cache_f16, pos_i64, inv_freq, heads,
                          kv_heads, head_dim, max_len, key_splits, split_workspace, stream);
}

extern "C" int qtip_decode_attention_rht(void* out_f16, const float* parts, int in_parts, size_t part_stride,
                                         const float* post_f32, float scale, const uint32_t* had_bits,
                                         int order, void* k_cache_f16, void* v_cache_f16,
                                         const void* pos_i64, const float* inv_freq, int heads,
                                         int kv_heads, int head_dim, int max_len, int key_splits,
                                         float* split_workspace, void* stream) {
  if (in_parts < 1 || in_parts > 16 || heads < 1 || kv_heads < 1 || head_dim < 64 || head_dim > 128 ||
      (part_stride & 3))
    return QTIP_E_SHAPE;
  AttnXf x = {};
  const int rc = fill_xf_slot(x, 0, parts, post_f32, had_bits, scale, order,
                              (long)(heads + 2 * kv_heads) * head_dim, head_dim);
  if (rc) return rc;
  x.part_stride = part_stride;
  x.in_parts = in_parts;
  return launch_attention(out_f16, nullptr, &x, 1, k_cache_f16, v_cache_f16, pos_i64, inv_freq, heads, kv_heads,
                          head_dim, max_len, key_splits, split_workspace, stream);
}

extern "C" int qtip_decode_attention_rht3(void* out_f16, const float* const* parts, int in_parts,
                                          size_t part_stride, const float* const* post_f32, const float* scale,
                                          const uint32_t* const* had_bits, const int* order, void* k_cache_f16,
                                          void* v_cache_f16, const void* pos_i64, const float* inv_freq,
                                          int heads, int kv_heads, int head_dim, int max_len, int key_splits,
                                          float* split_workspace, void* stream) {
  if (!parts || !post_f32 || !scale || !had_bits || !order) return QTIP_E_NULL;
  if (in_parts < 1 || in_parts > 16 || heads < 1 || kv_heads < 1 || head_dim < 64 || head_dim > 128 ||
      (part_stride & 3))
    return QTIP_E_SHAPE;
  AttnXf x = {};
  for (int s = 0; s < 3; ++s) {
    const long n = (long)(s == 0 ? heads : kv_heads) * head_dim;
    const int rc = fill_xf_slot(x, s, parts[s], post_f32[s], had_bits[s], scale[s], order[s], n, head_dim);
    if (rc) return rc;
  }
  x.part_stride = part_stride;
  x.in_parts = in_parts;
  return launch_attention(out_f16, nullptr, &x, 2, k_cache_f16, v_cache_f16, pos_i64, inv_freq, heads, kv_heads,
                          head_dim, max_len, key_splits, split_workspace, stream);
}

// ---- token head of the decode loop: final RMSNorm and the greedy pick ------------------------

namespace {

constexpr int kHeadThreads = 1024;

// out = w * fp16(x * rsqrt(mean(x^2) + eps)) for one vector (model/llama.py:129-135), one workgroup
__global__ __launch_bounds__(kHeadThreads) void rmsnorm_kernel(_Float16* __restrict__ out,
                                                               const _Float16* __restrict__ x,
                                                               const _Float16* __restrict__ w, float eps,
                                                               int n) {
  __shared__ float wsum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int MAXE = 16;  // n <= 16384
  float v[MAXE], g[MAXE];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < MAXE; ++e) {
    const int i = tid + e * kHeadThreads;
    v[e] = i < n ? (float)x[i] : 0.f;
    g[e] = i < n ? (float)w[i] : 0.f;
    ss += v[e] * v[e];
  }
  ss = qtip_wht::wave_sum(ss);
  if (lane == 0) wsum[wave] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int q = 0; q < 16; ++q) tot += wsum[q];
  const float rs = __builtin_amdgcn_rsqf(tot / (float)n + eps);
#pragma unroll
  for (int e = 0; e < MAXE; ++e) {
    const int i = tid + e * kHeadThreads;
    if (i < n) out[i] = (_Float16)(g[e] * (float)(_Float16)(v[e] * rs));
  }
}

// argmax of fp16 logits (first index among equal maxima, NaNs never win), stored as the next
// input token and into the history slot of this position; the position advances by one.  All in
// device memory, so a recorded graph decodes token after token without host work in between
// (eval/interactive_gen.py:43-69 does this with argmax, copies and an increment per token).
__global__ __launch_bounds__(kHeadThreads) void greedy_pick_kernel(const _Float16* __restrict__ logits, int vocab,
                                                                   long* __restrict__ tok, long* __restrict__ pos,
                                                                   long* __restrict__ hist, long hist_len,
                                                                   long hist_base) {
  __shared__ float bv[16];
  __shared__ int bi[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  const int nch = vocab >> 3;  // 16-byte chunks
  for (int c = tid; c < nch; c += kHeadThreads) {
    const uint4 raw = reinterpret_cast<const uint4*>(logits)[c];
    const _Float16* h = reinterpret_cast<const _Float16*>(&raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)h[e];
      if (f > best) {  // chunks come in increasing order per thread: the first maximum stays
        best = f;
        idx = c * 8 + e;
      }
    }
  }
  for (int i = (nch << 3) + tid; i < vocab; i += kHeadThreads) {
    const float f = (float)logits[i];
    if (f > best) {
      best = f;
      idx = i;
    }
  }
#pragma unroll
  for (int b = 0; b < 6; ++b) {
    const float ob = qtip_wht::lane_xor(best, b);
    const int oi = lane_xor_i(idx, b);
    if (ob > best || (ob == best && oi < idx)) {
      best = ob;
      idx = oi;
    }
  }
  if (lane == 0) {
    bv[wave] = best;
    bi[wave] = idx;
  }
  __syncthreads();
  if (tid == 0) {
    for (int q = 1; q < 16; ++q)
      if (bv[q] > best || (bv[q] == best && bi[q] < idx)) {
        best = bv[q];
        idx = bi[q];
      }
    if (idx == 0x7fffffff) idx = 0;  // nothing compared greater than -inf
    const long p = pos[0];
    const long slot = p - hist_base;
    if (hist && slot >= 0 && slot < hist_len) hist[slot] = idx;
    tok[0] = idx;
    pos[0] = p + 1;
  }
}

}  // namespace

extern "C" int qtip_rmsnorm(void* out_f16, const void* x_f16, const void* weight_f16, float eps, int n,
                            void* stream) {
  if (!out_f16 || !x_f16 || !weight_f16) return QTIP_E_NULL;
  if (n < 1 || n > 16 * kHeadThreads) return QTIP_E_SHAPE;
  rmsnorm_kernel<<<1, kHeadThreads, 0, (hipStream_t)stream>>>((_Float16*)out_f16, (const _Float16*)x_f16,
                                                             (const _Float16*)weight_f16, eps, n);
  return (int)hipGetLastError();
}

extern "C" int qtip_greedy_pick(const void* logits_f16, int vocab, void* tok_i64, void* pos_i64,
                                void* history_i64, long history_len, long history_base, void* stream) {
  if (!logits_f16 || !tok_i64 || !pos_i64) return QTIP_E_NULL;
  if (vocab < 1 || history_len < 0 || (reinterpret_cast<uintptr_t>(logits_f16) & 15)) return QTIP_E_SHAPE;
  greedy_pick_kernel<<<1, kHeadThreads, 0, (hipStream_t)stream>>>((const _Float16*)logits_f16, vocab, (long*)tok_i64,
                                                                 (long*)pos_i64, (long*)history_i64, history_len,
                                                                 history_base);
  return (int)hipGetLastError();
}

// ---- sampled token pick ----------------------------------------------------------------------

namespace {

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// (value, index) pairs ordered by value descending, index ascending; `before(a, b)`: a comes first
__device__ __forceinline__ bool before(float av, int ai, float bv, int bi) {
  return av > bv || (av == bv && ai < bi);
}

// Sampling of eval/interactive_gen.py:15-40 in one launch: logits / temperature, everything below
// the top_k-th largest logit removed (ties with it stay, as torch.where(logits < kth, -inf, logits)
// keeps them), softmax, and a draw by the exponential race argmax(p_i / q_i), q_i ~ Exp(1) - which
// is argmax(logit_i / T - log q_i).  The q_i come from a counter-based generator keyed by (seed,
// draw counter, i); the counter lives in device memory and advances with every launch, so a
// recorded graph draws fresh numbers at every replay.  Bookkeeping as in greedy_pick_kernel.
__global__ __launch_bounds__(kHeadThreads) void sample_pick_kernel(const _Float16* __restrict__ logits, int vocab,
                                                                   float inv_temperature, int top_k, uint32_t seed,
                                                                   long* __restrict__ counter, long* __restrict__ tok,
                                                                   long* __restrict__ pos, long* __restrict__ hist,
                                                                   long hist_len, long hist_base) {
  __shared__ float bv[16];
  __shared__ int bi[16];
  __shared__ float sel_v;
  __shared__ int sel_i;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // block-wide first element in (value desc, index asc) order among those after (pv, pi)
  auto next_after = [&](float pv, int pi, auto&& score) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = tid; i < vocab; i += kHeadThreads) {
      const float raw = (float)logits[i];
      if (before(pv, pi, raw, i)) {  // strictly after the previous pick
        const float f = score(raw, i);
        if (before(f, i, best, idx)) {
          best = f;
          idx = i;
        }
      }
    }
#pragma unroll
    for (int b = 0; b < 6; ++b) {
      const float ob = qtip_wht::lane_xor(best, b);
      const int oi = lane_xor_i(idx, b);
      if (before(ob, oi, best, idx)) {
        best = ob;
        idx = oi;
      }
    }
    __syncthreads();  // the previous round's result has been read by everyone
    if (lane == 0) {
      bv[wave] = best;
      bi[wave] = idx;
    }
    __syncthreads();
    if (tid == 0) {
      for (int q = 1; q < 16; ++q)
        if (before(bv[q], bi[q], best, idx)) {
          best = bv[q];
          idx = bi[q];
        }
      sel_v = best;
      sel_i = idx;
    }
    __syncthreads();
  };
  // ---- the top_k-th largest logit (with multiplicity): top_k rounds of "next in order"
  float kth = -INFINITY;
  if (top_k > 0 && top_k < vocab) {
    float pv = INFINITY;
    int pi = -1;
    for (int r = 0; r < top_k; ++r) {
      next_after(pv, pi, [](float raw, int) { return raw; });
      pv = sel_v;
      pi = sel_i;
    }
    kth = pv;
  }
  // ---- the race: argmax over the kept entries of logit / T - log(q), q = -log(u)
  const uint32_t draw = (uint32_t)counter[0];
  const uint32_t key = mix32(seed ^ mix32(draw + 0x9e3779b9U));
  next_after(INFINITY, -1, [&](float raw, int i) {
    if (raw < kth) return -INFINITY;
    const uint32_t h = mix32(key ^ mix32((uint32_t)i * 0x85ebca6bU + 1u));
    const float u = ((float)(h >> 8) + 0.5f) * (1.0f / 16777216.0f);  // (0, 1)
    return raw * inv_temperature - __logf(-__logf(u));
  });
  if (tid == 0) {
    int idx = sel_i;
    if (idx == 0x7fffffff) idx = 0;
    const long p = pos[0];
    const long slot = p - hist_base;
    if (hist && slot >= 0 && slot < hist_len) hist[slot] = idx;
    tok[0] = idx;
    pos[0] = p + 1;
    counter[0] = (long)draw + 1;
  }
}

}  // namespace

extern "C" int qtip_sample_pick(const void* logits_f16, int vocab, float temperature, int top_k,
                                unsigned seed, void* counter_i64, void* tok_i64, void* pos_i64,
                                void* history_i64, long history_len, long history_base, void* stream) {
  if (!logits_f16 || !counter_i64 || !tok_i64 || !pos_i64) return QTIP_E_NULL;
  if (vocab < 1 || history_len < 0 || top_k < 0 || top_k > 64) return QTIP_E_SHAPE;
  const float t = temperature > 1e-5f ? temperature : 1e-5f;  // max(temperature, 1e-5) as the reference
  sample_pick_kernel<<<1, kHeadThreads, 0, (hipStream_t)stream>>>((const _Float16*)logits_f16, vocab, 1.0f / t, top_k,
                                                                 seed, (long*)counter_i64, (long*)tok_i64,
                                                                 (long*)pos_i64, (long*)history_i64, history_len,
                                                                 history_base);
  return (int)hipGetLastError();
}
