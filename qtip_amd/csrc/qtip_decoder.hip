// Single-token decode attention for the end-to-end decode loop: rotary
// embedding of q and k, KV-cache write and attention over the cache in one
// launch (the reference runs these as a dozen framework kernels:
// model/llama.py:264-295 RoPE, model/cache_utils.py:1173-1193 cache update,
// model/llama.py:866-880 scaled-dot-product attention).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qtip_hip.h"

namespace {

constexpr int kAttnThreads = 1024;
constexpr int kMaxHeadDim = 256;

__device__ __forceinline__ float wave_reduce_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_reduce_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// One workgroup per query head.  qkv: [H*D | Hkv*D | Hkv*D] fp16 of the new
// token; k_cache / v_cache: [Hkv][max_len][D] fp16; pos_ptr: position of the
// new token (device memory, so that a recorded graph follows the position).
template <int D>
__global__ __launch_bounds__(kAttnThreads) void decode_attn_kernel(
    _Float16* __restrict__ out, const _Float16* __restrict__ qkv, _Float16* __restrict__ k_cache,
    _Float16* __restrict__ v_cache, const long* __restrict__ pos_ptr,
    const float* __restrict__ inv_freq, int H, int Hkv, int max_len) {
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

  // ---- rotary embedding in fp16 arithmetic: x*cos + rotate_half(x)*sin
  if (tid < D) {
    const int i = tid < half ? tid : tid - half;
    // the angle is the fp32 product the reference forms; its reduction to a fraction of a turn is
    // done in fp64 (exact to 2^-29 of a turn at position 4096), the hardware cos / sin take turns.
    // (cosf / sinf with their large-argument paths cost ~0.5 us on this kernel's critical path.)
    const float ang = (float)pos * inv_freq[i];
    const double turns = (double)ang * 0.15915494309189535;
    const float fr = (float)(turns - __builtin_floor(turns));
    const _Float16 c = (_Float16)__builtin_amdgcn_cosf(fr), s = (_Float16)__builtin_amdgcn_sinf(fr);
    const _Float16 q0 = q_in[tid], k0 = k_in[tid];
    const _Float16 qr = tid < half ? (_Float16)(-(float)q_in[tid + half]) : q_in[tid - half];
    const _Float16 kr = tid < half ? (_Float16)(-(float)k_in[tid + half]) : k_in[tid - half];
    const _Float16 qe = (_Float16)((float)(_Float16)((float)q0 * (float)c) + (float)(_Float16)((float)qr * (float)s));
    const _Float16 ke = (_Float16)((float)(_Float16)((float)k0 * (float)c) + (float)(_Float16)((float)kr * (float)s));
    q_s[tid] = (float)qe;
    k_s[tid] = (float)ke;
    v_s[tid] = (float)v_in[tid];
    if (blockIdx.x == 0 && pos < max_len) {
      kc[(size_t)pos * D + tid] = ke;
      vc[(size_t)pos * D + tid] = v_in[tid];
    }
  }
  __syncthreads();

  // ---- scores: 8 lanes per key (16 dims each), 128 keys per pass
  const float sm_scale = rsqrtf((float)D);
  const int nkeys = pos + 1 < max_len ? pos + 1 : max_len;
  const int sub = tid & 7, kq = tid >> 3;
  constexpr int dper = D >> 3;  // dims per lane (multiple of 8: D % 64 == 0)
  float mx = -INFINITY;
  // four keys per thread group and round, all of their loads issued before the first use
  constexpr int KU = 4;
  for (int t0 = 0; t0 < nkeys; t0 += KU * (kAttnThreads / 8)) {
    uint4 raw[KU][dper / 8];
#pragma unroll
    for (int u = 0; u < KU; ++u) {
      const int t = t0 + kq + u * (kAttnThreads / 8);
      const int tc = (t < nkeys && t != pos) ? t : 0;  // clamped: the new key comes from LDS
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
      s += __shfl_xor(s, 1);
      s += __shfl_xor(s, 2);
      s += __shfl_xor(s, 4);
      s *= sm_scale;
      if (t < nkeys) {
        if (sub == 0) p_s[t] = s;
        mx = fmaxf(mx, s);
      }
    }
  }
  mx = wave_reduce_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) mx = fmaxf(mx, red[w]);
  float sum = 0.f;
  for (int t = tid; t < nkeys; t += kAttnThreads) {
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
  constexpr int DG = D >> 3, TG = kAttnThreads / DG;  // 16 dim groups, 64 key groups for D = 128
  const int dg = tid % DG, tg = tid / DG;
  float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  constexpr int VU = 8;  // values per thread and round, loaded before the first use
  for (int t0 = tg; t0 < nkeys; t0 += VU * TG) {
    uint4 raw[VU];
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int t = t0 + u * TG;
      const int tc = (t < nkeys && t != pos) ? t : 0;
      raw[u] = *reinterpret_cast<const uint4*>(vc + (size_t)tc * D + dg * 8);
    }
#pragma unroll
    for (int u = 0; u < VU; ++u) {
      const int t = t0 + u * TG;
      if (t < nkeys) {
        const float pt = p_s[t];
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
  if (tid < D) out[(size_t)h * D + tid] = (_Float16)(acc[tid] * inv);
}

}  // namespace

extern "C" int qtip_decode_attention(void* out_f16, const void* qkv_f16, void* k_cache_f16,
                                     void* v_cache_f16, const void* pos_i64, const float* inv_freq,
                                     int heads, int kv_heads, int head_dim, int max_len, void* stream) {
  if (!out_f16 || !qkv_f16 || !k_cache_f16 || !v_cache_f16 || !pos_i64 || !inv_freq) return QTIP_E_NULL;
  if (heads < 1 || kv_heads < 1 || heads % kv_heads || head_dim < 64 || head_dim > kMaxHeadDim ||
      (head_dim & (head_dim - 1)) || max_len < 1 || max_len > 4096)
    return QTIP_E_SHAPE;
  const size_t lds = (size_t)(3 * kMaxHeadDim + 32 + 8192 + max_len) * sizeof(float);
#define QTIP_ATTN(DD)                                                                               \
  decode_attn_kernel<DD><<<dim3((unsigned)(heads / kv_heads), (unsigned)kv_heads), kAttnThreads, lds, (hipStream_t)stream>>>(                          \
      (_Float16*)out_f16, (const _Float16*)qkv_f16, (_Float16*)k_cache_f16, (_Float16*)v_cache_f16,  \
      (const long*)pos_i64, inv_freq, heads, kv_heads, max_len)
  switch (head_dim) {
    case 64: QTIP_ATTN(64); break;
    case 128: QTIP_ATTN(128); break;
    default: QTIP_ATTN(256); break;
  }
#undef QTIP_ATTN
  return (int)hipGetLastError();
}
