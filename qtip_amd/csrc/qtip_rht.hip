// Randomised Hadamard transform kernel and its launchers (qtip_rht,
// qtip_rht_fused).  Declarations: include/qtip_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qtip_hip.h"
#include "qtip_wht.h"

using namespace qtip_wht;

namespace {

constexpr int kRhtThreads = 1024;
constexpr int kMaxParts = 16;

// out = post * scale * (H_order (x) H_A (x) H_pp) (pre * f(in)) [+ residual],  n = order * A * pp.
// The power-of-two part is split as H_A (x) H_pp (Sylvester matrices factor
// that way) so that OT = order * A workgroups share one vector: workgroup
// (iK, iA) produces the pp outputs of its row of the (order*A)-wide mix,
//   z[c] = sum_{jK,jA} (-1)^(bits[iK][jK] + popcount(iA & jA)) v[(jK*A + jA)*pp + c],
// followed by a pp-point Walsh-Hadamard transform of z.  The transform is
// latency-bound (a vector is a few KB), so every thread issues all of its
// loads (n / 1024 elements and their companions) before the first use; the
// pp-point transform runs on cross-lane exchanges inside a wave for the low
// six index bits and needs one LDS transposition for the rest.
//
// Optional element-wise prologue f (what the layers around a QTIP linear do
// to its input) and epilogue:
//   PRE_RMSNORM   f(x) = fp16(w * fp16(x * rsqrt(mean(x^2) + eps)))   (model/llama.py:129-135)
//   PRE_SILU_MUL  f = fp16(fp16(silu(g)) * u), g = in[i], u = in[n + i] (model/llama.py:399-400)
//   residual      out = fp16(residual + fp16(result))                 (model/llama.py:964,979)
enum { PRE_NONE = 0, PRE_RMSNORM = 1, PRE_SILU_MUL = 2 };

struct RhtParams {
  void* out;
  const void* in;
  const uint32_t* had_bits;
  const _Float16* pre;       // SU or null
  const float* post;         // SV or null
  const _Float16* norm_w;    // PRE_RMSNORM weight
  const _Float16* residual;  // or null
  size_t part_stride;
  size_t in_row_stride;      // elements between consecutive rows of `in`
  size_t post_row_stride;    // elements between the rows' `post` vectors (0: one vector for all rows)
  size_t pre_row_stride;     // the same for `pre`
  float scale, eps;
  int in_parts, n, order, logA, pp, pre_mode;
  // from the host (divisions and search loops in the prologue of a latency-bound kernel are time on
  // its critical path): log2 of the column groups (vectorised form) or of the columns (scalar form),
  // log2 of the waves holding a row in the transform, passes over the vector
  int lcg, logw, npass;
};

template <typename T>
__device__ __forceinline__ float ldf(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldf<float>(const float* p, size_t i) {
  return p[i];
}
template <>
__device__ __forceinline__ float ldf<_Float16>(const _Float16* p, size_t i) {
  return (float)p[i];
}

// CH = loads in flight per thread and pass; FUSED enables the prologue modes
// (which need the raw elements of the whole row, so the row must fit one pass);
// RI = rows iK of the order-wide mix one workgroup produces (the loaded
// elements are reused for all of them, which divides the load traffic of the
// large table orders by RI).  Sign bits are indexed [jK][iK] so that the RI
// signs of one element are adjacent bits of one word.
template <typename TIn, typename TOut, int CH, bool FUSED, int RI>
__global__ __launch_bounds__(kRhtThreads) void rht_kernel(const RhtParams P) {
  __shared__ float red[RI][kRhtThreads];  // partial sums, then the exchange buffer of the transform
  __shared__ float wsum[16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int A = 1 << P.logA;
  // blockIdx.x = (iK / RI) * A + iA   (RI > 1 only with A == 1)
  const int iK0 = (blockIdx.x >> P.logA) * RI, iA = blockIdx.x & (A - 1);
  const size_t r = blockIdx.y;
  const int n = P.n, pp = P.pp, order = P.order;
  const TIn* src = reinterpret_cast<const TIn*>(P.in) + r * P.in_row_stride;
  const int OT = order << P.logA;
  const int logc = P.lcg;              // log2(pp), pp <= kRhtThreads (launcher)
  const int JG = kRhtThreads >> logc;
  const int c = tid & (pp - 1), jg = tid >> logc;
  const int pre_mode = FUSED ? P.pre_mode : PRE_NONE;

  float z[RI];
#pragma unroll
  for (int ri = 0; ri < RI; ++ri) z[ri] = 0.f;
  const int npass = P.npass;  // the same for every thread (barriers inside)
  for (int pass = 0; pass < npass; ++pass) {
    const int j0 = jg + pass * JG * CH;
    // ---- all loads of this pass: elements j = j0, j0+JG, ... of column c.
    // The loads are unconditional (out-of-range items re-read element c and are
    // masked afterwards) and nothing depends on them until all are issued.
    TIn xr[CH], ar[FUSED ? CH : 1];
    float xs[CH];
    _Float16 sr[CH];
    uint32_t br[CH];
    bool ok[CH];
    size_t idx[CH];
    // (one uniform branch per array, never per element: a load inside a
    // per-element branch is waited for at once)
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      ok[q] = j < OT;
      idx[q] = (size_t)(ok[q] ? j : 0) * pp + c;
      xr[q] = src[idx[q]];
      xs[q] = 0.f;
      sr[q] = (_Float16)1.f;
      br[q] = 0;
    }
    if (P.pre) {
#pragma unroll
      for (int q = 0; q < CH; ++q) sr[q] = P.pre[r * P.pre_row_stride + idx[q]];
    }
    if (order > 1) {
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        const int j = j0 + q * JG;
        const unsigned bit = (unsigned)((ok[q] ? j : 0) >> P.logA) * order + iK0;
        br[q] = P.had_bits[bit >> 5] >> (bit & 31);  // bits 0..RI-1: rows iK0 .. iK0+RI-1
      }
    }
    if (FUSED && pre_mode == PRE_RMSNORM) {
#pragma unroll
      for (int q = 0; q < CH; ++q) ar[q] = (TIn)P.norm_w[idx[q]];
    }
    if (FUSED && pre_mode == PRE_SILU_MUL) {
#pragma unroll
      for (int q = 0; q < CH; ++q) ar[q] = src[(size_t)n + idx[q]];
    }
    for (int w = 1; w < P.in_parts; ++w) {
#pragma unroll
      for (int q = 0; q < CH; ++q) xs[q] += ldf<TIn>(src + w * P.part_stride, idx[q]);
    }
    float v[CH], f[CH], aux[FUSED ? CH : 1];
    uint32_t sg[CH];
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      v[q] = ok[q] ? (float)xr[q] + xs[q] : 0.f;
      if (FUSED) aux[q] = (float)ar[q];
      f[q] = (float)sr[q];
      sg[q] = br[q] ^ ((uint32_t)__builtin_popcount(iA & (j & (A - 1))) & 1u);
    }
    // ---- element-wise prologue
    if (FUSED && pre_mode == PRE_RMSNORM) {
      float ss = 0.f;
#pragma unroll
      for (int q = 0; q < CH; ++q) ss += v[q] * v[q];
      ss = wave_sum(ss);
      if (lane == 0) wsum[tid >> 6] = ss;
      __syncthreads();
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < 16; ++w) tot += wsum[w];
      const float rs = __builtin_amdgcn_rsqf(tot / (float)n + P.eps);
#pragma unroll
      for (int q = 0; q < CH; ++q) v[q] = (float)(_Float16)(aux[q] * (float)(_Float16)(v[q] * rs));
    } else if (FUSED && pre_mode == PRE_SILU_MUL) {
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        const float g = v[q];
        const float sl = (float)(_Float16)(g * __builtin_amdgcn_rcpf(1.f + __expf(-g)));
        v[q] = (float)(_Float16)(sl * aux[q]);
      }
    }
    // ---- mix
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const uint32_t vf = __builtin_bit_cast(uint32_t, v[q] * f[q]);
#pragma unroll
      for (int ri = 0; ri < RI; ++ri) z[ri] += __builtin_bit_cast(float, vf ^ ((sg[q] >> ri) << 31));
    }
  }
  if (JG > 1) {
#pragma unroll
    for (int ri = 0; ri < RI; ++ri) red[ri][tid] = z[ri];
    __syncthreads();
  }
  // ---- thread t < RI*pp takes row t / pp, column t % pp
  const int row = tid >> logc, col = tid & (pp - 1);  // col keeps the lane index in its low bits
  const bool active = tid < RI * pp;
  float y = 0.f;
  if (active) {
    if (JG > 1) {
      for (int q = 0; q < JG; ++q) y += red[row][q * pp + col];
    } else {
      y = z[0];  // JG == 1 implies pp == 1024 and RI == 1
    }
  }
  // ---- pp-point transform
  const int logw = P.logw;
  const int W = 1 << logw;  // waves holding one row
  if (JG > 1 && W > 1) __syncthreads();  // the buffer is reused only when a row spans several waves
  const int nb0 = logc < 6 ? logc : 6;
  int cfin = col;
  if (active) {
    y = wht_lanes(y, nb0, lane);
    if (W > 1) red[row][col] = y;
  }
  if (W > 1) {
    __syncthreads();
    if (active) {
      // transposed read: the wave index of the element becomes the low lane bits
      const int wv = col >> 6;
      const int ew = lane & (W - 1);              // wave part of the element index
      const int el = (lane >> logw) + (64 >> logw) * wv;  // lane part of the element index
      cfin = 64 * ew + el;
      y = red[row][cfin];
      y = wht_lanes(y, logw, lane);
    }
  }
  if (active) {
    const size_t idx = ((size_t)(iK0 + row) * A + iA) * pp + cfin;
    float o = y * P.scale;
    if (P.post) o *= P.post[r * P.post_row_stride + idx];
    TOut* op = reinterpret_cast<TOut*>(P.out) + r * (size_t)n + idx;
    if (FUSED && P.residual) {
      const float res = (float)P.residual[r * (size_t)n + idx];
      *op = (TOut)(_Float16)(res + (float)(_Float16)o);
    } else {
      *op = (TOut)o;
    }
  }
}

// ---------------------------------------------------------------------------
// Vectorised form (pp a multiple of 8, 16-byte aligned rows): the same mix + transform, but a
// thread loads 8 consecutive columns of a row j with one 16-byte load (two for fp32 input), so
// a vector costs n/8192 load instructions per thread instead of n/1024 two-byte gathers - the
// scalar form is bound by the address rate of the vector-memory unit, not by bytes.
//   thread t: column group cg = t % (pp/8), row group jg = t / (pp/8); rows j = jg, jg + JG, ...
//   z[e] (8 columns) accumulates over the thread's rows, lanes that share cg are summed with
//   cross-lane adds, the 16 waves' partial vectors (8 row groups for pp = 1024) meet in LDS,
//   thread c < pp then owns column c for the pp-point transform as in the scalar form.
// The per-output operands (post, residual) are fetched at the start, so their latency (they are
// cold in the decode loop: every layer has its own) overlaps the loads of the vector.
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

template <typename TIn>
struct Raw8;
template <>
struct Raw8<_Float16> {
  uint4 a;
  __device__ __forceinline__ void load(const _Float16* p) { a = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void get(float v[8]) const {
    const half8v h = __builtin_bit_cast(half8v, a);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = (float)h[e];
  }
};
template <>
struct Raw8<float> {
  float4v a, b;
  __device__ __forceinline__ void load(const float* p) {
    a = *reinterpret_cast<const float4v*>(p);
    b = *reinterpret_cast<const float4v*>(p + 4);
  }
  __device__ __forceinline__ void get(float v[8]) const {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = a[e];
      v[4 + e] = b[e];
    }
  }
};

template <typename TIn, typename TOut, int CH, bool FUSED>
__global__ __launch_bounds__(kRhtThreads) void rht_vec_kernel(const RhtParams P) {
  __shared__ __align__(16) float red[8192];  // partial vectors [NP][pp], then the exchange buffer of the transform
  __shared__ float wsum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int A = 1 << P.logA;
  const int iK = blockIdx.x >> P.logA, iA = blockIdx.x & (A - 1);
  const size_t r = blockIdx.y;
  const int n = P.n, pp = P.pp, order = P.order;
  const TIn* src = reinterpret_cast<const TIn*>(P.in) + r * P.in_row_stride;
  const int OT = order << P.logA;
  // (logarithms and the pass count come from the host: divisions and search loops in the
  // prologue of a latency-bound kernel are time on its critical path)
  const int lcg = P.lcg;
  const int CG = 1 << lcg;             // column groups of 8 (power of two, 1 .. 128)
  const int JG = kRhtThreads >> lcg;   // row groups
  const int cg = tid & (CG - 1), jg = tid >> lcg;
  const int pre_mode = FUSED ? P.pre_mode : PRE_NONE;

  // ---- this thread's output element and its operands
  const bool active = tid < pp;
  const int logw = P.logw;
  const int W = 1 << logw;  // waves holding the row in the transform
  int cfin = tid;
  if (W > 1) {
    const int wv = tid >> 6;
    cfin = 64 * (lane & (W - 1)) + (lane >> logw) + (64 >> logw) * wv;  // after the transposed read
  }
  const size_t oidx = ((size_t)iK * A + iA) * pp + cfin;
  float postv = 1.f, resv = 0.f;
  if (active) {
    if (P.post) postv = P.post[r * P.post_row_stride + oidx];
    if (FUSED && P.residual) resv = (float)P.residual[r * (size_t)n + oidx];
  }

  float z[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) z[e] = 0.f;
  const int npass = P.npass;  // the same for every thread (barriers inside)
  for (int pass = 0; pass < npass; ++pass) {
    const int j0 = jg + pass * JG * CH;
    Raw8<TIn> xr[CH], ar[FUSED ? CH : 1];
    Raw8<_Float16> sr[CH], nw[FUSED ? CH : 1];
    uint32_t br[CH];
    bool ok[CH];
    size_t base[CH];
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      ok[q] = j < OT;
      base[q] = (size_t)(ok[q] ? j : 0) * pp + 8 * cg;
      xr[q].load(src + base[q]);
      br[q] = 0;
    }
    if (P.pre) {
#pragma unroll
      for (int q = 0; q < CH; ++q) sr[q].load(P.pre + r * P.pre_row_stride + base[q]);
    }
    if (order > 1) {
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        const int j = j0 + q * JG;
        const unsigned bit = (unsigned)((ok[q] ? j : 0) >> P.logA) * order + iK;
        br[q] = (P.had_bits[bit >> 5] >> (bit & 31)) & 1u;
      }
    }
    if (FUSED && pre_mode == PRE_RMSNORM) {
#pragma unroll
      for (int q = 0; q < CH; ++q) nw[q].load(P.norm_w + base[q]);
    }
    if (FUSED && pre_mode == PRE_SILU_MUL) {
#pragma unroll
      for (int q = 0; q < CH; ++q) ar[q].load(src + (size_t)n + base[q]);
    }
    float v[CH][8];
#pragma unroll
    for (int q = 0; q < CH; ++q) xr[q].get(v[q]);
    for (int w = 1; w < P.in_parts; ++w) {
      Raw8<TIn> pr[CH];
#pragma unroll
      for (int q = 0; q < CH; ++q) pr[q].load(src + w * P.part_stride + base[q]);
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        float t[8];
        pr[q].get(t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] += t[e];
      }
    }
#pragma unroll
    for (int q = 0; q < CH; ++q)
      if (!ok[q]) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] = 0.f;
      }
    // ---- element-wise prologue
    if (FUSED && pre_mode == PRE_RMSNORM) {
      float ss = 0.f;
#pragma unroll
      for (int q = 0; q < CH; ++q)
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += v[q][e] * v[q][e];
      ss = wave_sum(ss);
      if (lane == 0) wsum[wave] = ss;
      __syncthreads();
      float tot = 0.f;
#pragma unroll
      for (int w = 0; w < 16; ++w) tot += wsum[w];
      const float rs = __builtin_amdgcn_rsqf(tot / (float)n + P.eps);
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        float wn[8];
        nw[q].get(wn);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] = (float)(_Float16)(wn[e] * (float)(_Float16)(v[q][e] * rs));
      }
    } else if (FUSED && pre_mode == PRE_SILU_MUL) {
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        float up[8];
        ar[q].get(up);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float g = v[q][e];
          const float sl = (float)(_Float16)(g * __builtin_amdgcn_rcpf(1.f + __expf(-g)));
          v[q][e] = (float)(_Float16)(sl * up[e]);
        }
      }
    }
    // ---- mix
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      const uint32_t sg = (br[q] ^ ((uint32_t)__builtin_popcount(iA & (j & (A - 1))) & 1u)) << 31;
      float f[8];
      if (P.pre) {
        sr[q].get(f);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = 1.f;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        z[e] += __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v[q][e] * f[e]) ^ sg);
    }
  }
  // ---- lanes that share a column group (they differ in lane bits lcg .. 5)
#pragma unroll
  for (int b = 0; b < 6; ++b) {
    if (b >= lcg) {
#pragma unroll
      for (int e = 0; e < 8; ++e) z[e] += lane_xor(z[e], b);
    }
  }
  // ---- partial vectors to LDS: one per wave (CG <= 64) or one per row group (CG = 128)
  const int NP = CG <= 64 ? 16 : JG;
  const int part = CG <= 64 ? wave : jg;
  if (CG > 64 || lane < CG) {
    float4v* dst = reinterpret_cast<float4v*>(red + part * pp + 8 * cg);
    dst[0] = float4v{z[0], z[1], z[2], z[3]};
    dst[1] = float4v{z[4], z[5], z[6], z[7]};
  }
  __syncthreads();
  float y = 0.f;
  if (active) {
    for (int q = 0; q < NP; ++q) y += red[q * pp + tid];
  }
  if (W > 1) __syncthreads();  // the buffer is reused only when a row spans several waves
  // ---- pp-point transform of column tid
  const int nb0 = lcg + 3 < 6 ? lcg + 3 : 6;  // log2(pp), at most the six lane bits
  if (active) {
    y = wht_lanes(y, nb0, lane);
    if (W > 1) red[tid] = y;
  }
  if (W > 1) {
    __syncthreads();
    if (active) {
      y = red[cfin];
      y = wht_lanes(y, logw, lane);
    }
  }
  if (active) {
    const float o = y * P.scale * postv;
    TOut* op = reinterpret_cast<TOut*>(P.out) + r * (size_t)n + oidx;
    if (FUSED && P.residual) *op = (TOut)(_Float16)(resv + (float)(_Float16)o);
    else *op = (TOut)o;
  }
}

// The output transforms of gate and up and the SiLU * up that follows them, in one launch:
//   h = fp16(fp16(silu(gate)) * up),  [gate | up] = fp16(post * scale * (H_order (x) H_p)(sum of parts))
// (lib/codebook/bitshift.py:465-472 twice, model/llama.py:399-400).  A workgroup of the vectorised
// form reads the whole input anyway, so it produces the gate row AND the matching up row of the
// mix from the same loads and applies the element-wise step to the pp outputs it owns - once per
// element, where the [SiLU * up + input transform] launch that otherwise follows repeats it in
// every one of its workgroups.  ROWS = false: gate and up are the two halves of one transformed
// vector (fused up/gate projection; rows iK and iK + order / 2 of the mix).  ROWS = true: two
// vectors with a transform each (separate projections; the same row iK of either).
template <int CH, bool ROWS>
__global__ __launch_bounds__(kRhtThreads) void rht_vec_silu_pair_kernel(const RhtParams P) {
  __shared__ __align__(16) float red[2 * 8192];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int A = 1 << P.logA;
  const int iK = blockIdx.x >> P.logA, iA = blockIdx.x & (A - 1);
  const int n = P.n, pp = P.pp, order = P.order;
  const int iK2 = ROWS ? iK : iK + (order >> 1);
  const float* src = reinterpret_cast<const float*>(P.in);
  const float* src2 = ROWS ? src + P.in_row_stride : src;
  const int OT = order << P.logA;
  const int lcg = P.lcg;
  const int CG = 1 << lcg;
  const int JG = kRhtThreads >> lcg;
  const int cg = tid & (CG - 1), jg = tid >> lcg;
  const bool active = tid < pp;
  const int logw = P.logw;
  const int W = 1 << logw;
  int cfin = tid;
  if (W > 1) cfin = 64 * (lane & (W - 1)) + (lane >> logw) + (64 >> logw) * wave;
  const size_t oidx1 = ((size_t)iK * A + iA) * pp + cfin;
  const size_t oidx2 = ((size_t)iK2 * A + iA) * pp + cfin;
  float post1 = 1.f, post2 = 1.f;
  if (active && P.post) {
    post1 = P.post[oidx1];
    post2 = P.post[(ROWS ? P.post_row_stride : 0) + oidx2];
  }
  float z1[8], z2[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) z1[e] = z2[e] = 0.f;
  for (int pass = 0; pass < P.npass; ++pass) {
    const int j0 = jg + pass * JG * CH;
    Raw8<float> xr[CH], yr[ROWS ? CH : 1];
    uint32_t b1[CH], b2[CH];
    bool ok[CH];
    size_t base[CH];
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      ok[q] = j < OT;
      base[q] = (size_t)(ok[q] ? j : 0) * pp + 8 * cg;
      xr[q].load(src + base[q]);
      if constexpr (ROWS) yr[q].load(src2 + base[q]);
      b1[q] = b2[q] = 0;
    }
    if (order > 1) {
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        const int j = j0 + q * JG;
        const unsigned row = (unsigned)((ok[q] ? j : 0) >> P.logA) * order;
        const unsigned bit1 = row + iK, bit2 = row + iK2;
        b1[q] = (P.had_bits[bit1 >> 5] >> (bit1 & 31)) & 1u;
        b2[q] = (P.had_bits[bit2 >> 5] >> (bit2 & 31)) & 1u;
      }
    }
    float v[CH][8], u[ROWS ? CH : 1][8];
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      xr[q].get(v[q]);
      if constexpr (ROWS) yr[q].get(u[q]);
    }
    for (int w = 1; w < P.in_parts; ++w) {
      Raw8<float> pr[CH], qr[ROWS ? CH : 1];
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        pr[q].load(src + w * P.part_stride + base[q]);
        if constexpr (ROWS) qr[q].load(src2 + w * P.part_stride + base[q]);
      }
#pragma unroll
      for (int q = 0; q < CH; ++q) {
        float t[8];
        pr[q].get(t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[q][e] += t[e];
        if constexpr (ROWS) {
          qr[q].get(t);
#pragma unroll
          for (int e = 0; e < 8; ++e) u[q][e] += t[e];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < CH; ++q) {
      const int j = j0 + q * JG;
      if (ok[q]) {
        const uint32_t sc = (uint32_t)__builtin_popcount(iA & (j & (A - 1))) & 1u;
        const uint32_t s1 = (b1[q] ^ sc) << 31, s2 = (b2[q] ^ sc) << 31;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float a = v[q][e], b = ROWS ? u[q][e] : v[q][e];
          z1[e] += __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, a) ^ s1);
          z2[e] += __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, b) ^ s2);
        }
      }
    }
  }
#pragma unroll
  for (int b = 0; b < 6; ++b) {
    if (b >= lcg) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        z1[e] += lane_xor(z1[e], b);
        z2[e] += lane_xor(z2[e], b);
      }
    }
  }
  const int NP = CG <= 64 ? 16 : JG;
  const int part = CG <= 64 ? wave : jg;
  const int nb0 = lcg + 3 < 6 ? lcg + 3 : 6;
  // both vectors go through the reduction and the pp-point transform side by side: three
  // barriers for the pair
  float* red1 = red;
  float* red2 = red + 8192;
  if (CG > 64 || lane < CG) {
    float4v* d1 = reinterpret_cast<float4v*>(red1 + part * pp + 8 * cg);
    float4v* d2 = reinterpret_cast<float4v*>(red2 + part * pp + 8 * cg);
    d1[0] = float4v{z1[0], z1[1], z1[2], z1[3]};
    d1[1] = float4v{z1[4], z1[5], z1[6], z1[7]};
    d2[0] = float4v{z2[0], z2[1], z2[2], z2[3]};
    d2[1] = float4v{z2[4], z2[5], z2[6], z2[7]};
  }
  __syncthreads();
  float y1 = 0.f, y2 = 0.f;
  if (active) {
    for (int q = 0; q < NP; ++q) {
      y1 += red1[q * pp + tid];
      y2 += red2[q * pp + tid];
    }
  }
  if (W > 1) __syncthreads();  // the partial vectors are consumed before the buffers are reused
  if (active) {
    y1 = wht_lanes(y1, nb0, lane);
    y2 = wht_lanes(y2, nb0, lane);
    if (W > 1) {
      red1[tid] = y1;
      red2[tid] = y2;
    }
  }
  if (W > 1) {
    __syncthreads();
    if (active) {
      y1 = wht_lanes(red1[cfin], logw, lane);
      y2 = wht_lanes(red2[cfin], logw, lane);
    }
  }
  if (active) {
    const float g = (float)(_Float16)(y1 * P.scale * post1);
    const float up = (float)(_Float16)(y2 * P.scale * post2);
    const float sl = (float)(_Float16)(g * __builtin_amdgcn_rcpf(1.f + __expf(-g)));
    reinterpret_cast<_Float16*>(P.out)[oidx1] = (_Float16)(sl * up);
  }
}

template <typename TI, typename TO, bool FUSED>
int launch_rht_vec(const RhtParams& P, dim3 grid, long loads, hipStream_t st) {
  // a prologue needs the whole row in one pass
  if (FUSED && P.pre_mode == PRE_RMSNORM && loads > 4) return QTIP_E_SHAPE;
  // (the fused form with four loads in flight spills registers: only the RMSNorm prologue, which
  // cannot take a second pass, uses it; the sums run in the same order either way)
  const int ch = loads <= 1 ? 1 : (loads <= 2 || (FUSED && P.pre_mode != PRE_RMSNORM)) ? 2 : 4;
  RhtParams Q = P;
  Q.npass = (int)((loads + ch - 1) / ch);
  if (ch == 1) rht_vec_kernel<TI, TO, 1, FUSED><<<grid, kRhtThreads, 0, st>>>(Q);
  else if (ch == 2) rht_vec_kernel<TI, TO, 2, FUSED><<<grid, kRhtThreads, 0, st>>>(Q);
  else rht_vec_kernel<TI, TO, 4, FUSED><<<grid, kRhtThreads, 0, st>>>(Q);
  return (int)hipGetLastError();
}

template <typename TI, typename TO, bool FUSED>
int launch_rht_l(const RhtParams& P, dim3 grid, long loads, int ri, hipStream_t st) {
  // a prologue needs the whole row in one pass
  if (FUSED && P.pre_mode == PRE_RMSNORM && loads > 16) return QTIP_E_SHAPE;
  const int ch = ri == 4 ? (loads <= 8 ? 8 : 16) : (loads <= 4 ? 4 : loads <= 8 ? 8 : 16);
  RhtParams Q = P;
  Q.npass = (int)((loads + ch - 1) / ch);
  if (ri == 4) {
    if (ch == 8) rht_kernel<TI, TO, 8, FUSED, 4><<<grid, kRhtThreads, 0, st>>>(Q);
    else rht_kernel<TI, TO, 16, FUSED, 4><<<grid, kRhtThreads, 0, st>>>(Q);
  } else {
    if (ch == 4) rht_kernel<TI, TO, 4, FUSED, 1><<<grid, kRhtThreads, 0, st>>>(Q);
    else if (ch == 8) rht_kernel<TI, TO, 8, FUSED, 1><<<grid, kRhtThreads, 0, st>>>(Q);
    else rht_kernel<TI, TO, 16, FUSED, 1><<<grid, kRhtThreads, 0, st>>>(Q);
  }
  return (int)hipGetLastError();
}

// Many rows of a power-of-two size (n = 1024 * EPT, order 1): one workgroup per row does the
// whole transform - register butterflies, six lane levels, one exchange through LDS that swaps
// the wave bits with the low four lane bits, four more lane levels - and reads and writes the
// row once.  (The forms above split a row over order * A workgroups that each read all of it:
// right for one vector, whose transform is latency-bound, 40 times slower for a 1024-token prompt.)
template <int EPT, typename TIn, typename TOut>
__global__ __launch_bounds__(kRhtThreads) void rht_rows_kernel(const RhtParams P) {
  constexpr int N = kRhtThreads * EPT;
  __shared__ __align__(16) float xbuf[N + N / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t r = blockIdx.x;
  const int e_nat = tid * EPT;
  const int e_swp = (((lane & 15) << 6) | ((wave & 15) << 2) | (lane >> 4)) * EPT;
  const TIn* src = reinterpret_cast<const TIn*>(P.in) + r * P.in_row_stride;
  float v[EPT], pv[EPT];
  auto load = [&](const TIn* p, float t[EPT]) {
    if constexpr (sizeof(TIn) == 2) ld_f16<EPT>(reinterpret_cast<const _Float16*>(p), t);
    else ld_f32<EPT>(reinterpret_cast<const float*>(p), t);
  };
  load(src + e_nat, v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) pv[i] = 1.f;
  if (P.post) ld_f32<EPT>(P.post + r * P.post_row_stride + e_swp, pv);
  if (P.pre) {
    float sv[EPT];
    ld_f16<EPT>(P.pre + r * P.pre_row_stride + e_nat, sv);
    for (int w = 1; w < P.in_parts; ++w) {
      float t[EPT];
      load(src + w * P.part_stride + e_nat, t);
#pragma unroll
      for (int i = 0; i < EPT; ++i) v[i] += t[i];
    }
#pragma unroll
    for (int i = 0; i < EPT; ++i) v[i] *= sv[i];
  } else {
    for (int w = 1; w < P.in_parts; ++w) {
      float t[EPT];
      load(src + w * P.part_stride + e_nat, t);
#pragma unroll
      for (int i = 0; i < EPT; ++i) v[i] += t[i];
    }
  }
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xbuf[xidx<EPT>(e_nat + i)] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(xbuf[xidx<EPT>(e_swp + i)], 4, lane) * P.scale * pv[i];
  TOut* dst = reinterpret_cast<TOut*>(P.out) + r * (size_t)N + e_swp;
  if constexpr (sizeof(TOut) == 2) {
    _Float16 h[EPT];
#pragma unroll
    for (int i = 0; i < EPT; ++i) h[i] = (_Float16)v[i];
    st_f16<EPT>(reinterpret_cast<_Float16*>(dst), h);
  } else {
#pragma unroll
    for (int i = 0; i < EPT; ++i) reinterpret_cast<float*>(dst)[i] = v[i];
  }
}

template <typename TIn, typename TOut>
int launch_rht_rows(const RhtParams& P, int rows, hipStream_t st) {
  switch (P.n) {
    case 2048: rht_rows_kernel<2, TIn, TOut><<<rows, kRhtThreads, 0, st>>>(P); break;
    case 4096: rht_rows_kernel<4, TIn, TOut><<<rows, kRhtThreads, 0, st>>>(P); break;
    default: rht_rows_kernel<8, TIn, TOut><<<rows, kRhtThreads, 0, st>>>(P); break;
  }
  return (int)hipGetLastError();
}

// rows from which the one-workgroup-per-row form is used for the power-of-two sizes it covers
constexpr int kRowsFormMin = 8;

int launch_rht(RhtParams P, int out_dtype, int in_dtype, int rows, void* stream) {
  if (!P.out || !P.in) return QTIP_E_NULL;
  const int n = P.n, order = P.order;
  if (rows < 1 || rows > 65535 || n < 1 || order < 1 || P.in_parts < 1 || P.in_parts > kMaxParts)
    return QTIP_E_SHAPE;
  if (n % order) return QTIP_E_SHAPE;
  const int p = n / order;
  if (p & (p - 1)) return QTIP_E_SHAPE;
  if (order > 1 && !P.had_bits) return QTIP_E_NULL;
  if ((unsigned)out_dtype > 1u || (unsigned)in_dtype > 1u) return QTIP_E_DTYPE;
  // split the power-of-two part: pp points per workgroup (<= 1024), A row
  // groups.  Every workgroup reads the whole vector (n / 1024 loads per thread
  // whatever the split), so A only trades L2 traffic (order*A*n elements)
  // against the size of the in-workgroup transform: up to 64 workgroups per vector.
  int pp = p, logA = 0;
  while (pp > kRhtThreads) {
    pp >>= 1;
    ++logA;
  }
  while (pp > 64 && ((long)order << (logA + 1)) <= 64) {
    pp >>= 1;
    ++logA;
  }
  const long OT = (long)order << logA;
  P.logA = logA;
  P.pp = pp;
  hipStream_t st = (hipStream_t)stream;
  const bool fused = P.pre_mode != PRE_NONE || P.residual != nullptr;
  {
    const size_t ez = in_dtype == QTIP_F16 ? 2 : 4;
    const bool rows_form = !fused && order == 1 && rows >= kRowsFormMin && (n == 2048 || n == 4096 || n == 8192) &&
                           (reinterpret_cast<uintptr_t>(P.in) & 15u) == 0 && (reinterpret_cast<uintptr_t>(P.out) & 15u) == 0 &&
                           ((P.in_row_stride * ez) & 15u) == 0 && ((P.part_stride * ez) & 15u) == 0 &&
                           (!P.pre || (reinterpret_cast<uintptr_t>(P.pre) & 15u) == 0) &&
                           (!P.post || ((reinterpret_cast<uintptr_t>(P.post) & 15u) == 0 && (P.post_row_stride & 3u) == 0));
    if (rows_form) {
      if (in_dtype == QTIP_F16 && out_dtype == QTIP_F16) return launch_rht_rows<_Float16, _Float16>(P, rows, st);
      if (in_dtype == QTIP_F16) return launch_rht_rows<_Float16, float>(P, rows, st);
      if (out_dtype == QTIP_F16) return launch_rht_rows<float, _Float16>(P, rows, st);
      return launch_rht_rows<float, float>(P, rows, st);
    }
  }
  if (fused && out_dtype != QTIP_F16) return QTIP_E_DTYPE;  // fused forms exist for the combinations the decode loop uses
  // vectorised form: 8 columns per thread, 16-byte loads
  const size_t esz = in_dtype == QTIP_F16 ? 2 : 4;
  // (vectors of up to 4096 elements stay on the scalar form: it has fewer phases and its few
  // loads per thread are not the limit there)
  const bool vec_ok = pp >= 8 && n > 4096 && (reinterpret_cast<uintptr_t>(P.in) & 15u) == 0 &&
                      ((P.in_row_stride * esz) & 15u) == 0 && ((P.part_stride * esz) & 15u) == 0 &&
                      (!P.pre || (reinterpret_cast<uintptr_t>(P.pre) & 15u) == 0) &&
                      (!P.norm_w || (reinterpret_cast<uintptr_t>(P.norm_w) & 15u) == 0) &&
                      !(P.pre_mode == PRE_SILU_MUL && ((size_t)n * esz & 15u));
  if (vec_ok) {
    int lcg = 0, logw = 0;
    while ((8 << lcg) < pp) ++lcg;
    while ((64 << logw) < pp) ++logw;
    P.lcg = lcg;
    P.logw = logw;
    const int JGv = kRhtThreads / (pp >> 3);
    const long vloads = (OT + JGv - 1) / JGv;
    dim3 vgrid((unsigned)OT, rows);
    if (fused) {
      if (in_dtype == QTIP_F16) return launch_rht_vec<_Float16, _Float16, true>(P, vgrid, vloads, st);
      return launch_rht_vec<float, _Float16, true>(P, vgrid, vloads, st);
    }
    if (in_dtype == QTIP_F16 && out_dtype == QTIP_F16) return launch_rht_vec<_Float16, _Float16, false>(P, vgrid, vloads, st);
    if (in_dtype == QTIP_F16 && out_dtype == QTIP_F32) return launch_rht_vec<_Float16, float, false>(P, vgrid, vloads, st);
    if (in_dtype == QTIP_F32 && out_dtype == QTIP_F16) return launch_rht_vec<float, _Float16, false>(P, vgrid, vloads, st);
    return launch_rht_vec<float, float, false>(P, vgrid, vloads, st);
  }
  {
    int logc = 0, logw = 0;
    while ((1 << logc) < pp) ++logc;
    while ((64 << logw) < pp) ++logw;
    P.lcg = logc;
    P.logw = logw;
  }
  const int JG = kRhtThreads / pp;
  const long loads = (OT + JG - 1) / JG;
  // large table orders: four rows of the mix per workgroup
  const int ri = (logA == 0 && order >= 64 && order % 4 == 0 && 4 * pp <= kRhtThreads && JG > 1) ? 4 : 1;
  dim3 grid((unsigned)(OT / ri), rows);
  if (fused) {
    if (in_dtype == QTIP_F16) return launch_rht_l<_Float16, _Float16, true>(P, grid, loads, ri, st);
    return launch_rht_l<float, _Float16, true>(P, grid, loads, ri, st);
  }
  if (in_dtype == QTIP_F16 && out_dtype == QTIP_F16) return launch_rht_l<_Float16, _Float16, false>(P, grid, loads, ri, st);
  if (in_dtype == QTIP_F16 && out_dtype == QTIP_F32) return launch_rht_l<_Float16, float, false>(P, grid, loads, ri, st);
  if (in_dtype == QTIP_F32 && out_dtype == QTIP_F16) return launch_rht_l<float, _Float16, false>(P, grid, loads, ri, st);
  return launch_rht_l<float, float, false>(P, grid, loads, ri, st);
}

// ---------------------------------------------------------------------------
// Two transforms of one hidden-size vector in one workgroup: the output transform of a linear
// layer, the residual addition, the RMSNorm of the next block and the input transform of the
// next linear layer (all four are separate launches otherwise, each with its own cold operands):
//   x_new = fp16(residual + fp16(post * scale_out * H (sum of parts)))
//   xt    = fp16(scale_in * H (pre * fp16(w * fp16(x_new * rsqrt(mean(x_new^2) + eps)))))
// n = 1024 * EPT is a power of two (both transforms of order 1).  Element e = [wave 4][lane 6][i]
// (i = log2 EPT register bits).  A transform runs its butterflies over the register bits, the six
// lane bits, and - after one exchange through LDS that swaps the wave bits with the low four
// lane bits - the remaining four bits.  The first transform leaves the data in the swapped
// layout, which is as good as any for the element-wise middle part; the second transform swaps
// back, so xt is stored in natural order.
template <int EPT>
__global__ __launch_bounds__(kRhtThreads) void rht_chain_kernel(
    _Float16* __restrict__ xt_out, _Float16* __restrict__ x_out, const float* __restrict__ parts,
    int in_parts, size_t part_stride, const float* __restrict__ post, float scale_out,
    const _Float16* __restrict__ residual, const _Float16* __restrict__ norm_w, float eps,
    const _Float16* __restrict__ pre, float scale_in) {
  constexpr int N = kRhtThreads * EPT;
  __shared__ __align__(16) float xbuf[N + N / 64];
  __shared__ float wsum[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t row = blockIdx.x;
  parts += row * N;
  // natural layout: e = tid * EPT + i;  swapped layout: wave bits <-> low four lane bits
  const int e_nat = tid * EPT;
  const int e_swp = (((lane & 15) << 6) | ((wave & 15) << 2) | (lane >> 4)) * EPT;
  // ---- operands of the middle part, in the swapped layout (issued first: they are cold)
  float pv[EPT], rv[EPT], wv[EPT], sv[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) pv[i] = sv[i] = 1.f;
  if (post) ld_f32<EPT>(post + e_swp, pv);
  ld_f16<EPT>(residual + row * N + e_swp, rv);
  ld_f16<EPT>(norm_w + e_swp, wv);
  if (pre) ld_f16<EPT>(pre + e_swp, sv);
  // ---- first transform
  float v[EPT];
  ld_f32<EPT>(parts + e_nat, v);
  for (int w = 1; w < in_parts; ++w) {
    float t[EPT];
    ld_f32<EPT>(parts + w * part_stride + e_nat, t);
#pragma unroll
    for (int i = 0; i < EPT; ++i) v[i] += t[i];
  }
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xbuf[xidx<EPT>(e_nat + i)] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(xbuf[xidx<EPT>(e_swp + i)], 4, lane);
  // ---- residual, RMSNorm, sign vector of the next layer
  float ss = 0.f;
  _Float16 xn[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const float o = v[i] * scale_out * pv[i];
    xn[i] = (_Float16)(rv[i] + (float)(_Float16)o);
    v[i] = (float)xn[i];
    ss += v[i] * v[i];
  }
  st_f16<EPT>(x_out + row * N + e_swp, xn);
  ss = wave_sum(ss);
  if (lane == 0) wsum[wave] = ss;
  __syncthreads();  // also: every read of xbuf above is done
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) tot += wsum[w];
  const float rs = __builtin_amdgcn_rsqf(tot / (float)N + eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = (float)(_Float16)(wv[i] * (float)(_Float16)(v[i] * rs)) * sv[i];
  // ---- second transform, from the swapped layout back to the natural one
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xbuf[xidx<EPT>(e_swp + i)] = v[i];
  __syncthreads();
  // the bits still missing are the top four of the element's lane field = lane bits 2..5 here
  _Float16 xo[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    float y = xbuf[xidx<EPT>(e_nat + i)];
    y = wht_lanes(y, 6, lane, 2);
    xo[i] = (_Float16)(y * scale_in);
  }
  st_f16<EPT>(xt_out + row * N + e_nat, xo);
}

}  // namespace

extern "C" {

int qtip_rht(void* out, int out_dtype, const void* in, int in_dtype, int in_parts, int rows, int n,
             int order, const uint32_t* had_bits, const void* pre_f16, const float* post_f32,
             float scale, void* stream) {
  RhtParams P{};
  P.out = out;
  P.in = in;
  P.had_bits = had_bits;
  P.pre = (const _Float16*)pre_f16;
  P.post = post_f32;
  P.part_stride = (size_t)(rows > 0 ? rows : 0) * (size_t)(n > 0 ? n : 0);
  P.in_row_stride = (size_t)(n > 0 ? n : 0);
  P.scale = scale;
  P.in_parts = in_parts;
  P.n = n;
  P.order = order;
  P.pre_mode = PRE_NONE;
  return launch_rht(P, out_dtype, in_dtype, rows, stream);
}

int qtip_rht_post_rows(void* out, int out_dtype, const void* in, int in_dtype, int in_parts, int rows, int n,
                       int order, const uint32_t* had_bits, const float* post_rows_f32, float scale,
                       void* stream) {
  if (!post_rows_f32) return QTIP_E_NULL;
  RhtParams P{};
  P.out = out;
  P.in = in;
  P.had_bits = had_bits;
  P.post = post_rows_f32;
  P.post_row_stride = (size_t)(n > 0 ? n : 0);
  P.part_stride = (size_t)(rows > 0 ? rows : 0) * (size_t)(n > 0 ? n : 0);
  P.in_row_stride = (size_t)(n > 0 ? n : 0);
  P.scale = scale;
  P.in_parts = in_parts;
  P.n = n;
  P.order = order;
  P.pre_mode = PRE_NONE;
  return launch_rht(P, out_dtype, in_dtype, rows, stream);
}

int qtip_rht_fused(void* out, int out_dtype, const void* in, int in_dtype, int in_parts, int rows,
                   int n, int order, const uint32_t* had_bits, const void* pre_f16,
                   const float* post_f32, float scale, int pre_mode, const void* norm_weight_f16,
                   float eps, const void* residual_f16, void* stream) {
  if (pre_mode < PRE_NONE || pre_mode > PRE_SILU_MUL) return QTIP_E_SHAPE;
  if (pre_mode == PRE_RMSNORM && !norm_weight_f16) return QTIP_E_NULL;
  if (pre_mode != PRE_NONE && in_parts != 1) return QTIP_E_SHAPE;
  RhtParams P{};
  P.out = out;
  P.in = in;
  P.had_bits = had_bits;
  P.pre = (const _Float16*)pre_f16;
  P.post = post_f32;
  P.norm_w = (const _Float16*)norm_weight_f16;
  P.residual = (const _Float16*)residual_f16;
  P.part_stride = (size_t)(rows > 0 ? rows : 0) * (size_t)(n > 0 ? n : 0);
  // gate and up halves sit side by side in a row of 2n elements
  P.in_row_stride = (size_t)(n > 0 ? n : 0) * (pre_mode == PRE_SILU_MUL ? 2 : 1);
  P.scale = scale;
  P.eps = eps;
  P.in_parts = in_parts;
  P.n = n;
  P.order = order;
  P.pre_mode = pre_mode;
  return launch_rht(P, out_dtype, in_dtype, rows, stream);
}

int qtip_rht_silu_pair(void* out_f16, const float* in_f32, int in_parts, int two_vectors, int n, int order,
                       const uint32_t* had_bits, const float* post_f32, float scale, void* stream) {
  // n: length of one transformed vector (two_vectors: gate and up have one each; otherwise they are
  // the halves of the one vector and out holds n / 2 values)
  if (!out_f16 || !in_f32) return QTIP_E_NULL;
  if (n < 1 || order < 1 || in_parts < 1 || in_parts > kMaxParts || n % order) return QTIP_E_SHAPE;
  if (!two_vectors && (order & 1)) return QTIP_E_SHAPE;  // gate and up are whole rows of the table mix
  const int p = n / order;
  if (p & (p - 1)) return QTIP_E_SHAPE;
  if (order > 1 && !had_bits) return QTIP_E_NULL;
  int pp = p, logA = 0;
  while (pp > kRhtThreads) {
    pp >>= 1;
    ++logA;
  }
  while (pp > 64 && ((long)order << (logA + 1)) <= 64) {
    pp >>= 1;
    ++logA;
  }
  if (pp < 8 || (reinterpret_cast<uintptr_t>(in_f32) & 15u) || ((size_t)n * 4 & 15u)) return QTIP_E_SHAPE;
  RhtParams P{};
  P.out = out_f16;
  P.in = in_f32;
  P.had_bits = had_bits;
  P.post = post_f32;
  P.post_row_stride = (size_t)n;
  P.in_row_stride = (size_t)n;
  P.part_stride = (size_t)n * (two_vectors ? 2 : 1);
  P.scale = scale;
  P.in_parts = in_parts;
  P.n = n;
  P.order = order;
  P.logA = logA;
  P.pp = pp;
  int lcg = 0, logw = 0;
  while ((8 << lcg) < pp) ++lcg;
  while ((64 << logw) < pp) ++logw;
  P.lcg = lcg;
  P.logw = logw;
  const long OT = (long)order << logA;
  const int JGv = kRhtThreads / (pp >> 3);
  const long loads = (OT + JGv - 1) / JGv;
  // (two vectors in flight: four loads of each per pass do not fit the 128 registers of a 1024-thread workgroup)
  const int ch = loads <= 1 ? 1 : (loads <= 2 || two_vectors) ? 2 : 4;
  P.npass = (int)((loads + ch - 1) / ch);
  const unsigned grid = (unsigned)(two_vectors ? OT : OT / 2);
  hipStream_t st = (hipStream_t)stream;
  if (two_vectors) {
    if (ch == 1) rht_vec_silu_pair_kernel<1, true><<<grid, kRhtThreads, 0, st>>>(P);
    else rht_vec_silu_pair_kernel<2, true><<<grid, kRhtThreads, 0, st>>>(P);
  } else {
    if (ch == 1) rht_vec_silu_pair_kernel<1, false><<<grid, kRhtThreads, 0, st>>>(P);
    else if (ch == 2) rht_vec_silu_pair_kernel<2, false><<<grid, kRhtThreads, 0, st>>>(P);
    else rht_vec_silu_pair_kernel<4, false><<<grid, kRhtThreads, 0, st>>>(P);
  }
  return (int)hipGetLastError();
}

int qtip_rht_fused_pre_rows(void* out_f16, const void* in_f16, int rows, int n, int order,
                            const uint32_t* had_bits, const void* pre_rows_f16, float scale,
                            const void* norm_weight_f16, float eps, void* stream) {
  if (!pre_rows_f16 || !norm_weight_f16) return QTIP_E_NULL;
  if ((reinterpret_cast<uintptr_t>(pre_rows_f16) & 15u) || ((size_t)(n > 0 ? n : 0) * 2 & 15u)) return QTIP_E_ALIGN;
  RhtParams P{};
  P.out = out_f16;
  P.in = in_f16;
  P.had_bits = had_bits;
  P.pre = (const _Float16*)pre_rows_f16;
  P.pre_row_stride = (size_t)(n > 0 ? n : 0);
  P.norm_w = (const _Float16*)norm_weight_f16;
  P.part_stride = 0;
  P.in_row_stride = 0;  // every row transforms the same input vector
  P.scale = scale;
  P.eps = eps;
  P.in_parts = 1;
  P.n = n;
  P.order = order;
  P.pre_mode = PRE_RMSNORM;
  return launch_rht(P, QTIP_F16, QTIP_F16, rows, stream);
}

int qtip_rht_chain(void* xt_out_f16, void* x_out_f16, const float* parts, int in_parts, int rows, int n,
                   const float* post_f32, float scale_out, const void* residual_f16,
                   const void* norm_weight_f16, float eps, const void* pre_f16, float scale_in,
                   void* stream) {
  if (!xt_out_f16 || !x_out_f16 || !parts || !residual_f16 || !norm_weight_f16) return QTIP_E_NULL;
  if (rows < 1 || rows > 65535 || in_parts < 1 || in_parts > kMaxParts) return QTIP_E_SHAPE;
  if (n != 2048 && n != 4096 && n != 8192) return QTIP_E_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const size_t stride = (size_t)rows * n;
#define QTIP_CHAIN(E)                                                                              \
  rht_chain_kernel<E><<<rows, kRhtThreads, 0, st>>>(                                               \
      (_Float16*)xt_out_f16, (_Float16*)x_out_f16, parts, in_parts, stride, post_f32, scale_out, \
      (const _Float16*)residual_f16, (const _Float16*)norm_weight_f16, eps, (const _Float16*)pre_f16, scale_in)
  switch (n) {
    case 2048: QTIP_CHAIN(2); break;
    case 4096: QTIP_CHAIN(4); break;
    default: QTIP_CHAIN(8); break;
  }
#undef QTIP_CHAIN
  return (int)hipGetLastError();
}

}  // extern "C"
