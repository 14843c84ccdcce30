// libqtip_hip.so: gfx950 kernels and C ABI for QTIP's quantized-linear
// inference path.  Declarations and the reference interfaces each entry
// point replaces are in include/qtip_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qtip_hip.h"
#include "qtip_device.h"

using namespace qtip;

namespace {

constexpr int kThreads = 1024;  // 16 waves per workgroup, one workgroup per CU
constexpr int kWaves = kThreads / 64;
constexpr int kMaxSplit = 16;

__device__ __forceinline__ float dpp_xor1(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1 /* quad_perm 1,0,3,2 */,
                                         0xF, 0xF, false));
}
__device__ __forceinline__ float swz_xor16(float v) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
__device__ __forceinline__ float xor32(float v) {
  uint32_t u = __builtin_bit_cast(uint32_t, v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  // r[0]: lanes 0-31 keep their value, lanes 32-63 receive lanes 0-31;
  // r[1]: lanes 0-31 receive lanes 32-63, lanes 32-63 keep theirs.
  const bool upper = (threadIdx.x & 32) != 0;
  return __builtin_bit_cast(float, upper ? r[0] : r[1]);
}

// ---------------------------------------------------------------------------
// decode: packed stream -> dense fp16 (m, k)
// ---------------------------------------------------------------------------
template <int K>
__global__ __launch_bounds__(kThreads, 1) void decode_kernel(uint16_t* __restrict__ out,
                                                             const uint8_t* __restrict__ packed,
                                                             const uint32_t* __restrict__ tlut,
                                                             int m, int k) {
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  build_lut(lut, tlut, threadIdx.x, kThreads);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = (uint32_t)a << 2;
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;
  const long total = (long)(m >> 5) * nwl;  // wave-loads in the matrix
  const size_t rb_bytes = (size_t)nkb * 128 * K;
  for (long w = (long)blockIdx.x * kWaves + wave; w < total; w += (long)gridDim.x * kWaves) {
    const int rb = (int)(w / nwl), wl = (int)(w - (long)rb * nwl);
    const int kb = 4 * wl + g;
    if (kb >= nkb) continue;
    const LaneData<K> ld =
        load_lane<K>(packed + (size_t)rb * rb_bytes + (size_t)kb * 128 * K + a * 8 * K);
    uint32_t st[2][4][4];
    lane_states<K>(ld, st);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int kh = t >> 1, mh = t & 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int jh = j >> 1, rh = j & 1;
        u32x2 v;
        v[0] = lut_lookup(lut, st[0][t][j], slot4);
        v[1] = lut_lookup(lut, st[1][t][j], slot4);
        const size_t row = (size_t)rb * 32 + 16 * mh + 8 * rh + (a >> 1);
        const size_t col = (size_t)kb * 32 + 16 * kh + 8 * jh + 4 * (a & 1);
        *reinterpret_cast<u32x2*>(out + row * k + col) = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// decompress + matvec
// ---------------------------------------------------------------------------
constexpr size_t kMatvecLds = kLut128Bytes + 2 * kWaves * 32 * sizeof(float);
constexpr size_t kMatvecXBytes = 28 * 1024;  // LDS left for the x values of a workgroup's k range

// 32 states of one wave-load.  All hashes, addresses and the 32 table reads
// are issued first and the 32 dot products follow, so a read has the rest of
// the address arithmetic (a few hundred cycles) to come back from LDS.
// slot4 = LDS address of the table + 4 * (lane % 32);
// acc[2*mh + rh] belongs to row 16*mh + 8*rh + a/2 of the 32-row block.
template <int K>
__device__ __forceinline__ void matvec_accumulate(const LaneData<K>& ld, const u32x2 xv[4],
                                                  uint32_t slot4, float acc[4]) {
  uint32_t P[16], W[32];
  packed_states<K>(ld, P);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t q = pk_hash(P[i]) & 0xFFC0FFC0u;
#if defined(QTIP_ABLATE_LDS)
    W[2 * i] = lut128_addr_lo(q, slot4);
    W[2 * i + 1] = lut128_addr_hi(q, slot4);
#else
    W[2 * i] = lds_word_abs(lut128_addr_lo(q, slot4));
    W[2 * i + 1] = lds_word_abs(lut128_addr_hi(q, slot4));
#endif
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int R = PkMeta<K>::R(i);
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      // (copy the vector element to a scalar first: bit_cast applied directly
      // to a vector-element lvalue reads element 0)
      const uint32_t xr = xv[PkMeta<K>::xq(i, hh)][R];
      acc[PkMeta<K>::acc(i, hh)] =
          __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, W[2 * i + hh]),
                                 __builtin_bit_cast(half2_t, xr), acc[PkMeta<K>::acc(i, hh)], false);
    }
  }
}

// Buffer-addressed streaming loads: the address is (SGPR descriptor, SGPR byte
// offset, per-lane VGPR offset), so walking the stream costs no vector ALU work.
template <int K>
__device__ __forceinline__ LaneData<K> load_lane_buf(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff,
                                                     uint32_t soff) {
  LaneData<K> r;
  constexpr int NT = 2;  // non-temporal: the stream is read once
  if constexpr (K == 2) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, NT);
#pragma unroll
    for (int i = 0; i < 4; ++i) r.d[i] = v[i];
  } else if constexpr (K == 3) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, NT);
    const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff + 16, soff, NT);
#pragma unroll
    for (int i = 0; i < 4; ++i) r.d[i] = v[i];
    r.d[4] = w[0];
    r.d[5] = w[1];
  } else {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, NT);
    const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff + 16, soff, NT);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r.d[i] = v[i];
      r.d[4 + i] = w[i];
    }
  }
  return r;
}

// x for a lane's columns of a wave-load: 4 x (4 consecutive fp16), 16 bytes apart
__device__ __forceinline__ void load_x_buf(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff,
                                           u32x2 xv[4]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) xv[q] = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff + 16 * q, soff, 0);
}

__device__ __forceinline__ void load_x(const uint16_t* __restrict__ xw, uint32_t xoff, u32x2 xv[4]) {
  const uint8_t* p = reinterpret_cast<const uint8_t*>(xw) + xoff;
#pragma unroll
  for (int q = 0; q < 4; ++q) xv[q] = *reinterpret_cast<const u32x2*>(p + 16 * q);
}

// Work unit = (32-row block rb, k split s).  The 16 waves of a workgroup take
// the unit's wave-loads round-robin (so the workgroup streams one contiguous
// run of bytes), reduce across lanes with DPP / ds_swizzle / permlane swaps and
// across waves through LDS in a fixed order, and store 32 sums to
// dst[s*m + 32*rb ...]: the result itself when S == 1, else one of S partial
// vectors that the consumer adds in order (deterministic either way).
//
// The launcher makes gridDim.x a multiple of S: a workgroup keeps one k range
// [wl0, wl1) and walks row blocks rb0, rb0 + rb_step, ...  A wave sees its work
// as a flat sequence of items (unit i, j) with wave-load wl0 + wave + 16*j;
// every unit has npw items per wave of which the first nvj are real (the same
// count in every unit).  DEPTH items are in flight; the prefetch runs ahead
// across unit boundaries and every load in the loop is unconditional (a
// conditional prefetch makes the compiler wait for it at once): padding items
// fetch offset 0 and are skipped by the arithmetic.
// XLDS: the x values of the workgroup's k range are staged in LDS once
// (needs 256 bytes per wave-load of the range) and read from there.
template <int K, int DEPTH, bool XLDS>
__global__ __launch_bounds__(kThreads, 1) void matvec_kernel(
    float* __restrict__ dst, const uint8_t* __restrict__ packed, const uint16_t* __restrict__ x,
    const uint32_t* __restrict__ tlut, int m, int k, int S, int wl_per) {
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  float* part = reinterpret_cast<float*>(smem + kLut128Bytes);  // [2][kWaves][32]
  uint8_t* xs_lds = smem + kLut128Bytes + 2 * kWaves * 32 * sizeof(float);  // [wl_per][256] when XLDS
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lives in an SGPR
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = lds_address(lut) + ((uint32_t)(lane & 31) << 2);
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;  // wave-loads per row block, the last may be partial
  const int nfull = nkb >> 2;      // full wave-loads per row block
  const int nrb = m >> 5;
  const uint32_t rb_bytes = (uint32_t)nkb * 128 * K;
  constexpr uint32_t WL_BYTES = 512 * K;
  const uint32_t loff = (uint32_t)lane * 8 * K;                // lane's bytes inside a wave-load
  const uint32_t xoff = (uint32_t)(32 * g + 4 * (a & 1)) * 2;  // lane's x bytes inside a wave-load

  const int s = blockIdx.x % S;
  const int rb0 = blockIdx.x / S;
  const int rb_step = gridDim.x / S;
  const int wl0 = s * wl_per;
  const int wl1 = wl0 + wl_per < nwl ? wl0 + wl_per : nwl;
  const int wl1f = wl1 < nfull ? wl1 : nfull;           // end of the full wave-loads
  const int npw = (wl_per + kWaves - 1) / kWaves;       // items per wave and unit (padded)
  const int upw = (nrb - rb0 + rb_step - 1) / rb_step;  // units of this workgroup
  const int T = upw * npw;
  const int w_first = wl0 + wave;
  const int nvj = w_first < wl1f ? (wl1f - w_first + kWaves - 1) / kWaves : 0;  // real items per unit
  const bool tail_wave = wl1 > nfull && ((nfull - wl0) % kWaves) == wave;
  float* out_s = dst + (size_t)s * m;

  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(packed), 0, (int)((size_t)nrb * rb_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(x), 0, k * 2, 0x00020000);

  // load cursor: unit l_i (row block l_rb), item l_j
  int l_j = 0, l_t = 0;
  uint32_t l_rboff = (uint32_t)rb0 * rb_bytes;
  const uint32_t rb_step_bytes = (uint32_t)rb_step * rb_bytes;
  LaneData<K> buf[DEPTH];
  u32x2 xbuf[XLDS ? 1 : DEPTH][4];
  auto issue = [&](int d) {
    const bool valid = l_j < nvj && l_t < T;
    const uint32_t wl = (uint32_t)(w_first + l_j * kWaves);
    const uint32_t woff = valid ? l_rboff + wl * WL_BYTES : 0u;
    const uint32_t xw = valid ? wl * 256u : 0u;
    buf[d] = load_lane_buf<K>(rs_w, loff, woff);
    if constexpr (!XLDS) load_x_buf(rs_x, xoff, xw, xbuf[d]);
    ++l_t;
    if (++l_j == npw) {
      l_j = 0;
      l_rboff += rb_step_bytes;
    }
  };
  // the first loads go out before the table is built
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) issue(d);

  build_lut128(lut, tlut, tid, kThreads);
  if constexpr (XLDS) {
    // x of wave-loads [wl0, wl1): 16 bytes per thread and pass
    const int xbytes = (wl1 - wl0) * 256;
    const int kbytes = k * 2;
    for (int o = tid * 16; o < xbytes; o += kThreads * 16) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (wl0 * 256 + o < kbytes)
        v = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint8_t*>(x) + (size_t)wl0 * 256 + o);
      *reinterpret_cast<u32x4*>(xs_lds + o) = v;
    }
  }
  __syncthreads();
  const uint32_t xs_lane = lds_address(xs_lds) + xoff + (uint32_t)wave * 256u;  // wave-load w_first

  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  int parity = 0, c_j = 0, c_rb = rb0;
  for (int t = 0; t < T; t += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (t + d < T) {
        if (c_j < nvj) {
          if constexpr (XLDS) {
            typedef __attribute__((address_space(3))) const u32x2 lds_u32x2_t;
            u32x2 xv[4];
            const uint32_t xa = xs_lane + (uint32_t)c_j * (kWaves * 256u);
#pragma unroll
            for (int q = 0; q < 4; ++q) xv[q] = *(lds_u32x2_t*)(uintptr_t)(xa + 16u * q);
            matvec_accumulate<K>(buf[d], xv, slot4, acc);
          } else {
            matvec_accumulate<K>(buf[d], xbuf[d], slot4, acc);
          }
        }
      }
      // the stage's registers are refilled only after their last use, so the
      // refill reuses them in place (no copies, no wait on the new load)
      issue(d);
      if (t + d < T && ++c_j == npw) {
        // ---- end of a unit: ragged tail, reductions, store
        // k/32 not a multiple of 4: one wave takes the partial wave-load with
        // the lanes of the missing blocks switched off
        if (tail_wave && 4 * nfull + g < nkb) {
          u32x2 xt[4];
          load_x(x + (size_t)nfull * 128, xoff, xt);
          const LaneData<K> tail =
              load_lane<K>(packed + (size_t)c_rb * rb_bytes + (size_t)nfull * WL_BYTES + loff);
          matvec_accumulate<K>(tail, xt, slot4, acc);
        }
        float* pp = part + parity * (kWaves * 32);
        // lanes sharing a row differ in lane bits 0 (column half), 4 and 5 (block)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = acc[i];
          v += dpp_xor1(v);
          v += swz_xor16(v);
          v += xor32(v);
          if (g == 0 && (a & 1) == 0) pp[wave * 32 + (i >> 1) * 16 + (i & 1) * 8 + (a >> 1)] = v;
          acc[i] = 0.f;
        }
        __syncthreads();
        if (tid < 32) {
          float sum = 0.f;
#pragma unroll
          for (int w = 0; w < kWaves; ++w) sum += pp[w * 32 + tid];
          out_s[c_rb * 32 + tid] = sum;
        }
        parity ^= 1;  // the other buffer is free: its readers passed the barrier above
        c_j = 0;
        c_rb += rb_step;
      }
    }
  }
}

// out[i] = parts[0][i] + parts[1][i] + ... in that order
__global__ __launch_bounds__(256) void sum_parts_kernel(float* __restrict__ out,
                                                        const float* __restrict__ parts, int m,
                                                        int S) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= m) return;
  float sum = parts[i];
  for (int s = 1; s < S; ++s) sum += parts[(size_t)s * m + i];
  out[i] = sum;
}

// ---------------------------------------------------------------------------
// batched decompress -> LDS -> fp16 MFMA GEMM
// ---------------------------------------------------------------------------
constexpr int kGemmThreads = 512;
constexpr int kGemmWaves = kGemmThreads / 64;
constexpr int kStageStride = 128 + 8;                  // halfs per staged row (padding vs banks)
constexpr int kStageHalfs = 32 * kStageStride;         // one wave's 32 x 128 tile
constexpr int kStageBytes = kStageHalfs * 2;           // 8704

// out[b][row] for b < batch.  NB = number of 16-wide batch tiles per pass.
template <int K, int NB>
__global__ __launch_bounds__(kGemmThreads, 1) void gemm_kernel(
    float* __restrict__ out, const uint8_t* __restrict__ packed, const uint16_t* __restrict__ x,
    const uint32_t* __restrict__ tlut, int m, int k, int batch, int round_f16) {
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  uint8_t* stage_all = smem + kLutBytes;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = (uint32_t)a << 2;
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;
  const size_t rb_bytes = (size_t)nkb * 128 * K;
  const int nrb = m >> 5;
  constexpr int WL_BYTES = 512 * K;
  uint16_t* stage = reinterpret_cast<uint16_t*>(stage_all + wave * kStageBytes);
  float* red = reinterpret_cast<float*>(stage_all);  // reused after the k loop

  build_lut(lut, tlut, tid, kGemmThreads);
  __syncthreads();

  const int row16 = lane & 15, kgrp = lane >> 4;  // MFMA operand coordinates

  for (int rb = blockIdx.x; rb < nrb; rb += gridDim.x) {
    const uint8_t* base = packed + (size_t)rb * rb_bytes + (size_t)g * 128 * K + a * 8 * K;
    float4_t acc[2][NB];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[mt][nb] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int wl = wave; wl < nwl; wl += kGemmWaves) {
      const int kb = 4 * wl + g;
      const bool active = kb < nkb;
      uint32_t st[2][4][4];
      if (active) {
        const LaneData<K> ld = load_lane<K>(base + (size_t)wl * WL_BYTES);
        lane_states<K>(ld, st);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int kh = t >> 1, mh = t & 1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int jh = j >> 1, rh = j & 1;
          u32x2 v = {0u, 0u};
          if (active) {
            v[0] = lut_lookup(lut, st[0][t][j], slot4);
            v[1] = lut_lookup(lut, st[1][t][j], slot4);
          }
          const int row = 16 * mh + 8 * rh + (a >> 1);
          const int col = 32 * g + 16 * kh + 8 * jh + 4 * (a & 1);
          *reinterpret_cast<u32x2*>(stage + row * kStageStride + col) = v;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const size_t kcol0 = (size_t)wl * 128;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int kc = 32 * ks + 8 * kgrp;
        half8_t bfrag[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int b = 16 * nb + row16;
          u32x4 raw = {0u, 0u, 0u, 0u};
          if (b < batch && kcol0 + kc < (size_t)k)
            raw = *reinterpret_cast<const u32x4*>(x + (size_t)b * k + kcol0 + kc);
          bfrag[nb] = __builtin_bit_cast(half8_t, raw);
        }
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const half8_t afrag = *reinterpret_cast<const half8_t*>(
              stage + (16 * mt + row16) * kStageStride + kc);
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
            acc[mt][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag, bfrag[nb], acc[mt][nb], 0, 0, 0);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }

    // cross-wave reduction: red[wave][row 32][col 16*NB]
    __syncthreads();
    constexpr int NC = 16 * NB;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          red[(wave * 32 + 16 * mt + 4 * kgrp + i) * NC + 16 * nb + row16] = acc[mt][nb][i];
    __syncthreads();
    for (int e = tid; e < 32 * NC; e += kGemmThreads) {
      const int b = e >> 5, row = e & 31;  // consecutive threads -> consecutive rows of out
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kGemmWaves; ++w) sum += red[(w * 32 + row) * NC + b];
      if (round_f16) sum = (float)(_Float16)sum;
      if (b < batch) out[(size_t)b * m + rb * 32 + row] = sum;
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct DeviceInfo {
  int cus = 0;
  bool ok = false;
};

// One-time per-process set-up (CU count, LDS opt-in).  Runs on the first call
// of any launcher; callers that record HIP graphs make one eager call first.
DeviceInfo& device_info() {
  static DeviceInfo info = [] {
    DeviceInfo d;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return d;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      return d;
    d.cus = cus > 0 ? cus : 256;
    d.ok = true;
    return d;
  }();
  return info;
}

template <typename F>
hipError_t allow_lds(F* fn, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(fn),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

constexpr size_t kGemmLds = kLutBytes + kGemmWaves * kStageBytes;

hipError_t setup_once() {
  static hipError_t status = [] {
    hipError_t e;
#define QTIP_ALLOW(fn, bytes) \
  if ((e = allow_lds(fn, bytes)) != hipSuccess) return e;
    QTIP_ALLOW((decode_kernel<2>), kLutBytes)
    QTIP_ALLOW((decode_kernel<3>), kLutBytes)
    QTIP_ALLOW((decode_kernel<4>), kLutBytes)
    QTIP_ALLOW((matvec_kernel<2, 4, false>), kMatvecLds)
    QTIP_ALLOW((matvec_kernel<3, 3, false>), kMatvecLds)
    QTIP_ALLOW((matvec_kernel<4, 2, false>), kMatvecLds)
    QTIP_ALLOW((matvec_kernel<2, 6, true>), kMatvecLds + kMatvecXBytes)
    QTIP_ALLOW((matvec_kernel<3, 4, true>), kMatvecLds + kMatvecXBytes)
    QTIP_ALLOW((matvec_kernel<4, 3, true>), kMatvecLds + kMatvecXBytes)
    QTIP_ALLOW((gemm_kernel<2, 1>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<2, 2>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<2, 4>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<3, 1>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<3, 2>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<3, 4>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<4, 1>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<4, 2>), kGemmLds)
    QTIP_ALLOW((gemm_kernel<4, 4>), kGemmLds)
#undef QTIP_ALLOW
    return hipSuccess;
  }();
  return status;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_common(const void* a, const void* b, const void* c, const void* d, int m, int k,
                 int bits) {
  if (!a || !b || !c || !d) return QTIP_E_NULL;
  if (bits < 2 || bits > 4) return QTIP_E_SHAPE;
  if (m <= 0 || k <= 0 || (m & 31) || (k & 31)) return QTIP_E_SHAPE;
  if ((long)m * k * bits / 8 >= (1L << 31)) return QTIP_E_SHAPE;  // 32-bit buffer offsets
  return QTIP_OK;
}

// k split so that (m/32)*S units fill the machine evenly
int choose_split(int m, int k, int bits, int cus) {
  const int nrb = m >> 5;
  const int nwl = ((k >> 5) + 3) >> 2;
  int best = 1;
  double best_cost = 1e30;
  for (int S = 1; S <= kMaxSplit; S *= 2) {
    if (nwl / S < kWaves && S > 1) break;  // keep at least one wave-load per wave
    const long units = (long)nrb * S;
    const long rounds = (units + cus - 1) / cus;
    // cost: rounds * (unit bytes + fixed per-unit overhead expressed in bytes)
    const double unit_bytes = (double)nwl / S * 512.0 * bits;
    const double cost = rounds * (unit_bytes + 12288.0 + (S > 1 ? 4096.0 : 0.0));
    if (cost < best_cost * 0.97) {
      best_cost = cost;
      best = S;
    }
  }
  return best;
}

}  // namespace

extern "C" {

int qtip_abi_version(void) { return 3; }

const char* qtip_error_string(int code) {
  switch (code) {
    case QTIP_OK: return "ok";
    case QTIP_E_SHAPE: return "qtip: unsupported shape (need m % 32 == 0, k % 32 == 0, bits in 2..4, sizes in range)";
    case QTIP_E_NULL: return "qtip: null pointer argument";
    case QTIP_E_ALIGN: return "qtip: pointer not 16-byte aligned";
    case QTIP_E_WORKSPACE: return "qtip: workspace too small";
    case QTIP_E_DTYPE: return "qtip: unknown dtype code";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "qtip: unknown error";
  }
}

int qtip_decode(void* out_f16, const void* packed, const void* tlut, int m, int k, int bits,
                void* stream) {
  int rc = check_common(out_f16, packed, tlut, tlut, m, k, bits);
  if (rc) return rc;
  if (!aligned16(out_f16) || !aligned16(packed) || (reinterpret_cast<uintptr_t>(tlut) & 3u))
    return QTIP_E_ALIGN;
  DeviceInfo& di = device_info();
  if (!di.ok) return (int)hipErrorInvalidDevice;
  hipError_t e = setup_once();
  if (e != hipSuccess) return (int)e;
  const long total = (long)(m >> 5) * (((k >> 5) + 3) >> 2);
  long want = (total + kWaves - 1) / kWaves;
  const int grid = (int)(want < di.cus ? want : di.cus);
  hipStream_t st = (hipStream_t)stream;
  auto* o = (uint16_t*)out_f16;
  auto* p = (const uint8_t*)packed;
  auto* t = (const uint32_t*)tlut;
  switch (bits) {
    case 2: decode_kernel<2><<<grid, kThreads, kLutBytes, st>>>(o, p, t, m, k); break;
    case 3: decode_kernel<3><<<grid, kThreads, kLutBytes, st>>>(o, p, t, m, k); break;
    default: decode_kernel<4><<<grid, kThreads, kLutBytes, st>>>(o, p, t, m, k); break;
  }
  return (int)hipGetLastError();
}

int qtip_matvec_split(int m, int k, int bits) {
  if (m <= 0 || k <= 0 || (m & 31) || (k & 31) || bits < 2 || bits > 4) return 0;
  DeviceInfo& di = device_info();
  if (!di.ok) return 0;
  return choose_split(m, k, bits, di.cus);
}

size_t qtip_matvec_workspace_bytes(int m, int k, int bits) {
  const int S = qtip_matvec_split(m, k, bits);
  return S > 1 ? (size_t)S * m * sizeof(float) : 0;
}

static int launch_matvec(float* dst, const void* packed, const void* x_f16, const void* tlut, int m,
                         int k, int bits, int S, hipStream_t st) {
  DeviceInfo& di = device_info();
  const long units = (long)(m >> 5) * S;
  long grid = units < di.cus ? units : di.cus;
  grid -= grid % S;  // a workgroup keeps one k range (units is a multiple of S, so grid >= S)
  const int nwl = ((k >> 5) + 3) >> 2;
  const int wl_per = (nwl + S - 1) / S;
  auto* p = (const uint8_t*)packed;
  auto* xx = (const uint16_t*)x_f16;
  auto* t = (const uint32_t*)tlut;
  const size_t xbytes = (size_t)wl_per * 256;
  if (xbytes <= kMatvecXBytes) {
    const size_t lds = kMatvecLds + xbytes;
    switch (bits) {
      case 2: matvec_kernel<2, 6, true><<<(int)grid, kThreads, lds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
      case 3: matvec_kernel<3, 4, true><<<(int)grid, kThreads, lds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
      default: matvec_kernel<4, 3, true><<<(int)grid, kThreads, lds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
    }
  } else {
    switch (bits) {
      case 2: matvec_kernel<2, 4, false><<<(int)grid, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
      case 3: matvec_kernel<3, 3, false><<<(int)grid, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
      default: matvec_kernel<4, 2, false><<<(int)grid, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, S, wl_per); break;
    }
  }
  return (int)hipGetLastError();
}

static int check_matvec(const void* out, const void* packed, const void* x_f16, const void* tlut,
                        int m, int k, int bits) {
  int rc = check_common(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (!aligned16(packed) || (reinterpret_cast<uintptr_t>(x_f16) & 7u) ||
      (reinterpret_cast<uintptr_t>(tlut) & 3u) || (reinterpret_cast<uintptr_t>(out) & 3u))
    return QTIP_E_ALIGN;
  if (!device_info().ok) return (int)hipErrorInvalidDevice;
  hipError_t e = setup_once();
  return e == hipSuccess ? QTIP_OK : (int)e;
}

int qtip_decompress_matvec_parts(float* parts, const void* packed, const void* x_f16,
                                 const void* tlut, int m, int k, int bits, int nparts,
                                 void* stream) {
  int rc = check_matvec(parts, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (nparts < 1 || nparts > kMaxSplit || nparts > ((((k >> 5) + 3) >> 2))) return QTIP_E_SHAPE;
  return launch_matvec(parts, packed, x_f16, tlut, m, k, bits, nparts, (hipStream_t)stream);
}

int qtip_decompress_matvec(float* out, const void* packed, const void* x_f16, const void* tlut,
                           int m, int k, int bits, void* workspace, size_t workspace_bytes,
                           void* stream) {
  int rc = check_matvec(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  int S = 1;
  if (workspace) {
    S = choose_split(m, k, bits, device_info().cus);
    if (S > 1 && workspace_bytes < (size_t)S * m * sizeof(float)) return QTIP_E_WORKSPACE;
    if (!aligned16(workspace)) return QTIP_E_ALIGN;
  }
  hipStream_t st = (hipStream_t)stream;
  if (S == 1) return launch_matvec(out, packed, x_f16, tlut, m, k, bits, 1, st);
  rc = launch_matvec((float*)workspace, packed, x_f16, tlut, m, k, bits, S, st);
  if (rc) return rc;
  sum_parts_kernel<<<(m + 255) / 256, 256, 0, st>>>(out, (const float*)workspace, m, S);
  return (int)hipGetLastError();
}

int qtip_decompress_gemm(float* out, const void* packed, const void* x_f16, const void* tlut,
                         int m, int k, int bits, int batch, int round_f16, void* stream) {
  int rc = check_common(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (batch < 1 || batch > 65535) return QTIP_E_SHAPE;
  if (!aligned16(packed) || !aligned16(x_f16) || (reinterpret_cast<uintptr_t>(tlut) & 3u) ||
      (reinterpret_cast<uintptr_t>(out) & 3u))
    return QTIP_E_ALIGN;
  DeviceInfo& di = device_info();
  if (!di.ok) return (int)hipErrorInvalidDevice;
  hipError_t e = setup_once();
  if (e != hipSuccess) return (int)e;
  const int nrb = m >> 5;
  const int grid = nrb < di.cus ? nrb : di.cus;
  hipStream_t st = (hipStream_t)stream;
  auto* p = (const uint8_t*)packed;
  auto* t = (const uint32_t*)tlut;
  // batch handled in passes of at most 64 rows
  for (int b0 = 0; b0 < batch; b0 += 64) {
    const int nb = batch - b0 < 64 ? batch - b0 : 64;
    float* o = out + (size_t)b0 * m;
    const uint16_t* xx = (const uint16_t*)x_f16 + (size_t)b0 * k;
#define QTIP_GEMM(KB, NBT) \
  gemm_kernel<KB, NBT><<<grid, kGemmThreads, kGemmLds, st>>>(o, p, xx, t, m, k, nb, round_f16)
#define QTIP_GEMM_K(KB)            \
  if (nb <= 16) QTIP_GEMM(KB, 1);  \
  else if (nb <= 32) QTIP_GEMM(KB, 2); \
  else QTIP_GEMM(KB, 4);
    switch (bits) {
      case 2: QTIP_GEMM_K(2) break;
      case 3: QTIP_GEMM_K(3) break;
      default: QTIP_GEMM_K(4) break;
    }
#undef QTIP_GEMM_K
#undef QTIP_GEMM
    hipError_t le = hipGetLastError();
    if (le != hipSuccess) return (int)le;
  }
  return QTIP_OK;
}

}  // extern "C"
