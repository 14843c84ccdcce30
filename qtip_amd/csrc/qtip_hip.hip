// libqtip_hip.so: gfx950 kernels and C ABI for QTIP's quantized-linear
// inference path.  Declarations and the reference interfaces each entry
// point replaces are in include/qtip_hip.h.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <type_traits>

#include "../../include/qtip_hip.h"
#include "qtip_device.h"
#include "qtip_wht.h"

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
// ---------------------------------------------------------------------------
// decode: packed stream -> dense fp16 (m, k)
//
// Write-bound (2 bytes out per K/8 bytes in), so what matters is the shape of the stores.  A lane
// decodes 4-column pieces of 16 different rows; stored as they come, a row of the matrix receives
// 8 bytes per lane and the memory system sees partial cache lines (measured 2.4 TB/s against
// 6.9 TB/s for a fill).  Each wave therefore turns its wave-load (32 rows x 128 columns) round
// in LDS, a quarter (8 rows x 256 bytes) at a time: pieces go in with the 16-byte chunk index
// xor-ed with the row (conflict free both ways), come back as one 16-byte chunk per lane, and a
// store instruction writes four 256-byte row segments - whole cache lines only.  The 128 KiB
// table of the matvec (32 replicas, one bank per lane) serves the lookups; the next wave-load
// of the stream is requested before the current one is decoded.
// ---------------------------------------------------------------------------
constexpr size_t kDecodeLds = kLut128Bytes + kWaves * 2048;

template <int K>
__global__ __launch_bounds__(kThreads, 1) void decode_kernel(uint16_t* __restrict__ out,
                                                             const uint8_t* __restrict__ packed,
                                                             const uint32_t* __restrict__ tlut,
                                                             int m, int k) {
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  build_lut128(lut, tlut, threadIdx.x, kThreads);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = lds_address(lut) + ((uint32_t)(lane & 31) << 2);
  uint8_t* stage = smem + kLut128Bytes + wave * 2048;  // this wave's [8 rows][256 bytes]
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;
  const long total = (long)(m >> 5) * nwl;  // wave-loads in the matrix
  const size_t rb_bytes = (size_t)nkb * 128 * K;
  const long step = (long)gridDim.x * kWaves;
  auto fetch = [&](long ww) {
    const long wc = ww < total ? ww : total - 1;
    const int rb = (int)(wc / nwl), wl = (int)(wc - (long)rb * nwl);
    int kb = 4 * wl + g;
    kb = kb < nkb ? kb : nkb - 1;  // blocks past the row's end (k / 32 not a multiple of 4) are decoded but not stored
    return load_lane<K>(packed + (size_t)rb * rb_bytes + (size_t)kb * 128 * K + a * 8 * K);
  };
  // The stream is requested NB wave-loads ahead.  (Loads and stores share one in-order completion
  // counter, so a wait for a requested wave-load also waits for the stores issued before the
  // request; requesting 2, 4 or 8 wave-loads at a time to meet that wait less often measured no
  // faster - the memory system, not the wave, holds the stores back.)
  constexpr int NB = 1;
  long w = (long)blockIdx.x * kWaves + wave;
  LaneData<K> cur[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b) cur[b] = fetch(w + b * step);
  // piece (kh, jh) of this lane inside a quarter, and the chunk it reads back
  const int r8 = a >> 1;
  const int row_rd = lane >> 4, c_rd = lane & 15;
  for (; w < total; w += NB * step) {
    LaneData<K> nxt[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) nxt[b] = fetch(w + (NB + b) * step);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const long wb = w + b * step;
      if (wb >= total) break;  // the same for every lane of the wave
      const int rb = (int)(wb / nwl), wl = (int)(wb - (long)rb * nwl);
      uint32_t P[16], W[32];
      packed_states<K>(cur[b], P);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t q = pk_hash(P[i]) & 0xFFC0FFC0u;
        W[2 * i] = lds_word_abs(lut128_addr_lo(q, slot4));
        W[2 * i + 1] = lds_word_abs(lut128_addr_hi(q, slot4));
      }
      const bool store_ok = 4 * wl + (c_rd >> 2) < nkb;
#pragma unroll
      for (int mh = 0; mh < 2; ++mh)
#pragma unroll
        for (int rh = 0; rh < 2; ++rh) {
#pragma unroll
          for (int kh = 0; kh < 2; ++kh)
#pragma unroll
            for (int jh = 0; jh < 2; ++jh) {
              const int t = 2 * kh + mh, j = 2 * jh + rh;
              const int chunk = 4 * g + 2 * kh + jh;
              u32x2 v = {W[w_index<K>(0, t, j)], W[w_index<K>(1, t, j)]};
              *reinterpret_cast<u32x2*>(stage + r8 * 256 + ((chunk ^ r8) << 4) + 8 * (a & 1)) = v;
            }
          // the wave reads what its other lanes wrote: LDS serves a wave's requests in order
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const int r = row_rd + 4 * i;
            const u32x4 v = *reinterpret_cast<const u32x4*>(stage + r * 256 + ((c_rd ^ r) << 4));
            const size_t row = (size_t)rb * 32 + 16 * mh + 8 * rh + r;
            const size_t col = (size_t)wl * 128 + c_rd * 8;
            if (store_ok) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(out + row * k + col));
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) cur[b] = nxt[b];
  }
}

// ---------------------------------------------------------------------------
// decompress + matvec
// ---------------------------------------------------------------------------
constexpr size_t kMatvecLds = kLut128Bytes + 2 * kWaves * 32 * sizeof(float);
constexpr size_t kMatvecXBytes = 28 * 1024;  // LDS left for the x values of a workgroup's k range

// Buffer-addressed streaming loads: the address is (SGPR descriptor, SGPR byte
// offset, per-lane VGPR offset), so walking the stream costs no vector ALU work.
template <int K>
__device__ __forceinline__ LaneData<K> load_lane_buf(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff,
                                                     uint32_t soff) {
  LaneData<K> r;
  // Non-temporal where a load instruction covers whole cache lines (one 16-byte load per lane at 2
  // bits) or nearly so (3 bits): the stream is read once.  At 4 bits a lane's two 16-byte loads
  // split every line between two instructions, and with the hint the second one fetches the line
  // from L2 again: plain loads are 10 % faster there (57344x8192: 47.7 -> 41.5 us).
  constexpr int NT = K == 4 ? 0 : 2;
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

// Input transform of the layer inside the matvec prologue (k = 1024 * EPT a power of two):
// xs[e] = fp16(scale * (H_k (su * x))[e]) for the whole vector, written to LDS where the
// kernel keeps its activations.  Every workgroup computes the whole transform (a few thousand
// butterflies per thread, hidden behind the latency of the first weight loads) - it replaces
// a separate transform launch.  `xchg` (k + k/64 floats) is the table's LDS, not yet built.
// Element e = [wave 4][lane 6][i]: butterflies over the register bits, the six lane bits and,
// after one exchange through LDS that swaps the wave bits with the low four lane bits, the rest.
template <int EPT>
__device__ __forceinline__ void xform_prologue(const float v_in[8], float scale, float* xchg,
                                               _Float16* xs, int tid, int lane, int wave) {
  using namespace qtip_wht;
  float v[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = v_in[i];
  const int e_nat = tid * EPT;
  const int e_swp = (((lane & 15) << 6) | ((wave & 15) << 2) | (lane >> 4)) * EPT;
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xchg[xidx<EPT>(e_nat + i)] = v[i];
  __syncthreads();
  _Float16 o[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) o[i] = (_Float16)(wht_lanes(xchg[xidx<EPT>(e_swp + i)], 4, lane) * scale);
  st_f16<EPT>(xs + e_swp, o);
  __syncthreads();  // xchg is free for the table, xs is complete
}

// XFORM == 2: the whole boundary between two linear layers of a decoder in front of the matvec,
//   x_new = residual + fp16(scale_out * post * H_k (sum of the previous layer's partial results)),
//   x_t   = fp16(scale_in * H_k (su * RMSNorm(x_new) * norm_w)),    parts_out = hatW . x_t
// i.e. the output transform of the previous QuantizedLinear with the residual addition, the
// RMSNorm and the input transform of this one (what rht_chain_kernel does in a launch of its
// own).  Every workgroup recomputes the k-point boundary - a few microseconds of work on 1024
// threads, most of it while the first stream requests are in flight - and workgroup (0, 0)
// stores x_new for the layers that follow.
struct ChainArgs {
  const float* parts;        // [in_parts][k] fp32 partial results of the previous linear layer
  const float* post;         // its output sign vector times its scale (SV), k fp32
  const _Float16* residual;  // the residual stream, k fp16
  const _Float16* norm_w;    // RMSNorm weight, k fp16
  _Float16* x_out;           // the new residual stream, k fp16
  size_t part_stride;        // floats between partial results
  float scale_out, eps;
  int in_parts;
};
// Up to three matrices with the same k and bit width in one launch (the separate q / k / v or
// gate / up projections of a decoder layer): the workgroups blockIdx.y in
// [wg_begin[g], wg_begin[g + 1]) serve matrix g with its own stream, table, sign vector and
// output rows; everything else (k split, layer boundary, x_out) is shared.
struct GroupArgs {
  float* dst[3];              // first output row of the matrix inside a partial result
  const uint8_t* packed[3];
  const uint32_t* tlut[3];
  const uint16_t* su[3];
  const uint16_t* x[3];       // the matrices' own inputs (plain form; unused with a layer boundary)
  int m[3];
  int wg_begin[4];
  int upw_q[3], upw_r[3];
  size_t part_stride;         // floats between partial results
};
// Timeline build (-DQTIP_STAMPS, used by `bench.py --timeline` through a library of its own; the
// product library is built without it): waves 0 and 15 of every matvec workgroup keep a few
// readings of the 100 MHz constant clock in registers and wave 0 stores them when it ends, into
// the slot of its launch's shape, so that after a graph replay the buffer holds the last launch
// of every shape.
//   0 first instruction   1 table words picked   2 at the first barrier   3 past it
//   4 end of the kernel   5 first instruction of wave 15   15 first wave-load of wave 0 in registers
//   6-10 the transform / layer boundary of the prologue (see QTIP_STAMP_SV)
// (nothing is read inside the loop: a clock reading there makes every wait in it a full one; and
// only two waves read the clock: 4096 waves reading it at once queue up behind each other)
#ifdef QTIP_STAMPS
constexpr int kStampSlots = 64, kStampWgs = 256, kStampN = 16;
__device__ unsigned long long g_stamps[kStampSlots][kStampWgs][kStampN];
#define QTIP_STAMP_DECL unsigned long long stamp_v[kStampN] = {};
#define QTIP_STAMP(i) if (wave == 0 || (i == 0 && wave == kWaves - 1)) stamp_v[i] = __builtin_amdgcn_s_memrealtime();
#define QTIP_STAMP_FIRST_LOAD() if (wave == 0) { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH - 1)); stamp_v[15] = __builtin_amdgcn_s_memrealtime(); }
// inside the layer boundary of the prologue (sv = the kernel's stamp_v): 6 entered, 7 / 8 / 9 past its
// first / second / third barrier (first transform, RMSNorm sum, second transform), 10 left
#define QTIP_STAMP_SV(i) if (wave == 0 && sv) sv[i] = __builtin_amdgcn_s_memrealtime();
#define QTIP_STAMP_PTR stamp_v
#else
#define QTIP_STAMP_DECL
#define QTIP_STAMP(i)
#define QTIP_STAMP_FIRST_LOAD()
#define QTIP_STAMP_SV(i)
#define QTIP_STAMP_PTR nullptr
#endif
template <typename T>
__device__ __forceinline__ T pick3(const T (&a)[3], int g) {
  return g == 0 ? a[0] : (g == 1 ? a[1] : a[2]);
}

struct ChainRegs {  // a thread's operands, k / 1024 <= 8 consecutive elements each
  float v[8], pv[8], rv[8], wv[8], sv[8];
};

template <int EPT>
__device__ __forceinline__ void chain_load(const ChainArgs& c, const _Float16* su, int tid, int lane,
                                           int wave, ChainRegs& r) {
  using namespace qtip_wht;
  const int e_nat = tid * EPT;
  const int e_swp = (((lane & 15) << 6) | ((wave & 15) << 2) | (lane >> 4)) * EPT;
  // operands of the middle part in the swapped layout, the partial results in the natural one
  ld_f32<EPT>(c.post + e_swp, r.pv);
  ld_f16<EPT>(c.residual + e_swp, r.rv);
  ld_f16<EPT>(c.norm_w + e_swp, r.wv);
  ld_f16<EPT>(su + e_swp, r.sv);
  ld_f32<EPT>(c.parts + e_nat, r.v);
  for (int w = 1; w < c.in_parts; ++w) {
    float t[EPT];
    ld_f32<EPT>(c.parts + w * c.part_stride + e_nat, t);
#pragma unroll
    for (int i = 0; i < EPT; ++i) r.v[i] += t[i];
  }
}

// xbuf: k + k/64 floats of exchange buffer, wsum: 16 floats, xs: the k fp16 activations of the matvec
template <int EPT>
__device__ __forceinline__ void chain_compute(ChainRegs& r, const ChainArgs& c, float scale_in, float* xbuf,
                                              float* wsum, _Float16* xs, int tid, int lane, int wave,
                                              bool write_x, unsigned long long* sv = nullptr) {
  using namespace qtip_wht;
  constexpr int N = kThreads * EPT;
  (void)sv;
  QTIP_STAMP_SV(6)
  const int e_nat = tid * EPT;
  const int e_swp = (((lane & 15) << 6) | ((wave & 15) << 2) | (lane >> 4)) * EPT;
  float v[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = r.v[i];
  // ---- first transform (natural -> swapped layout)
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xbuf[xidx<EPT>(e_nat + i)] = v[i];
  __syncthreads();
  QTIP_STAMP_SV(7)
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(xbuf[xidx<EPT>(e_swp + i)], 4, lane);
  // ---- residual, RMSNorm, sign vector of this layer
  float ss = 0.f;
  _Float16 xn[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const float o = v[i] * c.scale_out * r.pv[i];
    xn[i] = (_Float16)(r.rv[i] + (float)(_Float16)o);
    v[i] = (float)xn[i];
    ss += v[i] * v[i];
  }
  if (write_x) st_f16<EPT>(c.x_out + e_swp, xn);
  ss = wave_sum(ss);
  if (lane == 0) wsum[wave] = ss;
  __syncthreads();  // also: every read of xbuf above is done
  QTIP_STAMP_SV(8)
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < 16; ++w) tot += wsum[w];
  const float rs = __builtin_amdgcn_rsqf(tot / (float)N + c.eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = (float)(_Float16)(r.wv[i] * (float)(_Float16)(v[i] * rs)) * r.sv[i];
  // ---- second transform (swapped -> natural layout)
  wht_regs<EPT>(v);
#pragma unroll
  for (int i = 0; i < EPT; ++i) v[i] = wht_lanes(v[i], 6, lane);
#pragma unroll
  for (int i = 0; i < EPT; ++i) xbuf[xidx<EPT>(e_swp + i)] = v[i];
  __syncthreads();
  QTIP_STAMP_SV(9)
  // the bits still missing are the top four of the element's lane field = lane bits 2..5 here
  _Float16 xo[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    float y = xbuf[xidx<EPT>(e_nat + i)];
    y = wht_lanes(y, 6, lane, 2);
    xo[i] = (_Float16)(y * scale_in);
  }
  st_f16<EPT>(xs + e_nat, xo);
  __syncthreads();  // the exchange buffer is free for the table, xs is complete
  QTIP_STAMP_SV(10)
}

// Work unit = (32-row block rb, k split s).  The 16 waves of a workgroup take
// the unit's wave-loads round-robin (so the workgroup streams one contiguous
// run of bytes), reduce across the four blocks of a wave-load inside the MFMA, across the two
// column halves with one DPP exchange and across waves through LDS in a fixed order, and store 32 sums to
// dst[s*m + 32*rb ...]: the result itself when S == 1, else one of S partial
// vectors that the consumer adds in order (deterministic either way).
//
// The launcher's grid is (S, workgroups per k range): a workgroup keeps one k range
// [wl0, wl1) and walks row blocks rb0, rb0 + rb_step, ...  A wave sees its work
// as a flat sequence of items (unit i, j) with wave-load wl0 + wave + 16*j;
// every unit has npw items per wave of which the first nvj are real (the same
// count in every unit).  DEPTH items are in flight; the prefetch runs ahead
// across unit boundaries and every load in the loop is unconditional (a
// conditional prefetch makes the compiler wait for it at once): padding items
// use an out-of-range lane offset (the load returns zeros without a memory
// access) and are skipped by the arithmetic.
// XLDS: the x values of the workgroup's k range are staged in LDS once
// (needs 256 bytes per wave-load of the range) and read from there.
// XFORM: 0 = x is the matvec's fp16 input, 1 = x is the layer's raw input (input transform in the
// prologue), 2 = the previous layer's partial results (whole layer boundary in the prologue).
// XHALF: the k range needs up to twice the staging area and every workgroup has exactly one unit:
// x is staged in two halves, the second replacing the first in the middle of the unit (two more
// barriers per launch instead of x travelling through vector loads with every wave-load, which
// made the 28672-wide matrices 15-20 % slower).
// HALF: the row blocks that do not fill a last round of whole units (at most half a round of
// them) are cut by row half instead: workgroup w < upw_r takes the rows with rh = w % 2 of row
// block upw_q * rb_step + w / 2 after its upw_q whole units.  Such a half unit reads the block's
// whole stream but decodes half of its states (about 0.55 of a unit's time), and its rows are
// complete sums, so nothing has to be combined across workgroups: 320 row blocks on 256
// workgroups take 1.55 units of time instead of 2, 128 row blocks 0.55 instead of 1.
template <int K, int DEPTH, bool XLDS, int XFORM = 0, bool XHALF = false, bool GROUP = false, bool HALF = false>
__global__ __launch_bounds__(kThreads, 1) void matvec_kernel(
    float* __restrict__ dst_, const uint8_t* __restrict__ packed_, const uint16_t* __restrict__ x_,
    const uint32_t* __restrict__ tlut_, int m_, int k, int wl_per, int upw_q_, int upw_r_,
    const uint16_t* __restrict__ su_ = nullptr, float xscale = 1.f, const ChainArgs chain = ChainArgs{},
    const GroupArgs grp = GroupArgs{}) {
  static_assert(!XFORM || XLDS, "the transformed activations live in LDS");
  static_assert(!GROUP || XFORM == 2 || (XFORM == 0 && XLDS && !XHALF),
                "grouped launches exist for the layer-boundary form and the plain form with x in LDS");
  // the matrix this workgroup serves (uniform: scalar selects on kernel arguments)
  int gi = 0;
  if constexpr (GROUP) gi = (int)blockIdx.y >= grp.wg_begin[2] ? 2 : ((int)blockIdx.y >= grp.wg_begin[1] ? 1 : 0);
  float* __restrict__ dst = GROUP ? pick3(grp.dst, gi) : dst_;
  const uint8_t* __restrict__ packed = GROUP ? pick3(grp.packed, gi) : packed_;
  const uint32_t* __restrict__ tlut = GROUP ? pick3(grp.tlut, gi) : tlut_;
  const uint16_t* __restrict__ su = GROUP ? pick3(grp.su, gi) : su_;
  const uint16_t* __restrict__ x = (GROUP && XFORM == 0) ? pick3(grp.x, gi) : x_;
  const int m = GROUP ? pick3(grp.m, gi) : m_;
  const int upw_q = GROUP ? pick3(grp.upw_q, gi) : upw_q_;
  const int upw_r = GROUP ? pick3(grp.upw_r, gi) : upw_r_;
  static_assert(!XHALF || (XLDS && !XFORM), "two-half staging is a form of the plain staged x");
  static_assert(!HALF || (XLDS && !XFORM && !XHALF && !GROUP), "half units exist for the plain form with x in LDS");
  // wave-loads requested before the table is built.  With half units both: a half wave-load is
  // decoded in half the time, which no longer covers the latency of a load requested after the barrier.
  constexpr int FIRST = (DEPTH > 2 || HALF) ? 2 : 1;
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  float* part = reinterpret_cast<float*>(smem + kLut128Bytes);  // [2][kWaves][32]
  uint8_t* xs_lds = smem + kLut128Bytes + 2 * kWaves * 32 * sizeof(float);  // [wl_per][256] when XLDS
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, lives in an SGPR
  QTIP_STAMP_DECL
  QTIP_STAMP(0)
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

  // grid = (S, workgroups per k range): no integer division on the way to the first loads
  const int s = blockIdx.x;
  const int wg0 = GROUP ? (gi == 0 ? 0 : (gi == 1 ? grp.wg_begin[1] : grp.wg_begin[2])) : 0;
  const int rb0 = (int)blockIdx.y - wg0;
  const int rb_step = GROUP ? (gi == 0 ? grp.wg_begin[1] : (gi == 1 ? grp.wg_begin[2] : grp.wg_begin[3])) - wg0
                            : (int)gridDim.y;
  const int wl0 = s * wl_per;
  const int wl1 = wl0 + wl_per < nwl ? wl0 + wl_per : nwl;
  const int wl1f = wl1 < nfull ? wl1 : nfull;           // end of the full wave-loads
  const int npw = (wl_per + kWaves - 1) / kWaves;       // items per wave and unit (padded)
  // whole units of this workgroup: ceil((nrb - rb0) / rb_step), quotient and remainder from the host;
  // with HALF the remainder counts half units instead
  const int upw = HALF ? upw_q : upw_q + (rb0 < upw_r ? 1 : 0);
  const int T_full = upw * npw;
  const bool has_half = HALF && rb0 < upw_r;
  const int half_rh = rb0 & 1;
  const int half_rb = upw_q * rb_step + (rb0 >> 1);
  const int T = T_full + (has_half ? npw : 0);
  const int w_first = wl0 + wave;
  const int nvj = w_first < wl1f ? (wl1f - w_first + kWaves - 1) / kWaves : 0;  // real items per unit
  const bool tail_wave = wl1 > nfull && ((nfull - wl0) % kWaves) == wave;
  float* out_s = dst + (size_t)s * (GROUP ? grp.part_stride : (size_t)m);

  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(packed), 0, (int)((size_t)nrb * rb_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(x), 0, k * 2, 0x00020000);

  // load cursor: unit l_i (row block l_rb), item l_j
  int l_j = 0, l_t = 0;
  uint32_t l_rboff = (uint32_t)((HALF && upw == 0) ? half_rb : rb0) * rb_bytes;
  const uint32_t rb_step_bytes = (uint32_t)rb_step * rb_bytes;
  LaneData<K> buf[DEPTH];
  u32x2 xbuf[XLDS ? 1 : DEPTH][4];
  auto issue = [&](int d) {
    const bool valid = l_j < nvj && l_t < T;
    const uint32_t wl = (uint32_t)(w_first + l_j * kWaves);
    const uint32_t woff = valid ? l_rboff + wl * WL_BYTES : 0u;
    const uint32_t xw = valid ? wl * 256u : 0u;
    // padding items: a lane offset past the end of the descriptor returns zeros without touching
    // memory (reading offset 0 instead cost the small shapes up to 2 us: thousands of waves
    // hammering the same few cache lines)
    buf[d] = load_lane_buf<K>(rs_w, valid ? loff : 0x7FFFFF00u, woff);
    if constexpr (!XLDS) load_x_buf(rs_x, valid ? xoff : 0x7FFFFF00u, xw, xbuf[d]);
    ++l_t;
    if (++l_j == npw) {
      l_j = 0;
      l_rboff = (HALF && l_t == T_full) ? (uint32_t)half_rb * rb_bytes : l_rboff + rb_step_bytes;
    }
  };
  // Prologue loads in the order they are needed: the table words and x first, then the first
  // FIRST wave-loads of the stream; the other DEPTH - FIRST follow once the table is built and the
  // workgroup is past its barrier.  A CU serves requests in order from a finite queue: with all
  // DEPTH wave-loads of all 16 waves requested up front (25 MB over the chip at K = 2) the last
  // waves stall on issuing theirs until most of that data has arrived, and reach the table they
  // have yet to write - and the barrier every wave waits at - thousands of cycles late.
  // (Measured: 2 before / rest after is 3-10 % faster than all before on every shape tried; 1, 3
  // and 4 before are in between.)
  static_assert(kLutEntries * 8 == 8 * kThreads, "table build assumes 8 16-byte items per thread");
  uint32_t tw[4];  // item it*1024 + tid belongs to entry it*128 + tid/8; entries e and e+512 share a word
  // the wave's eight words of a pass come through the scalar cache (uniform address), which
  // keeps them out of the vector-memory queue that the stream requests fill
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const uint32_t* tp = tlut + it * 128 + wave * 8;
    // one 32-byte scalar load (the table needs dword alignment only).  Loaded word by word, the
    // compiler may fold the first select below into a per-lane load of tp[lane >> 3], and the wait
    // for that vector load also waits for the stream loads requested before it.
    typedef uint32_t u32x8_dw __attribute__((ext_vector_type(8), aligned(4)));
    const u32x8_dw sw = *reinterpret_cast<const u32x8_dw*>(tp);
    uint32_t v = sw[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) v = ((lane >> 3) == j) ? sw[j] : v;
    tw[it] = v;
  }
  QTIP_STAMP(1)
  u32x4 xstage[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
  u32x4 xstage2[XHALF ? 2 : 1] = {};
  const int jh = XHALF ? (npw + 1) >> 1 : npw;  // items per wave served by the first staging
  // wave-loads of the first staging (all of the range unless XHALF)
  const int wlx = XHALF ? ((wl1 - wl0) < jh * kWaves ? (wl1 - wl0) : jh * kWaves) : (wl1 - wl0);
  float xraw[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  ChainRegs cr;
  if constexpr (XFORM == 2) {
    const _Float16* sr = reinterpret_cast<const _Float16*>(su);
    switch (k >> 10) {
      case 2: chain_load<2>(chain, sr, tid, lane, wave, cr); break;
      case 4: chain_load<4>(chain, sr, tid, lane, wave, cr); break;
      default: chain_load<8>(chain, sr, tid, lane, wave, cr); break;
    }
  } else if constexpr (XFORM == 1) {
    // the raw activations and the sign vector of the layer, k / 1024 consecutive elements per thread
    using namespace qtip_wht;
    float sv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const _Float16* xr = reinterpret_cast<const _Float16*>(x);
    const _Float16* sr = reinterpret_cast<const _Float16*>(su);
    switch (k >> 10) {
      case 2: ld_f16<2>(xr + tid * 2, xraw); ld_f16<2>(sr + tid * 2, sv); break;
      case 4: ld_f16<4>(xr + tid * 4, xraw); ld_f16<4>(sr + tid * 4, sv); break;
      default: ld_f16<8>(xr + tid * 8, xraw); ld_f16<8>(sr + tid * 8, sv); break;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) xraw[i] *= sv[i];  // entries past k / 1024 are never read
  } else if constexpr (XLDS) {
    // x of wave-loads [wl0, wl0 + wlx): 16 bytes per thread and pass, at most 2 passes (28 KiB)
    const int xbytes = wlx * 256;
    const int kbytes = k * 2;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int o = (ps * kThreads + tid) * 16;
      if (o < xbytes && wl0 * 256 + o < kbytes)
        xstage[ps] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint8_t*>(x) + (size_t)wl0 * 256 + o);
    }
    if constexpr (XHALF) {
      const int xbytes2 = (wl1 - wl0 - wlx) * 256;
      const int base2 = (wl0 + wlx) * 256;
#pragma unroll
      for (int ps = 0; ps < 2; ++ps) {
        const int o = (ps * kThreads + tid) * 16;
        if (o < xbytes2 && base2 + o < kbytes)
          xstage2[ps] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint8_t*>(x) + (size_t)base2 + o);
      }
    }
  }
#pragma unroll
  for (int d = 0; d < FIRST; ++d) issue(d);

  if constexpr (XFORM == 2) {
    float* xbuf = reinterpret_cast<float*>(smem);
    float* wsum = xbuf + k + (k >> 6);
    _Float16* xs = reinterpret_cast<_Float16*>(xs_lds);
    const bool write_x = blockIdx.x == 0 && blockIdx.y == 0;
    switch (k >> 10) {
      case 2: chain_compute<2>(cr, chain, xscale, xbuf, wsum, xs, tid, lane, wave, write_x, QTIP_STAMP_PTR); break;
      case 4: chain_compute<4>(cr, chain, xscale, xbuf, wsum, xs, tid, lane, wave, write_x, QTIP_STAMP_PTR); break;
      default: chain_compute<8>(cr, chain, xscale, xbuf, wsum, xs, tid, lane, wave, write_x, QTIP_STAMP_PTR); break;
    }
  } else if constexpr (XFORM == 1) {
    QTIP_STAMP(6)
    float* xchg = reinterpret_cast<float*>(smem);
    _Float16* xs = reinterpret_cast<_Float16*>(xs_lds);
    switch (k >> 10) {
      case 2: xform_prologue<2>(xraw, xscale, xchg, xs, tid, lane, wave); break;
      case 4: xform_prologue<4>(xraw, xscale, xchg, xs, tid, lane, wave); break;
      default: xform_prologue<8>(xraw, xscale, xchg, xs, tid, lane, wave); break;
    }
    QTIP_STAMP(10)
  }
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const uint32_t w = tw[it & 3] ^ ((uint32_t)(it >> 2) << 15);
    const u32x4 v = {w, w, w, w};
    reinterpret_cast<u32x4*>(lut)[it * kThreads + tid] = v;
  }
  if constexpr (XLDS && !XFORM) {
    const int xbytes = wlx * 256;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int o = (ps * kThreads + tid) * 16;
      if (o < xbytes) *reinterpret_cast<u32x4*>(xs_lds + o) = xstage[ps];
    }
  }
  QTIP_STAMP(2)
  __syncthreads();
  QTIP_STAMP(3)
#pragma unroll
  for (int d = FIRST; d < DEPTH; ++d) issue(d);
  QTIP_STAMP_FIRST_LOAD()

  // wave-load w_first (the transformed vector is stored whole, a staged one from wl0 on)
  const uint32_t xs_lane = lds_address(xs_lds) + xoff + (uint32_t)(XFORM ? w_first : wave) * 256u;

  float4_t acc[4];  // [2*mh + rh]: rows 16*mh + 8*rh + a/2 of the unit's 32-row block
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
  int parity = 0, c_j = 0, c_rb = (HALF && upw == 0) ? half_rb : rb0;
  int c_jbase = 0;  // first item of the staging that is in LDS
  int prio_phase = wave >> 2;  // waves w, w + 4, w + 8, w + 12 share a SIMD
  // items [t0, t1) of the workgroup's item sequence, decoding all states (RH = -1) or one row half.
  // Whole and half units run in loops of their own: with both forms behind a branch in one loop
  // body the compiler loses track of the loads in flight and waits for all of them at every item.
  auto run = [&](auto rh_tag, const int t0, const int t1) {
  constexpr int RH = decltype(rh_tag)::value;
  auto accumulate = [&](const LaneData<K>& ld, const u32x2 xv[4]) {
    matvec_accumulate<K, RH>(ld, xv, slot4, acc);
  };
  for (int t = t0; t < t1; t += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      // The hardware serves the waves of a SIMD oldest first, so the oldest finishes its share of a
      // unit long before the youngest and the SIMD ends every unit on too few waves to hide
      // latencies: the top issue priority rotates through the four waves, item by item.
      switch ((prio_phase++) & 3) {
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
      }
      if (t + d < t1) {
        if (c_j < nvj) {
          if constexpr (XLDS) {
            typedef __attribute__((address_space(3))) const u32x2 lds_u32x2_t;
            u32x2 xv[4];
            const uint32_t xa = xs_lane + (uint32_t)(c_j - c_jbase) * (kWaves * 256u);
#pragma unroll
            for (int q = 0; q < 4; ++q) xv[q] = *(lds_u32x2_t*)(uintptr_t)(xa + 16u * q);
            accumulate(buf[d], xv);
          } else {
            accumulate(buf[d], xbuf[d]);
          }
        }
      }
      // the stage's registers are refilled only after their last use, so the
      // refill reuses them in place (no copies, no wait on the new load)
      issue(d);
      if (t + d < t1) ++c_j;
      if constexpr (XHALF) {
        // middle of the (only) unit: every wave has read its last x of the first half
        if (t + d < t1 && c_j == jh && jh < npw) {
          __syncthreads();
          const int xbytes2 = (wl1 - wl0 - wlx) * 256;
#pragma unroll
          for (int ps = 0; ps < 2; ++ps) {
            const int o = (ps * kThreads + tid) * 16;
            if (o < xbytes2) *reinterpret_cast<u32x4*>(xs_lds + o) = xstage2[ps];
          }
          __syncthreads();
          c_jbase = jh;
        }
      }
      if (t + d < t1 && c_j == npw) {
        // ---- end of a unit: ragged tail, reductions, store
        // k/32 not a multiple of 4: one wave takes the partial wave-load.  Every lane takes part
        // in an MFMA, so the lanes of the missing tile blocks (g >= nkb % 4) load x and the stream
        // with a lane offset that is out of range by itself: both come back as zeros without a
        // memory access, whatever the range check makes of the scalar offset.
        if (tail_wave) {
          const bool in_row = g < nkb - 4 * nfull;
          u32x2 xt[4];
          load_x_buf(rs_x, in_row ? xoff : 0x7FFFFF00u, (uint32_t)nfull * 256u, xt);
          const LaneData<K> tail = load_lane_buf<K>(rs_w, in_row ? loff : 0x7FFFFF00u,
                                                    (uint32_t)c_rb * rb_bytes + (uint32_t)nfull * WL_BYTES);
          accumulate(tail, xt);
        }
        float* pp = part + parity * (kWaves * 32);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // element a % 2 holds the lane's sum over the four blocks: an even lane adds its element 0
          // and element 1 of its odd neighbour (the other column half).  Written without a
          // per-lane choice of the element on purpose: with `v = odd ? e1 : e0; v += exchange(v)`
          // the compiler, knowing that only even lanes store, fed e0 into the exchange for every lane.
          const float v = acc[i][0] + dpp_xor1(acc[i][1]);
          acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
          if (g == 0 && (a & 1) == 0) pp[wave * 32 + (i >> 1) * 16 + (i & 1) * 8 + (a >> 1)] = v;
        }
        __syncthreads();
        // (a half unit owns the rows 16*mh + 8*rh + 0..7 of its rh only)
        if (tid < 32 && (RH < 0 || ((tid >> 3) & 1) == RH)) {
          float sum = 0.f;
#pragma unroll
          for (int w = 0; w < kWaves; ++w) sum += pp[w * 32 + tid];
          out_s[c_rb * 32 + tid] = sum;
        }
        parity ^= 1;  // the other buffer is free: its readers passed the barrier above
        c_j = 0;
        c_rb = (HALF && t + d + 1 == T_full) ? half_rb : c_rb + rb_step;
      }
    }
  }
  };
  run(std::integral_constant<int, -1>{}, 0, T_full);
  if constexpr (HALF) {
    if (has_half) {
      if (half_rh) run(std::integral_constant<int, 1>{}, T_full, T);
      else run(std::integral_constant<int, 0>{}, T_full, T);
    }
  }
#ifdef QTIP_STAMPS
  {
    QTIP_STAMP(4)
    const int wg = (int)blockIdx.x + (int)gridDim.x * (int)blockIdx.y;
    const int slot = ((m ^ k) >> 10) & (kStampSlots - 1);
    if (wg < kStampWgs && lane == 0) {
      if (wave == 0) {
#pragma unroll
        for (int i = 0; i < kStampN; ++i)
          if (i != 5) g_stamps[slot][wg][i] = stamp_v[i];
      } else if (wave == kWaves - 1) {
        g_stamps[slot][wg][5] = stamp_v[0];
      }
    }
  }
#endif
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
// batched decompress + fp16 MFMA GEMM
// ---------------------------------------------------------------------------
// out[b][row] = sum_col x[b][col] * W[row][col] with v_mfma_f32_16x16x32_f16:
// M = 16 batch rows, N = the 16 lanes of a DPP row, K = 32 columns.
//
// The decode leaves, for every (tile row half mh, row half rh, kh), in lane
// (g, a) the eight weights of matrix row 16*mh + 8*rh + a/2 at columns
// 32*g' + 16*kh + 4*(a%2) + {0..3, 8..11} (g' = the lane group's tile block):
// exactly the shape of an MFMA B operand (N index = a, K group = g), except
// that even and odd lanes hold different columns (the 4*(a%2) term).  Each
// product is therefore issued twice, once with the activations of columns
// +0..3 / +8..11 and once with +4..7 / +12..15, into two accumulators; in the
// first the even lanes' results are meaningful, in the second the odd lanes',
// and the other half is simply never read.  That spends half of the matrix
// core's work, which is free here (the kernel is bound by the decode), and
// needs no data movement between decode and MFMA: the table lookups land in
// the operand registers.
//
// Activations are shared through LDS: a workgroup (8 waves) works on 4 consecutive 32-row blocks
// at the same columns - wave w takes row block w % 4 and, of each pair of wave-loads, number
// w / 4 - so one 16*NB x 256 activation tile per stage serves all eight waves (read from L2 once
// per 128 matrix rows instead of once per 32; the per-wave reads measured 35-50 % of the run
// time before).  Tiles are double-buffered: loaded to registers two stages ahead, written to
// LDS one stage ahead, one barrier per stage.  Rows of the tile are 512 bytes with the 16-byte
// chunk index xor-ed with the row, which keeps both the 16-byte fills and the A-operand reads
// (16 lanes = 16 rows at the same chunk) free of bank conflicts.
// Work unit = (group of 4 row blocks, k split s); a workgroup keeps one s, so its sequence of
// activation tiles is the same for every unit and the pipeline runs across unit boundaries.
// S > 1 (few row blocks): fp32 partial results go to parts[s][batch][m] and are summed afterwards.
constexpr int kGemmRB = 4;  // row blocks per group
// Two shapes of workgroup: 8 waves (2 k slices, up to 256 VGPRs: two batch tiles) and 16 waves
// (4 k slices, 128 VGPRs: one batch tile, twice the waves to hide the latencies of a stage).
constexpr size_t kGemmTileBytes = 16 * 1024;  // 16*NB batch rows x 256*KS columns fp16, NB*KS == 4
constexpr size_t kGemmLds = kLut128Bytes + 2 * kGemmTileBytes;

template <int K, int NB, int DEPTH, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 1) void gemm_kernel(
    float* __restrict__ dst, const uint8_t* __restrict__ packed, const uint16_t* __restrict__ x,
    const uint32_t* __restrict__ tlut, int m, int k, int batch, int round_f16, int wl_per, int upw_q,
    int upw_r) {
  constexpr int THREADS = WAVES * 64;
  constexpr int KS = WAVES / kGemmRB;          // wave-loads per stage
  constexpr int ROWB = KS * 256;               // bytes per tile row
  constexpr int CPR = ROWB / 16;               // 16-byte chunks per tile row
  constexpr uint32_t TILE = 16 * NB * ROWB;
  static_assert(2 * TILE <= 2 * kGemmTileBytes, "tiles do not fit");
  static_assert(16 * NB * CPR == NB * THREADS, "NB chunks per thread and tile");
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  uint8_t* tiles = smem + kLut128Bytes;  // [2][16*NB rows][ROWB bytes]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rbi = wave & (kGemmRB - 1), ks = wave >> 2;
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = lds_address(lut) + ((uint32_t)(lane & 31) << 2);
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;  // wave-loads per row block; a partial last one meets zero activations
  const int nrb = m >> 5;
  const int ngroups = (nrb + kGemmRB - 1) / kGemmRB;
  const uint32_t rb_bytes = (uint32_t)nkb * 128 * K;
  constexpr uint32_t WL_BYTES = 512 * K;
  const uint32_t loff = (uint32_t)lane * 8 * K;
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(packed), 0, (int)((size_t)nrb * rb_bytes), 0x00020000);

  // grid = (S, workgroups per k range); unit counts as quotient and remainder from the host:
  // no integer division on the way to the first loads
  const int s = blockIdx.x;
  const int g0 = blockIdx.y, gstep = gridDim.y;
  const int wl0 = s * wl_per;                                   // wl_per is a multiple of KS
  const int wl1 = wl0 + wl_per < nwl ? wl0 + wl_per : nwl;
  const int nst = wl1 > wl0 ? (wl1 - wl0 + KS - 1) / KS : 0;    // stages (KS wave-loads each) per unit
  const int upw = upw_q + (g0 < upw_r ? 1 : 0);  // units of this workgroup: ceil((ngroups - g0) / gstep)
  const int T = upw * nst;
  float* out_s = dst + (size_t)s * batch * m;

  // ---- weight stream of this wave: item q = (unit q / nst, stage q % nst), DEPTH in flight
  int l_t = 0, l_q = 0, l_grp = g0;
  LaneData<K> buf[DEPTH];
  auto issue = [&](int d) {
    const int rb = l_grp * kGemmRB + rbi;
    const int wl = wl0 + KS * l_t + ks;
    const bool valid = l_q < T && rb < nrb && wl < wl1;
    // padding items, and the lanes past the row's end in a partial last wave-load (k / 32 not a
    // multiple of 4): a lane offset that is out of range by itself, zeros without a memory access
    const bool lane_ok = valid && 4 * wl + g < nkb;
    buf[d] = load_lane_buf<K>(rs_w, lane_ok ? loff : 0x7FFFFF00u,
                              valid ? (uint32_t)rb * rb_bytes + (uint32_t)wl * WL_BYTES : 0u);
    ++l_q;
    if (++l_t == nst) {
      l_t = 0;
      l_grp += gstep;
    }
  };
  // table words first (their loads return before the stream's), one stage of the stream before the
  // table is built, the others once the workgroup is past its first barrier
  constexpr int NTW = kLutEntries * 4 / THREADS;  // distinct table words per thread
  uint32_t tw[NTW];
#pragma unroll
  for (int j = 0; j < NTW; ++j) {
    // the wave's eight words of a pass through the scalar cache (uniform address), lane l keeps word l / 8
    const uint32_t* tp = tlut + j * (THREADS / 8) + wave * 8;
    uint32_t v = tp[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) v = ((lane >> 3) == e) ? tp[e] : v;
    tw[j] = v;
  }
  issue(0);

  // ---- activation tiles: thread fills NB 16-byte chunks per tile

  static_assert(DEPTH % 2 == 0, "stage parity must be static inside the unrolled loop");
  u32x4 xg[2][NB];  // tiles on their way: [parity of the stage][chunk]
  auto load_tile = [&](int slot, int t) {  // stage t of a unit -> registers
    const int col0 = 128 * (wl0 + KS * t);
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = i * THREADS + tid;
      const int b = idx / CPR, c = idx % CPR;
      const int col = col0 + 8 * c;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (b < batch && col < k) v = *reinterpret_cast<const u32x4*>(x + (size_t)b * k + col);
      xg[slot][i] = v;
    }
  };
  auto store_tile = [&](int slot, int bufi) {  // registers -> LDS buffer
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = i * THREADS + tid;
      const int b = idx / CPR, c = idx % CPR;
      *reinterpret_cast<u32x4*>(tiles + bufi * TILE + b * ROWB + ((c ^ (b & 7)) << 4)) = xg[slot][i];
    }
  };
  load_tile(0, 0);
  load_tile(1, nst > 1 ? 1 : 0);
#pragma unroll
  for (int it = 0; it < kLutEntries * 8 / THREADS; ++it) {
    // item it*THREADS + tid belongs to entry it*THREADS/8 + tid/8; entries e and e+512 share a word
    const uint32_t w = tw[it % NTW] ^ ((uint32_t)(it / NTW) << 15);
    const u32x4 v = {w, w, w, w};
    reinterpret_cast<u32x4*>(lut)[it * THREADS + tid] = v;
  }
  store_tile(0, 0);
  __syncthreads();
#pragma unroll
  for (int d = 1; d < DEPTH; ++d) issue(d);

  float4_t acc[2][2][2][NB];  // [mh][rh][column half][batch tile]
#pragma unroll
  for (int i = 0; i < 8 * NB; ++i) (&acc[0][0][0][0])[i] = float4_t{0.f, 0.f, 0.f, 0.f};

  // LDS byte offset (inside a tile) of this lane's A-operand chunks: row 16*nb + a, chunk 16*ks + 4*g + 2*kh + h
  uint32_t arow[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) arow[nb] = (uint32_t)(16 * nb + a) * ROWB;
  const uint32_t a7 = (uint32_t)(a & 7);
  const uint32_t tiles_addr = lds_address(tiles);

  int c_t = 0, c_grp = g0;
  for (int q = 0; q < T; q += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const bool live = q + d < T;  // uniform over the workgroup
      if (live) {
        // tile of stage q+d+2 to registers (slot = parity of that stage = parity of q+d)
        {
          int t2 = c_t + 2;
          if (t2 >= nst) t2 -= nst;
          if (t2 >= nst) t2 -= nst;  // nst == 1
          load_tile((q + d) & 1, t2);
        }
        const int rb = c_grp * kGemmRB + rbi;
        const int wl = wl0 + KS * c_t + ks;
        if (rb < nrb && wl < wl1) {
          typedef __attribute__((address_space(3))) const u32x4 lds_u32x4_t;
          const uint32_t tb = tiles_addr + (uint32_t)((q + d) & 1) * TILE;
          uint32_t P[16], W[32];
          packed_states<K>(buf[d], P);
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const uint32_t hq = pk_hash(P[i]) & 0xFFC0FFC0u;
            W[2 * i] = lds_word_abs(lut128_addr_lo(hq, slot4));
            W[2 * i + 1] = lds_word_abs(lut128_addr_hi(hq, slot4));
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int kh = 0; kh < 2; ++kh) {
            u32x4 xa[NB][2];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
              for (int h = 0; h < 2; ++h) {
                const uint32_t c = (uint32_t)(16 * ks + 4 * g + 2 * kh + h) ^ a7;
                xa[nb][h] = *(lds_u32x4_t*)(uintptr_t)(tb + arow[nb] + (c << 4));
              }
#pragma unroll
            for (int mh = 0; mh < 2; ++mh)
#pragma unroll
              for (int rh = 0; rh < 2; ++rh) {
                const int tt = 2 * kh + mh;
                const u32x4 wv = {W[w_index<K>(0, tt, rh)], W[w_index<K>(1, tt, rh)],
                                  W[w_index<K>(0, tt, 2 + rh)], W[w_index<K>(1, tt, 2 + rh)]};
                const half8_t bop = __builtin_bit_cast(half8_t, wv);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                  for (int ch = 0; ch < 2; ++ch) {
                    // columns +4*ch+{0..3} and +8+4*ch+{0..3} of the 16 loaded ones
                    const u32x4 xv = {xa[nb][0][2 * ch], xa[nb][0][2 * ch + 1], xa[nb][1][2 * ch],
                                      xa[nb][1][2 * ch + 1]};
                    acc[mh][rh][ch][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8_t, xv), bop, acc[mh][rh][ch][nb], 0, 0, 0);
                  }
              }
          }
        }
      }
      issue(d);
      if (live) {
        // tile of the next stage (in registers since the previous stage) into the other buffer
        store_tile((q + d + 1) & 1, (q + d + 1) & 1);
        __syncthreads();
        if (++c_t == nst) {
          // ---- end of a unit: the k slices of a row block meet in the buffer this stage used
          // (the next tile sits in the other one): slices 1 .. KS-1 hand their sums over in turn,
          // the wave of slice 0 adds them in that order, rounds and stores
          float* xch = reinterpret_cast<float*>(tiles + ((q + d) & 1) * TILE) + rbi * (16 * NB * 32);
          float vals[2][2][NB][4];
#pragma unroll
          for (int mh = 0; mh < 2; ++mh)
#pragma unroll
            for (int rh = 0; rh < 2; ++rh)
#pragma unroll
              for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                  // even lanes: own sum of the even columns + the odd neighbour's sum of the odd columns
                  // (no per-lane choice before the exchange, see matvec_kernel)
                  vals[mh][rh][nb][i] = acc[mh][rh][0][nb][i] + dpp_xor1(acc[mh][rh][1][nb][i]);
                  acc[mh][rh][0][nb][i] = 0.f;
                  acc[mh][rh][1][nb][i] = 0.f;
                }
          const int e0 = ((a >> 1) + 8 * g) * (16 * NB);  // even lanes: 32 slots of 16*NB floats
          for (int turn = 1; turn < KS; ++turn) {
            if (ks == turn && (a & 1) == 0) {
#pragma unroll
              for (int mh = 0; mh < 2; ++mh)
#pragma unroll
                for (int rh = 0; rh < 2; ++rh)
#pragma unroll
                  for (int nb = 0; nb < NB; ++nb)
                    *reinterpret_cast<float4_t*>(xch + e0 + ((mh * 2 + rh) * NB + nb) * 4) =
                        float4_t{vals[mh][rh][nb][0], vals[mh][rh][nb][1], vals[mh][rh][nb][2], vals[mh][rh][nb][3]};
            }
            __syncthreads();
            if (ks == 0 && (a & 1) == 0) {
#pragma unroll
              for (int mh = 0; mh < 2; ++mh)
#pragma unroll
                for (int rh = 0; rh < 2; ++rh)
#pragma unroll
                  for (int nb = 0; nb < NB; ++nb) {
                    const float4_t o = *reinterpret_cast<const float4_t*>(xch + e0 + ((mh * 2 + rh) * NB + nb) * 4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) vals[mh][rh][nb][i] += o[i];
                  }
            }
            __syncthreads();  // the next slice may overwrite; after the last turn the buffer becomes a tile again
          }
          const int rb = c_grp * kGemmRB + rbi;
          if (ks == 0 && (a & 1) == 0 && rb < nrb) {
#pragma unroll
            for (int mh = 0; mh < 2; ++mh)
#pragma unroll
              for (int rh = 0; rh < 2; ++rh)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                  for (int i = 0; i < 4; ++i) {
                    float sum = vals[mh][rh][nb][i];
                    if (round_f16) sum = (float)(_Float16)sum;
                    // lane (g, a even): batch row 16*nb + 4*g + i, matrix row 16*mh + 8*rh + a/2
                    const int bb = 16 * nb + 4 * g + i;
                    if (bb < batch) out_s[(size_t)bb * m + rb * 32 + 16 * mh + 8 * rh + (a >> 1)] = sum;
                  }
          }
          c_t = 0;
          c_grp += gstep;
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// 4-bit batched decompress + GEMM on a row-split lane map: no product is computed twice
// ---------------------------------------------------------------------------
// In gemm_kernel the two lanes that share a matrix row hold different column halves of it, which
// costs every product twice (and 64 accumulator registers for 32 batch rows, hence 8 waves).
// Here the two lanes of a pair load the SAME 64 bytes - the four reference lanes of one row of a
// 2x2 tile block, i.e. all 16 columns of that row in each of the four tiles - and split the
// STATES: a 32-bit chunk holds four states, the even lane decodes states 0 and 2 (rows r), the
// odd lane states 1 and 3 (rows r + 8).  A byte permutation with a per-lane selector puts the
// lane's two states of a chunk into one register, so the decode costs what it costs in
// gemm_kernel (32 lookups per lane and wave-load).  The 16 lanes of a DPP row now hold the same
// 8 columns of 16 different rows: a v_mfma_f32_16x16x32_f16 B operand whose every output is
// wanted.  Per wave-load and 16 batch rows: 8 products instead of 16, 8 accumulator registers
// instead of 32, so 32 batch rows run on the 16-wave workgroup (4 waves per SIMD).
// Lane (g, a): tile block g of the wave-load, row r = a / 2 (+ 8 for odd a) of either tile row
// half; registers D[cp][t]: reference lane 4 r + cp (columns 2 cp, 2 cp + 1 of an 8-column
// group), tile t = 2 kh + mh.  The successor chunk of cp = 3 sits two lanes on (row r + 1, the
// ring of 32 reference lanes closing inside the 16-lane row).
// The two lanes of a pair read the same bytes and the four 16-byte loads of a lane walk the same
// cache lines, so the loads are plain (cached) ones: with the non-temporal hint of the other
// kernels every load instruction fetched its lines from L2 again (43 us instead of 29 us at batch
// 8).  HBM traffic is unchanged.
// One activation tile (16 NB batch rows x 1024 columns) in LDS, single-buffered: the next tile
// waits in registers while the current one is used, two barriers per stage.
constexpr int kGemm4Waves = 16, kGemm4KS = 4;
constexpr size_t kGemm4TileBytes = 32 * 1024;
constexpr size_t kGemm4Lds = kLut128Bytes + kGemm4TileBytes;

template <int NB>
__global__ __launch_bounds__(kThreads, 1) void gemm4_kernel(
    float* __restrict__ dst, const uint8_t* __restrict__ packed, const uint16_t* __restrict__ x,
    const uint32_t* __restrict__ tlut, int m, int k, int batch, int round_f16, int wl_per, int upw_q,
    int upw_r) {
  constexpr int K = 4, DEPTH = 2, KS = kGemm4KS;
  constexpr int ROWB = KS * 256;  // bytes per tile row
  constexpr int CPR = ROWB / 16;  // 16-byte chunks per tile row
  constexpr uint32_t TILE = 16 * NB * ROWB;
  constexpr bool DB = 2 * TILE <= kGemm4TileBytes;  // room for two tiles: one barrier per stage instead of two
  static_assert(TILE <= kGemm4TileBytes, "tile does not fit");
  static_assert(16 * NB * CPR == NB * kThreads, "NB chunks per thread and tile");
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  uint8_t* tile = smem + kLut128Bytes;  // [1 or 2][16*NB rows][ROWB bytes]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rbi = wave & (kGemmRB - 1), ks = wave >> 2;
  const int a = lane & 15, g = lane >> 4;
  const uint32_t slot4 = lds_address(lut) + ((uint32_t)(lane & 31) << 2);
  const int nkb = k >> 5;
  const int nwl = (nkb + 3) >> 2;
  const int nrb = m >> 5;
  const int ngroups = (nrb + kGemmRB - 1) / kGemmRB;
  const uint32_t rb_bytes = (uint32_t)nkb * 128 * K;
  constexpr uint32_t WL_BYTES = 512 * K;
  const uint32_t loff = (uint32_t)g * (128 * K) + (uint32_t)(a >> 1) * (16 * K);  // the row's four reference lanes
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(packed), 0, (int)((size_t)nrb * rb_bytes), 0x00020000);
  // states 0 | 2 of a chunk for even lanes (the chunk as it is), 1 | 3 for odd lanes (chunk bytes
  // 2 1 | chunk byte 0, successor byte 3)
  const uint32_t sel = (a & 1) ? 0x06050403u : 0x07060504u;

  const int s = blockIdx.x;
  const int g0 = blockIdx.y, gstep = gridDim.y;
  const int wl0 = s * wl_per;  // wl_per is a multiple of KS
  const int wl1 = wl0 + wl_per < nwl ? wl0 + wl_per : nwl;
  const int nst = wl1 > wl0 ? (wl1 - wl0 + KS - 1) / KS : 0;  // stages per unit
  const int upw = upw_q + (g0 < upw_r ? 1 : 0);
  const int T = upw * nst;
  float* out_s = dst + (size_t)s * batch * m;

  struct Raw {
    uint32_t d[4][4];  // [cp][t]
  };
  int l_t = 0, l_q = 0, l_grp = g0;
  Raw buf[DEPTH];
  auto issue = [&](int d) {
    const int rb = l_grp * kGemmRB + rbi;
    const int wl = wl0 + KS * l_t + ks;
    const bool valid = l_q < T && rb < nrb && wl < wl1;
    // padding items, and the lanes past the row's end in a partial last wave-load: a lane offset
    // that is out of range by itself, zeros without a memory access
    const uint32_t vo = (valid && 4 * wl + g < nkb) ? loff : 0x7FFFFF00u;
    const uint32_t so = valid ? (uint32_t)rb * rb_bytes + (uint32_t)wl * WL_BYTES : 0u;
#pragma unroll
    for (int cp = 0; cp < 4; ++cp) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs_w, vo + 16 * cp, so, 0);
#pragma unroll
      for (int t = 0; t < 4; ++t) buf[d].d[cp][t] = v[t];
    }
    ++l_q;
    if (++l_t == nst) {
      l_t = 0;
      l_grp += gstep;
    }
  };
  // table words through the scalar cache first, one stage of the stream before the table is built
  uint32_t tw[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t* tp = tlut + j * 128 + wave * 8;
    uint32_t v = tp[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) v = ((lane >> 3) == e) ? tp[e] : v;
    tw[j] = v;
  }
  issue(0);

  static_assert(DEPTH % 2 == 0, "stage parity must be static inside the unrolled loop");
  u32x4 xg[2][NB];  // tiles on their way: [parity of the stage][chunk], requested two stages ahead
  auto load_tile = [&](int slot, int t) {  // stage t of a unit -> registers
    const int col0 = 128 * (wl0 + KS * t);
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = i * kThreads + tid;
      const int b = idx / CPR, c = idx % CPR;
      const int col = col0 + 8 * c;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (b < batch && col < k) v = *reinterpret_cast<const u32x4*>(x + (size_t)b * k + col);
      xg[slot][i] = v;
    }
  };
  // registers -> LDS buffer (the buffer of the stage's parity when there are two), chunk index
  // xor-ed with the row: conflict-free both ways
  auto store_tile = [&](int slot) {
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const int idx = i * kThreads + tid;
      const int b = idx / CPR, c = idx % CPR;
      *reinterpret_cast<u32x4*>(tile + (DB ? slot * TILE : 0u) + b * ROWB + ((c ^ (b & 7)) << 4)) = xg[slot][i];
    }
  };
  load_tile(0, 0);
  load_tile(1, nst > 1 ? 1 : 0);
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const uint32_t w = tw[it & 3] ^ ((uint32_t)(it >> 2) << 15);
    const u32x4 v = {w, w, w, w};
    reinterpret_cast<u32x4*>(lut)[it * kThreads + tid] = v;
  }
  store_tile(0);
  __syncthreads();
  issue(1);

  float4_t acc[2][NB];  // [mh][batch tile]
#pragma unroll
  for (int i = 0; i < 2 * NB; ++i) (&acc[0][0])[i] = float4_t{0.f, 0.f, 0.f, 0.f};
  uint32_t arow[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) arow[nb] = (uint32_t)(16 * nb + a) * ROWB;
  const uint32_t a7 = (uint32_t)(a & 7);
  const uint32_t tile_addr = lds_address(tile);
  typedef __attribute__((address_space(3))) const u32x4 lds_u32x4_t;

  int c_t = 0, c_grp = g0;
  for (int q = 0; q < T; q += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const bool live = q + d < T;  // uniform over the workgroup
      if (live) {
        const int rb = c_grp * kGemmRB + rbi;
        const int wl = wl0 + KS * c_t + ks;
        if (rb < nrb && wl < wl1) {
          const Raw& R = buf[d];
          const uint32_t tb = tile_addr + (DB ? (uint32_t)((q + d) & 1) * TILE : 0u);
          uint32_t W[4][4][2];  // [cp][t][jh]
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            // successor of reference lane 4 r + 3: reference lane 4 (r + 1), two lanes on in the row
            const uint32_t nx = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)R.d[0][t], 0x12E /* row_ror:14 */,
                                                                      0xF, 0xF, false);
#pragma unroll
            for (int cp = 0; cp < 4; ++cp) {
              const uint32_t c = R.d[cp][t];
              const uint32_t cn = cp < 3 ? R.d[cp + 1][t] : nx;
              const uint32_t P = perm(c, cn, sel);  // high half: state 0 or 1, low half: state 2 or 3
              const uint32_t hq = pk_hash(P) & 0xFFC0FFC0u;
              W[cp][t][0] = lds_word_abs(lut128_addr_hi(hq, slot4));
              W[cp][t][1] = lds_word_abs(lut128_addr_lo(hq, slot4));
            }
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int kh = 0; kh < 2; ++kh)
#pragma unroll
            for (int jh = 0; jh < 2; ++jh) {
              u32x4 xa[NB];
              const uint32_t c = (uint32_t)(16 * ks + 4 * g + 2 * kh + jh) ^ a7;
#pragma unroll
              for (int nb = 0; nb < NB; ++nb)
                xa[nb] = *(lds_u32x4_t*)(uintptr_t)(tb + arow[nb] + (c << 4));
#pragma unroll
              for (int mh = 0; mh < 2; ++mh) {
                const int t = 2 * kh + mh;
                const u32x4 wv = {W[0][t][jh], W[1][t][jh], W[2][t][jh], W[3][t][jh]};
                const half8_t bop = __builtin_bit_cast(half8_t, wv);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                  acc[mh][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa[nb]), bop,
                                                                       acc[mh][nb], 0, 0, 0);
              }
            }
        }
      }
      issue(d);
      if (live) {
        if constexpr (DB) {
          // the next tile (in registers since the previous stage) into the other buffer, the one
          // after it on its way (slot = parity of that stage = parity of this one)
          store_tile((q + d + 1) & 1);
          int t2 = c_t + 2;
          if (t2 >= nst) t2 -= nst;
          if (t2 >= nst) t2 -= nst;  // nst == 1
          load_tile((q + d) & 1, t2);
        }
        __syncthreads();  // every wave has read this stage's tile (and, with two buffers, written the next)
        const int rb = c_grp * kGemmRB + rbi;
        if (++c_t == nst) {
          // ---- end of a unit: the k slices of a row block meet in the tile buffer (free between the
          // two barriers of a stage): slices 1 .. KS-1 hand their sums over in turn, the wave of
          // slice 0 adds them in that order, rounds and stores
          float* xch = reinterpret_cast<float*>(tile + (DB ? (uint32_t)((q + d) & 1) * TILE : 0u)) + rbi * (64 * 8 * NB);
          float4_t vals[2][NB];
#pragma unroll
          for (int mh = 0; mh < 2; ++mh)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
              vals[mh][nb] = acc[mh][nb];
              acc[mh][nb] = float4_t{0.f, 0.f, 0.f, 0.f};
            }
          for (int turn = 1; turn < KS; ++turn) {
            if (ks == turn) {
#pragma unroll
              for (int mh = 0; mh < 2; ++mh)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                  *reinterpret_cast<float4_t*>(xch + ((mh * NB + nb) * 64 + lane) * 4) = vals[mh][nb];
            }
            __syncthreads();
            if (ks == 0) {
#pragma unroll
              for (int mh = 0; mh < 2; ++mh)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                  const float4_t o = *reinterpret_cast<const float4_t*>(xch + ((mh * NB + nb) * 64 + lane) * 4);
                  vals[mh][nb] += o;
                }
            }
            __syncthreads();
          }
          if (ks == 0 && rb < nrb) {
#pragma unroll
            for (int mh = 0; mh < 2; ++mh)
#pragma unroll
              for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                  float sum = vals[mh][nb][i];
                  if (round_f16) sum = (float)(_Float16)sum;
                  // lane (g, a): batch row 16*nb + 4*g + i, matrix row 16*mh + 8*(a%2) + a/2
                  const int bb = 16 * nb + 4 * g + i;
                  if (bb < batch) out_s[(size_t)bb * m + rb * 32 + 16 * mh + 8 * (a & 1) + (a >> 1)] = sum;
                }
          }
          c_t = 0;
          c_grp += gstep;
        }
        if constexpr (!DB) {
          // one buffer: the next tile (in registers since the previous stage) goes in now, the one
          // after it on its way (slot = parity of that stage = parity of this one)
          store_tile((q + d + 1) & 1);
          int t2 = c_t + 1;
          if (t2 >= nst) t2 -= nst;
          load_tile((q + d) & 1, t2);
          __syncthreads();  // the next tile is complete
        }
      }
    }
  }
}

// out[i] = parts[0][i] + ... (+ rounding through fp16) for the split-k GEMM
__global__ __launch_bounds__(256) void sum_parts_round_kernel(float* __restrict__ out,
                                                              const float* __restrict__ parts, long n,
                                                              int S, int round_f16) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float sum = parts[i];
  for (int s = 1; s < S; ++s) sum += parts[(size_t)s * n + i];
  out[i] = round_f16 ? (float)(_Float16)sum : sum;
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
// Device memory the allocation-free entry point keeps its split-k partial sums in: one copy per
// GPU the library runs on, held until the process ends.  In host code this name is only a handle
// for hipGetSymbolAddress (never a device address): launches take DeviceState::scratch_ptr.
constexpr size_t kScratchFloats = 64 * 1024;  // 256 KiB
static __device__ __align__(256) float scratch[kScratchFloats];


template <typename F>
hipError_t allow_lds(F* fn, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(fn),
                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

hipError_t allow_lds_all() {
  hipError_t e;
#define QTIP_ALLOW(fn, bytes) \
  if ((e = allow_lds(fn, bytes)) != hipSuccess) return e;
  QTIP_ALLOW((decode_kernel<2>), kDecodeLds)
  QTIP_ALLOW((decode_kernel<3>), kDecodeLds)
  QTIP_ALLOW((decode_kernel<4>), kDecodeLds)
  QTIP_ALLOW((matvec_kernel<2, 2, false>), kMatvecLds)
  QTIP_ALLOW((matvec_kernel<3, 2, false>), kMatvecLds)
  QTIP_ALLOW((matvec_kernel<4, 2, false>), kMatvecLds)
  QTIP_ALLOW((matvec_kernel<2, 2, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 0, false, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 0, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true, 0, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true, 0, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 2, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true, 2, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true, 2, false, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 0, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true, 0, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true, 0, true>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 1>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true, 1>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true, 1>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<2, 2, true, 2>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<3, 2, true, 2>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((matvec_kernel<4, 2, true, 2>), kMatvecLds + kMatvecXBytes)
  QTIP_ALLOW((gemm_kernel<2, 1, 4, 16>), kGemmLds)
  QTIP_ALLOW((gemm_kernel<2, 2, 4, 8>), kGemmLds)
  QTIP_ALLOW((gemm_kernel<3, 1, 2, 16>), kGemmLds)
  QTIP_ALLOW((gemm_kernel<3, 2, 4, 8>), kGemmLds)
  QTIP_ALLOW((gemm4_kernel<1>), kGemm4Lds)
  QTIP_ALLOW((gemm4_kernel<2>), kGemm4Lds)
#undef QTIP_ALLOW
  return hipSuccess;
}

// Per-device set-up: CU count, LDS opt-in of every kernel, address of this device's copy of
// `scratch`.  qtip_init() runs it for the current device; a launcher that meets a device for the
// first time runs it too (none of it allocates or synchronises, but hipFuncSetAttribute is not
// a call to make while a stream is being captured: callers that record graphs call qtip_init()
// first).
struct DeviceState {
  int cus = 0;
  float* scratch_ptr = nullptr;
  std::atomic<bool> done{false};  // set last, read first: the fields above are complete when it is true
};
constexpr int kMaxDevices = 64;
DeviceState g_devices[kMaxDevices];
std::mutex g_devices_mutex;

// What a launcher learns about its device in one look: rc = 0, QTIP_E_NOT_INIT (first use of the
// device inside a stream capture: the set-up is not run there and nothing is launched) or the
// hipError_t of a failed set-up (tried again by the next call).
struct Ready {
  int rc;
  int cus;
  float* scratch;
};

// State of the current device, set up on first use.  `launching`: the caller is about to
// enqueue work on `st`.  One hipGetDevice per call; the mutex only on the first use of a device.
Ready ready(bool launching, hipStream_t st) {
  int dev = -1;
  const hipError_t ge = hipGetDevice(&dev);
  if (ge != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return Ready{(int)(ge != hipSuccess ? ge : hipErrorInvalidDevice), 0, nullptr};
  DeviceState& d = g_devices[dev];
  if (d.done.load(std::memory_order_acquire)) return Ready{0, d.cus, d.scratch_ptr};
  std::lock_guard<std::mutex> lock(g_devices_mutex);
  if (d.done.load(std::memory_order_relaxed)) return Ready{0, d.cus, d.scratch_ptr};
  if (launching) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    const hipError_t ce = hipStreamIsCapturing(st, &cs);
    if (ce == hipErrorStreamCaptureImplicit || (ce == hipSuccess && cs != hipStreamCaptureStatusNone))
      return Ready{QTIP_E_NOT_INIT, 0, nullptr};
    if (ce != hipSuccess) (void)hipGetLastError();  // the query's own error is not the caller's
  }
  int cus = 0;
  hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess) e = allow_lds_all();
  float* sp = nullptr;
  if (e == hipSuccess) e = hipGetSymbolAddress(reinterpret_cast<void**>(&sp), HIP_SYMBOL(scratch));
  if (e == hipSuccess && !sp) e = hipErrorInvalidSymbol;
  if (e != hipSuccess) return Ready{(int)e, 0, nullptr};
  d.cus = cus > 0 ? cus : 256;
  d.scratch_ptr = sp;
  d.done.store(true, std::memory_order_release);
  return Ready{0, d.cus, d.scratch_ptr};
}
Ready ready(void* stream) { return ready(true, (hipStream_t)stream); }

// CU count of the current device for the size queries: no set-up (they may be a process's first
// call on the device and may come while a stream is being captured), 0 when there is no device.
int query_cus() {
  int dev = -1, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  const DeviceState& d = g_devices[dev];
  if (d.done.load(std::memory_order_acquire)) return d.cus;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  return cus > 0 ? cus : 256;
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

// k split S for the shape: a workgroup walks `rounds` units of nwl/S wave-loads, and when the
// caller wants the summed vector (not the parts) a split costs one more small launch.
// Cost model of the k split, in units of one wave-load per wave (~0.08 us), fitted to launch times
// measured with cold weights: a unit costs its wave-loads per wave plus ~8 of fixed work (flush,
// barrier, stores; ~2 more when the output is a partial vector), a k range longer than the x
// staging area of LDS makes every wave-load ~20 % dearer (x then travels through vector loads),
// and a launch does not get shorter than ~24 however little each workgroup has to do.
int choose_split(int m, int k, int bits, int cus, bool summed) {
  (void)bits;
  const int nrb = m >> 5;
  const int nwl = ((k >> 5) + 3) >> 2;
  int best = 1;
  double best_cost = 1e30;
  for (int S = 1; S <= kMaxSplit; S *= 2) {
    if (nwl / S < kWaves && S > 1) break;  // keep at least one wave-load per wave
    const long units = (long)nrb * S;
    const long rounds = (units + cus - 1) / cus;
    const int wl_per = (nwl + S - 1) / S;
    const bool x_in_lds = (size_t)wl_per * 256 <= kMatvecXBytes;
    const double per_unit = (double)nwl / S * (x_in_lds ? 1.0 : 1.2) + 8.0 + (S > 1 ? 2.0 : 0.0);
    double cost = rounds * per_unit;
    if (cost < 24.0) cost = 24.0;
    if (S > 1 && summed) cost += 53.0;
    if (cost < best_cost * 0.97) {
      best_cost = cost;
      best = S;
    }
  }
  return best;
}

}  // namespace

extern "C" {

int qtip_abi_version(void) { return 20; }

int qtip_init(void) { return ready(false, nullptr).rc; }

const char* qtip_error_string(int code) {
  switch (code) {
    case QTIP_OK: return "ok";
    case QTIP_E_SHAPE: return "qtip: unsupported shape (need m % 32 == 0, k % 32 == 0, bits in 2..4, sizes in range)";
    case QTIP_E_NULL: return "qtip: null pointer argument";
    case QTIP_E_ALIGN: return "qtip: pointer not 16-byte aligned";
    case QTIP_E_WORKSPACE: return "qtip: workspace too small";
    case QTIP_E_DTYPE: return "qtip: unknown dtype code";
    case QTIP_E_NOT_INIT:
      return "qtip: first call on this device came inside a stream capture; call qtip_init() (or any "
             "launcher) on the device before capturing";
    case QTIP_E_SCRATCH:
      return "qtip: the partial sums of this call exceed the library's static scratch (256 KiB); use "
             "qtip_decompress_matvec with a caller workspace";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "qtip: unknown error";
  }
}

int qtip_decode(void* out_f16, const void* packed, const void* tlut, int m, int k, int bits,
                void* stream) {
  int rc = check_common(out_f16, packed, tlut, tlut, m, k, bits);
  if (rc) return rc;
  if (!aligned16(out_f16) || !aligned16(packed) || (reinterpret_cast<uintptr_t>(tlut) & 3u))
    return QTIP_E_ALIGN;
  const Ready di = ready(stream);
  if (di.rc) return di.rc;
  const long total = (long)(m >> 5) * (((k >> 5) + 3) >> 2);
  long want = (total + kWaves - 1) / kWaves;
  const int grid = (int)(want < di.cus ? want : di.cus);
  hipStream_t st = (hipStream_t)stream;
  auto* o = (uint16_t*)out_f16;
  auto* p = (const uint8_t*)packed;
  auto* t = (const uint32_t*)tlut;
  switch (bits) {
    case 2: decode_kernel<2><<<grid, kThreads, kDecodeLds, st>>>(o, p, t, m, k); break;
    case 3: decode_kernel<3><<<grid, kThreads, kDecodeLds, st>>>(o, p, t, m, k); break;
    default: decode_kernel<4><<<grid, kThreads, kDecodeLds, st>>>(o, p, t, m, k); break;
  }
  return (int)hipGetLastError();
}

int qtip_matvec_split(int m, int k, int bits) {
  if (m <= 0 || k <= 0 || (m & 31) || (k & 31) || bits < 2 || bits > 4) return 0;
  const int cus = query_cus();
  return cus ? choose_split(m, k, bits, cus, false) : 0;
}

size_t qtip_matvec_workspace_bytes(int m, int k, int bits) {
  if (m <= 0 || k <= 0 || (m & 31) || (k & 31) || bits < 2 || bits > 4) return 0;
  const int cus = query_cus();
  if (!cus) return 0;
  const int S = choose_split(m, k, bits, cus, true);
  return S > 1 ? (size_t)S * m * sizeof(float) : 0;
}

static int launch_matvec(const Ready& di, float* dst, const void* packed, const void* x_f16, const void* tlut,
                         int m, int k, int bits, int S, hipStream_t st, const void* su_f16 = nullptr,
                         float xscale = 1.f, const ChainArgs* chain = nullptr) {
  const long units = (long)(m >> 5) * S;
  long grid = units < di.cus ? units : di.cus;
  grid -= grid % S;  // a workgroup keeps one k range (units is a multiple of S, so grid >= S)
  const int nwl = ((k >> 5) + 3) >> 2;
  const int wl_per = (nwl + S - 1) / S;
  auto* p = (const uint8_t*)packed;
  auto* xx = (const uint16_t*)x_f16;
  auto* t = (const uint32_t*)tlut;
  const int per_range = (int)(grid / S);  // workgroups per k range, each walks row blocks rb0, rb0 + per_range, ...
  const dim3 g2((unsigned)S, (unsigned)per_range);
  const int uq = (m >> 5) / per_range, ur = (m >> 5) % per_range;
  if (su_f16) {
    // input transform inside the prologue: the whole transformed vector lives in LDS
    const size_t lds = kMatvecLds + (size_t)k * 2;
    auto* sg = (const uint16_t*)su_f16;
    if (chain) {
      switch (bits) {
        case 2: matvec_kernel<2, 2, true, 2><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale, *chain); break;
        case 3: matvec_kernel<3, 2, true, 2><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale, *chain); break;
        default: matvec_kernel<4, 2, true, 2><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale, *chain); break;
      }
      return (int)hipGetLastError();
    }
    switch (bits) {
      case 2: matvec_kernel<2, 2, true, 1><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale); break;
      case 3: matvec_kernel<3, 2, true, 1><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale); break;
      default: matvec_kernel<4, 2, true, 1><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur, sg, xscale); break;
    }
    return (int)hipGetLastError();
  }
  const size_t xbytes = (size_t)wl_per * 256;
  // row blocks left over by the rounds of whole units, when they fill at most half a round of the
  // full grid: each is cut into its two row halves (see HALF at the kernel).  The half units follow
  // the whole ones in the same two-stage load pipeline, so the whole units must end on an even
  // item.  Measured at 2 bits: 10240x8192 11.1 -> 9.8 us, 12288x4096 7.15 -> 6.6 us, and matrices
  // that do not fill one round - 4096x4096 4.8 -> 4.55 us, 4096x11008 7.9 -> 6.9 us (half the
  // decode per workgroup on twice the workgroups).  At 3 and 4 bits the doubled stream of the
  // left-over blocks costs what the halved decode saves (slower on the 4096-wide matrices, 2-4 %
  // faster on 10240x8192 only), so those keep whole units.
  const int full_range = di.cus / S;
  const int left = full_range > 0 ? (m >> 5) % full_range : 0;
  const int whole = full_range > 0 ? (m >> 5) / full_range : 0;
  const bool even_items = (((wl_per + kWaves - 1) / kWaves) & 1) == 0;
  if (bits == 2 && xbytes <= kMatvecXBytes && left > 0 && 2 * left <= full_range && (whole == 0 || even_items)) {
    const dim3 gh((unsigned)S, (unsigned)(whole > 0 ? full_range : 2 * left));
    matvec_kernel<2, 2, true, 0, false, false, true><<<gh, kThreads, kMatvecLds + xbytes, st>>>(
        dst, p, xx, t, m, k, wl_per, whole, 2 * left);
    return (int)hipGetLastError();
  }
  if (xbytes <= kMatvecXBytes) {
    const size_t lds = kMatvecLds + xbytes;
    switch (bits) {
      case 2: matvec_kernel<2, 2, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      case 3: matvec_kernel<3, 2, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      default: matvec_kernel<4, 2, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
    }
  } else if (uq == 1 && ur == 0 && (size_t)((((wl_per + kWaves - 1) / kWaves) + 1) >> 1) * kWaves * 256 <= kMatvecXBytes) {
    // one unit per workgroup and a k range of at most twice the staging area: x in two halves
    const size_t lds = kMatvecLds + kMatvecXBytes;
    switch (bits) {
      case 2: matvec_kernel<2, 2, true, 0, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      case 3: matvec_kernel<3, 2, true, 0, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      default: matvec_kernel<4, 2, true, 0, true><<<g2, kThreads, lds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
    }
  } else {
    switch (bits) {
      case 2: matvec_kernel<2, 2, false><<<g2, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      case 3: matvec_kernel<3, 2, false><<<g2, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
      default: matvec_kernel<4, 2, false><<<g2, kThreads, kMatvecLds, st>>>(dst, p, xx, t, m, k, wl_per, uq, ur); break;
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
  return QTIP_OK;
}

#ifdef QTIP_STAMPS
// copies the clock readings of the timeline build (64 x 256 x 16 x 8 bytes) to host memory;
// synchronises the device
int qtip_debug_stamps(void* host_buf) {
  hipError_t e = hipDeviceSynchronize();
  if (e == hipSuccess) e = hipMemcpyFromSymbol(host_buf, HIP_SYMBOL(g_stamps), sizeof(g_stamps));
  return (int)e;
}
#endif

int qtip_decompress_matvec_parts(float* parts, const void* packed, const void* x_f16,
                                 const void* tlut, int m, int k, int bits, int nparts,
                                 void* stream) {
  int rc = check_matvec(parts, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (nparts < 1 || nparts > kMaxSplit || nparts > ((((k >> 5) + 3) >> 2))) return QTIP_E_SHAPE;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  return launch_matvec(rd, parts, packed, x_f16, tlut, m, k, bits, nparts, (hipStream_t)stream);
}

int qtip_decompress_matvec_parts_rht(float* parts, const void* packed, const void* x_raw_f16,
                                     const void* su_f16, float scale, const void* tlut, int m, int k,
                                     int bits, int nparts, void* stream) {
  int rc = check_matvec(parts, packed, x_raw_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (!su_f16) return QTIP_E_NULL;
  if (k != 2048 && k != 4096 && k != 8192) return QTIP_E_SHAPE;
  if (nparts < 1 || nparts > kMaxSplit || nparts > (k >> 7)) return QTIP_E_SHAPE;
  if (!aligned16(x_raw_f16) || !aligned16(su_f16)) return QTIP_E_ALIGN;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  return launch_matvec(rd, parts, packed, x_raw_f16, tlut, m, k, bits, nparts, (hipStream_t)stream, su_f16, scale);
}

int qtip_decompress_matvec_parts_chain(float* parts, const void* packed, const void* tlut, int m, int k,
                                       int bits, int nparts, const float* prev_parts, int prev_nparts,
                                       size_t prev_part_stride, const float* post, float scale_out,
                                       const void* residual_f16, const void* norm_w_f16, float eps,
                                       const void* su_f16, float scale_in, void* x_out_f16,
                                       void* stream) {
  int rc = check_matvec(parts, packed, su_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (!prev_parts || !post || !residual_f16 || !norm_w_f16 || !x_out_f16) return QTIP_E_NULL;
  if (k != 2048 && k != 4096 && k != 8192) return QTIP_E_SHAPE;
  if (nparts < 1 || nparts > kMaxSplit || nparts > (k >> 7)) return QTIP_E_SHAPE;
  if (prev_nparts < 1 || prev_nparts > kMaxSplit || x_out_f16 == residual_f16) return QTIP_E_SHAPE;
  if (!aligned16(prev_parts) || !aligned16(post) || !aligned16(residual_f16) || !aligned16(norm_w_f16) ||
      !aligned16(su_f16) || !aligned16(x_out_f16) || ((prev_part_stride * sizeof(float)) & 15u))
    return QTIP_E_ALIGN;
  ChainArgs c;
  c.parts = prev_parts;
  c.post = post;
  c.residual = (const _Float16*)residual_f16;
  c.norm_w = (const _Float16*)norm_w_f16;
  c.x_out = (_Float16*)x_out_f16;
  c.part_stride = prev_part_stride;
  c.scale_out = scale_out;
  c.eps = eps;
  c.in_parts = prev_nparts;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  return launch_matvec(rd, parts, packed, su_f16, tlut, m, k, bits, nparts, (hipStream_t)stream, su_f16, scale_in, &c);
}

}  // extern "C"

// Workgroups per k range shared out among the matrices of a grouped launch in proportion to
// their row blocks (at least one each, never more than a matrix has row blocks); fills every
// field of GroupArgs except the pointers' meaning-specific ones (su / x).  Returns the number of
// workgroups per k range, 0 if the device is too small for the group.
static int share_out_group(int cus, GroupArgs& ga, float* parts, int ngroups, const void* const* packed,
                           const void* const* tlut, const int* m, int S, long m_total) {
  const int P = cus / S;
  if (P < ngroups) return 0;
  int nrb[3] = {0, 0, 0}, wg[3] = {0, 0, 0};
  long nrb_total = 0;
  for (int g = 0; g < ngroups; ++g) {
    nrb[g] = m[g] >> 5;
    nrb_total += nrb[g];
  }
  int used = 0;
  for (int g = 0; g < ngroups; ++g) {
    long w = (long)P * nrb[g] / nrb_total;
    if (w < 1) w = 1;
    if (w > nrb[g]) w = nrb[g];
    wg[g] = (int)w;
    used += wg[g];
  }
  while (used > P) {  // the minimum of one per matrix can overshoot
    int big = 0;
    for (int g = 1; g < ngroups; ++g)
      if (wg[g] > wg[big]) big = g;
    --wg[big];
    --used;
  }
  for (bool grown = true; used < P && grown;) {  // leftovers go where a workgroup has the most units
    grown = false;
    int best = -1;
    double most = 1.0;
    for (int g = 0; g < ngroups; ++g) {
      const double load = (double)nrb[g] / wg[g];
      if (wg[g] < nrb[g] && load > most) {
        most = load;
        best = g;
      }
    }
    if (best >= 0) {
      ++wg[best];
      ++used;
      grown = true;
    }
  }
  int begin = 0;
  long col = 0;
  for (int g = 0; g < 3; ++g) {
    const int gg = g < ngroups ? g : ngroups - 1;
    ga.dst[g] = parts + (g < ngroups ? col : 0);
    ga.packed[g] = (const uint8_t*)packed[gg];
    ga.tlut[g] = (const uint32_t*)tlut[gg];
    ga.su[g] = nullptr;
    ga.x[g] = nullptr;
    ga.m[g] = m[gg];
    ga.wg_begin[g] = g < ngroups ? begin : used;
    ga.upw_q[g] = g < ngroups ? nrb[g] / wg[g] : 0;
    ga.upw_r[g] = g < ngroups ? nrb[g] % wg[g] : 0;
    if (g < ngroups) {
      begin += wg[g];
      col += m[g];
    }
  }
  ga.wg_begin[3] = used;
  ga.part_stride = (size_t)m_total;
  return used;
}

extern "C" {

int qtip_decompress_matvec_group_chain(float* parts, int ngroups, const void* const* packed,
                                       const void* const* tlut, const void* const* su_f16, const int* m,
                                       int k, int bits, int nparts, const float* prev_parts,
                                       int prev_nparts, size_t prev_part_stride, const float* post,
                                       float scale_out, const void* residual_f16, const void* norm_w_f16,
                                       float eps, float scale_in, void* x_out_f16, void* stream) {
  if (!parts || !packed || !tlut || !su_f16 || !m) return QTIP_E_NULL;
  if (ngroups < 1 || ngroups > 3) return QTIP_E_SHAPE;
  long m_total = 0;
  for (int g = 0; g < ngroups; ++g) {
    int rc = check_matvec(parts, packed[g], su_f16[g], tlut[g], m[g], k, bits);
    if (rc) return rc;
    if (!aligned16(su_f16[g])) return QTIP_E_ALIGN;
    m_total += m[g];
  }
  if (!prev_parts || !post || !residual_f16 || !norm_w_f16 || !x_out_f16) return QTIP_E_NULL;
  if (k != 2048 && k != 4096 && k != 8192) return QTIP_E_SHAPE;
  if (nparts < 1 || nparts > kMaxSplit || nparts > (k >> 7)) return QTIP_E_SHAPE;
  if (prev_nparts < 1 || prev_nparts > kMaxSplit || x_out_f16 == residual_f16) return QTIP_E_SHAPE;
  if (!aligned16(prev_parts) || !aligned16(post) || !aligned16(residual_f16) || !aligned16(norm_w_f16) ||
      !aligned16(x_out_f16) || ((prev_part_stride * sizeof(float)) & 15u))
    return QTIP_E_ALIGN;
  ChainArgs c;
  c.parts = prev_parts;
  c.post = post;
  c.residual = (const _Float16*)residual_f16;
  c.norm_w = (const _Float16*)norm_w_f16;
  c.x_out = (_Float16*)x_out_f16;
  c.part_stride = prev_part_stride;
  c.scale_out = scale_out;
  c.eps = eps;
  c.in_parts = prev_nparts;

  const int S = nparts;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  GroupArgs ga;
  const int used = share_out_group(rd.cus, ga, parts, ngroups, packed, tlut, m, S, m_total);
  if (used == 0) return QTIP_E_SHAPE;
  for (int g = 0; g < 3; ++g) ga.su[g] = (const uint16_t*)su_f16[g < ngroups ? g : ngroups - 1];
  const int nwl = ((k >> 5) + 3) >> 2;
  const int wl_per = (nwl + S - 1) / S;
  const dim3 g2((unsigned)S, (unsigned)used);
  const size_t lds = kMatvecLds + (size_t)k * 2;
  hipStream_t st = (hipStream_t)stream;
  switch (bits) {
    case 2: matvec_kernel<2, 2, true, 2, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, scale_in, c, ga); break;
    case 3: matvec_kernel<3, 2, true, 2, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, scale_in, c, ga); break;
    default: matvec_kernel<4, 2, true, 2, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, scale_in, c, ga); break;
  }
  return (int)hipGetLastError();
}

int qtip_decompress_matvec_group(float* parts, int ngroups, const void* const* packed,
                                 const void* const* x_f16, const void* const* tlut, const int* m, int k,
                                 int bits, int nparts, void* stream) {
  if (!parts || !packed || !tlut || !x_f16 || !m) return QTIP_E_NULL;
  if (ngroups < 1 || ngroups > 3) return QTIP_E_SHAPE;
  long m_total = 0;
  for (int g = 0; g < ngroups; ++g) {
    int rc = check_matvec(parts, packed[g], x_f16[g], tlut[g], m[g], k, bits);
    if (rc) return rc;
    if (!aligned16(x_f16[g])) return QTIP_E_ALIGN;
    m_total += m[g];
  }
  const int nwl = ((k >> 5) + 3) >> 2;
  if (nparts < 1 || nparts > kMaxSplit || nparts > nwl) return QTIP_E_SHAPE;
  const int S = nparts;
  const int wl_per = (nwl + S - 1) / S;
  const size_t xbytes = (size_t)wl_per * 256;
  if (xbytes > kMatvecXBytes) return QTIP_E_SHAPE;  // the grouped plain form keeps x in LDS
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  GroupArgs ga;
  const int used = share_out_group(rd.cus, ga, parts, ngroups, packed, tlut, m, S, m_total);
  if (used == 0) return QTIP_E_SHAPE;
  for (int g = 0; g < 3; ++g) ga.x[g] = (const uint16_t*)x_f16[g < ngroups ? g : ngroups - 1];
  const dim3 g2((unsigned)S, (unsigned)used);
  const size_t lds = kMatvecLds + xbytes;
  hipStream_t st = (hipStream_t)stream;
  switch (bits) {
    case 2: matvec_kernel<2, 2, true, 0, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, 1.f, ChainArgs{}, ga); break;
    case 3: matvec_kernel<3, 2, true, 0, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, 1.f, ChainArgs{}, ga); break;
    default: matvec_kernel<4, 2, true, 0, false, true><<<g2, kThreads, lds, st>>>(nullptr, nullptr, nullptr, nullptr, 0, k, wl_per, 0, 0, nullptr, 1.f, ChainArgs{}, ga); break;
  }
  return (int)hipGetLastError();
}

int qtip_decompress_matvec(float* out, const void* packed, const void* x_f16, const void* tlut,
                           int m, int k, int bits, void* workspace, size_t workspace_bytes,
                           void* stream) {
  int rc = check_matvec(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  int S = 1;
  if (workspace) {
    S = choose_split(m, k, bits, rd.cus, true);
    if (S > 1 && workspace_bytes < (size_t)S * m * sizeof(float)) return QTIP_E_WORKSPACE;
    if (!aligned16(workspace)) return QTIP_E_ALIGN;
  }
  hipStream_t st = (hipStream_t)stream;
  if (S == 1) return launch_matvec(rd, out, packed, x_f16, tlut, m, k, bits, 1, st);
  rc = launch_matvec(rd, (float*)workspace, packed, x_f16, tlut, m, k, bits, S, st);
  if (rc) return rc;
  sum_parts_kernel<<<(m + 255) / 256, 256, 0, st>>>(out, (const float*)workspace, m, S);
  return (int)hipGetLastError();
}

int qtip_decompress_matvec_noalloc(float* out, const void* packed, const void* x_f16, const void* tlut,
                                   int m, int k, int bits, int nparts, void* stream) {
  int rc = check_matvec(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  const Ready rd = ready(stream);
  if (rd.rc) return rd.rc;
  const int nwl = ((k >> 5) + 3) >> 2;
  if (nparts < 0 || nparts > kMaxSplit || nparts > nwl) return QTIP_E_SHAPE;
  int S = nparts;
  if (S == 0) {
    // the library's own choice, halved until its partial sums fit the scratch (S = 1 needs none)
    S = choose_split(m, k, bits, rd.cus, true);
    while (S > 1 && (size_t)S * m > kScratchFloats) S >>= 1;
  }
  hipStream_t st = (hipStream_t)stream;
  if (S == 1) return launch_matvec(rd, out, packed, x_f16, tlut, m, k, bits, 1, st);
  if ((size_t)S * m > kScratchFloats) return QTIP_E_SCRATCH;  // only a split the caller asked for
  // every one of the S * m partial sums is written before it is read: nothing to clear
  float* parts = rd.scratch;
  rc = launch_matvec(rd, parts, packed, x_f16, tlut, m, k, bits, S, st);
  if (rc) return rc;
  sum_parts_kernel<<<(m + 255) / 256, 256, 0, st>>>(out, parts, m, S);
  return (int)hipGetLastError();
}

// k split of the batched GEMM: groups of 4 row blocks are the parallel units, so matrices with
// few rows are also cut along k (only when the caller provides room for the partial results)
static int gemm_split(int m, int k, int cus) {
  const int ngroups = ((m >> 5) + kGemmRB - 1) / kGemmRB;
  const int nwl = ((k >> 5) + 3) >> 2;
  int S = 1;
  while (S < kMaxSplit && ngroups * S * 2 <= cus && nwl / (S * 2) >= 8) S *= 2;
  return S;
}

size_t qtip_gemm_workspace_bytes(int m, int k, int bits, int batch) {
  if (m <= 0 || k <= 0 || (m & 31) || (k & 31) || bits < 2 || bits > 4 || batch < 1) return 0;
  const int cus = query_cus();
  if (!cus) return 0;
  const int S = gemm_split(m, k, cus);
  return S > 1 ? (size_t)S * (batch < 32 ? batch : 32) * m * sizeof(float) : 0;
}

int qtip_decompress_gemm(float* out, const void* packed, const void* x_f16, const void* tlut,
                         int m, int k, int bits, int batch, int round_f16, void* workspace,
                         size_t workspace_bytes, void* stream) {
  int rc = check_common(out, packed, x_f16, tlut, m, k, bits);
  if (rc) return rc;
  if (batch < 1 || batch > 65535) return QTIP_E_SHAPE;
  if (!aligned16(packed) || !aligned16(x_f16) || (reinterpret_cast<uintptr_t>(tlut) & 3u) ||
      (reinterpret_cast<uintptr_t>(out) & 3u))
    return QTIP_E_ALIGN;
  const Ready di = ready(stream);
  if (di.rc) return di.rc;
  int S = 1;
  if (workspace) {
    S = gemm_split(m, k, di.cus);
    if (S > 1 && workspace_bytes < (size_t)S * (batch < 32 ? batch : 32) * m * sizeof(float))
      return QTIP_E_WORKSPACE;
    if (!aligned16(workspace)) return QTIP_E_ALIGN;
  }
  const int ngroups = ((m >> 5) + kGemmRB - 1) / kGemmRB;
  const int nwl = ((k >> 5) + 3) >> 2;
  hipStream_t st = (hipStream_t)stream;
  auto* p = (const uint8_t*)packed;
  auto* t = (const uint32_t*)tlut;
  // batch handled in passes of at most 32 rows: two 16-row MFMA tiles on the 8-wave workgroup;
  // up to 16 rows run on the 16-wave workgroup (4 wave-loads per stage)
  for (int b0 = 0; b0 < batch; b0 += 32) {
    const int nb = batch - b0 < 32 ? batch - b0 : 32;
    const bool rowsplit = bits == 4;  // the 4-bit kernel without duplicated products, 16 waves for every batch
    const int KS = (rowsplit || nb <= 16) ? 4 : 2;
    int Sp = S;
    int wl_per = (nwl + Sp - 1) / Sp;
    wl_per = (wl_per + KS - 1) / KS * KS;  // stages are groups of KS wave-loads
    Sp = (nwl + wl_per - 1) / wl_per;      // rounding up may have emptied the last ranges
    const long units = (long)ngroups * Sp;
    long grid = units < di.cus ? units : di.cus;
    grid -= grid % Sp;  // a workgroup keeps one k range
    const int per_range = (int)(grid / Sp);
    const dim3 g2((unsigned)Sp, (unsigned)per_range);
    float* o = out + (size_t)b0 * m;
    float* d = Sp > 1 ? (float*)workspace : o;
    const int rnd = Sp > 1 ? 0 : round_f16;
    const uint16_t* xx = (const uint16_t*)x_f16 + (size_t)b0 * k;
#define QTIP_GEMM(KB, NBT, WV)                                                                          \
  gemm_kernel<KB, NBT, (KB == 2 ? 4 : (WV == 16 ? 2 : 4)), WV><<<g2, WV * 64, kGemmLds, st>>>( \
      d, p, xx, t, m, k, nb, rnd, wl_per, ngroups / per_range, ngroups % per_range)
#define QTIP_GEMM_K(KB)               \
  if (nb <= 16) QTIP_GEMM(KB, 1, 16); \
  else QTIP_GEMM(KB, 2, 8);
    if (rowsplit) {
      if (nb <= 16)
        gemm4_kernel<1><<<g2, kThreads, kGemm4Lds, st>>>(d, p, xx, t, m, k, nb, rnd, wl_per, ngroups / per_range,
                                                         ngroups % per_range);
      else
        gemm4_kernel<2><<<g2, kThreads, kGemm4Lds, st>>>(d, p, xx, t, m, k, nb, rnd, wl_per, ngroups / per_range,
                                                         ngroups % per_range);
    } else {
      if (bits == 2) { QTIP_GEMM_K(2) } else { QTIP_GEMM_K(3) }
    }
#undef QTIP_GEMM_K
#undef QTIP_GEMM
    hipError_t le = hipGetLastError();
    if (le != hipSuccess) return (int)le;
    if (Sp > 1) {
      const long n = (long)nb * m;
      sum_parts_round_kernel<<<(int)((n + 255) / 256), 256, 0, st>>>(o, (const float*)workspace, n, Sp, round_f16);
      le = hipGetLastError();
      if (le != hipSuccess) return (int)le;
    }
  }
  return QTIP_OK;
}

}  // extern "C"
