// Device-side building blocks shared by the decode, matvec and GEMM kernels.
//
// Lane mapping (all bit widths K = 2,3,4).  The packed stream is an array
// [m/32][k/32][ref lane 32][kh 2][mh 2][K bytes]: one 2x2 block of 16x16 tiles
// is 128*K contiguous bytes and "ref lane" l owns 4*K of them (one K-byte
// chunk of each of the four tiles).  A chunk decodes only together with the
// leading 16 bits of ref lane (l+1) mod 32's chunk of the same tile.
//
// A 64-wide wavefront reads four consecutive 2x2 blocks ("wave-load",
// 512*K bytes).  Lane = 16*g + a takes block g and the two ref lanes 2a and
// 2a+1, i.e. 8*K contiguous bytes.  Ref lane 2a finds its successor in the
// same lane's registers; ref lane 2a+1 needs lane a+1's first chunk, and the
// ring closes inside the 16-lane DPP row (row_ror:15), so the neighbour
// exchange never leaves the VALU.
//
// Per wave-load a lane decodes 32 states = 64 weights:
//   rows    32*rb + 16*mh + 8*rh + a/2          (mh, rh in {0,1})
//   columns 32*kb + 16*kh + 8*jh + 4*(a%2) + {0,1 (ref A), 2,3 (ref B)}
// with tile t = 2*kh + mh inside the ref lane's bytes and state j = 2*jh + rh
// inside the chunk.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qtip {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// LDS weight table: 1024 entries (9 index bits + the sign bit of the hash as
// a tenth), each replicated 16 times so that a lane reads replica (lane % 16).
// Entry e sits at byte e*64, which is exactly bits 6..15 of the hash value.
constexpr int kLutEntries = 1024;
constexpr int kLutBytes = kLutEntries * 64;

// Fill the table from the raw 512 x (fp16,fp16) tunable LUT.  Entry
// e = sign*512 + q holds tlut[q] with element 0 (the low half) negated when
// sign is set: the quantlut_sym rule.
__device__ __forceinline__ void build_lut(uint32_t* lut, const uint32_t* __restrict__ tlut,
                                          int tid, int nthreads) {
  for (int e = tid; e < kLutEntries; e += nthreads) {
    uint32_t w = tlut[e & 511] ^ ((uint32_t)(e >> 9) << 15);
    u32x4 v = {w, w, w, w};
    u32x4* dst = reinterpret_cast<u32x4*>(lut + e * 16);
    dst[0] = v;
    dst[1] = v;
    dst[2] = v;
    dst[3] = v;
  }
}

template <int K>
struct LaneData {
  uint32_t d[2 * K];  // ref lane A = d[0..K), ref lane B = d[K..2K)
};

// A lane's 8*K bytes of the stream for the dense decode.  Plain loads: beside that kernel's
// non-temporal stores, non-temporal loads measured 15-20 % slower at every bit width
// (57344x8192 at 2 bits: 237 -> 198 us), and at 4 bits a lane's two 16-byte loads share
// their cache lines, which the hint makes the second one fetch from L2 again.
template <int K>
__device__ __forceinline__ LaneData<K> load_lane(const uint8_t* __restrict__ p) {
  LaneData<K> r;
  if constexpr (K == 3) {
    const u32x2* q = reinterpret_cast<const u32x2*>(p);
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      u32x2 v = q[i];
      r.d[2 * i] = v[0];
      r.d[2 * i + 1] = v[1];
    }
  } else {
    const u32x4* q = reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int i = 0; i < K / 2; ++i) {
      u32x4 v = q[i];
      r.d[4 * i] = v[0];
      r.d[4 * i + 1] = v[1];
      r.d[4 * i + 2] = v[2];
      r.d[4 * i + 3] = v[3];
    }
  }
  return r;
}

// Chunk of tile t of one ref lane (e = that ref lane's K dwords) as the
// big-endian integer of its 8*K stream bits.
template <int K>
__device__ __forceinline__ uint32_t chunk(const uint32_t* e, int t) {
  if constexpr (K == 2) {
    return (t & 1) ? (e[t >> 1] >> 16) : (e[t >> 1] & 0xFFFFu);
  } else if constexpr (K == 3) {
    switch (t) {
      case 0: return e[0] & 0xFFFFFFu;
      case 1: return (e[0] >> 24) | ((e[1] & 0xFFFFu) << 8);
      case 2: return (e[1] >> 16) | ((e[2] & 0xFFu) << 16);
      default: return e[2] >> 8;
    }
  } else {
    return e[t];
  }
}

// value of lane (a+1) mod 16 of the same 16-lane row
__device__ __forceinline__ uint32_t from_next_lane16(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x12F /* row_ror:15 */, 0xF, 0xF, false);
}

// All 32 states of a lane's wave-load: st[R][t][j], R = ref lane (A,B),
// t = tile 2*kh+mh, j = state inside the chunk.  Only the low 16 bits of each
// value are meaningful; higher bits hold leftovers of the window and are
// harmless because the hash uses the low 16 bits of its result only.
template <int K>
__device__ __forceinline__ void lane_states(const LaneData<K>& ld, uint32_t st[2][4][4]) {
  uint32_t own[2][4], top[2][4];
#pragma unroll
  for (int R = 0; R < 2; ++R)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      own[R][t] = chunk<K>(&ld.d[R * K], t);
      top[R][t] = own[R][t] >> (8 * K - 16);
    }
  // what the previous lane's ref B needs from this lane's ref A
  uint32_t s01, s23;
  if constexpr (K == 2) {
    s01 = ld.d[0];
    s23 = ld.d[1];
  } else {
    s01 = top[0][0] | (top[0][1] << 16);
    s23 = top[0][2] | (top[0][3] << 16);
  }
  const uint32_t r01 = from_next_lane16(s01);
  const uint32_t r23 = from_next_lane16(s23);
  uint32_t nxt[2][4];
#pragma unroll
  for (int t = 0; t < 4; ++t) nxt[0][t] = top[1][t];
  nxt[1][0] = r01 & 0xFFFFu;
  nxt[1][1] = r01 >> 16;
  nxt[1][2] = r23 & 0xFFFFu;
  nxt[1][3] = r23 >> 16;
#pragma unroll
  for (int R = 0; R < 2; ++R)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t o = own[R][t];
      const uint32_t v = (o << 16) | nxt[R][t];  // low 32 bits of chunk || next16
      if constexpr (K == 2) {
        st[R][t][0] = o;
        st[R][t][1] = v >> 12;
        st[R][t][2] = v >> 8;
        st[R][t][3] = v >> 4;
      } else if constexpr (K == 3) {
        st[R][t][0] = o >> 8;
        st[R][t][1] = o >> 2;
        st[R][t][2] = v >> 12;
        st[R][t][3] = v >> 6;
      } else {
        st[R][t][0] = o >> 16;
        st[R][t][1] = o >> 8;
        st[R][t][2] = o;
        st[R][t][3] = v >> 8;
      }
    }
}

// HYB lookup: p = s*(s+1); bits 6..15 of p address the sign-folded table.
__device__ __forceinline__ uint32_t lut_lookup(const uint32_t* lut, uint32_t s, uint32_t slot4) {
  const uint32_t p = __umul24(s, s) + s;
  const uint32_t addr = (p & 0xFFC0u) | slot4;
  return *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(lut) + addr);
}

// ---------------------------------------------------------------------------
// Fast path of the matvec: conflict-free table and packed 16-bit hashing.
//
// Table: 1024 entries x 32 replicas x 4 bytes = 128 KiB, entry e at byte
// e*128, replica (lane % 32) at +4*(lane%32): every lane of a half-wave reads
// its own LDS bank, so a gather of 64 random entries takes the same time as a
// broadcast.  Two states travel in one register (16 bits each):
//   hash      v_pk_mad_u16  p = s*s + s           (one instruction, two states)
//   mask      v_and_b32     q = p & 0xFFC0FFC0    (bits 6..15 = entry, both halves)
//   address   v_mad_u32_u16 a = q.half * 2 + slot4 (op_sel picks the half)
// The instructions are written as inline asm because the compiler rewrites
// s*s+s into add+mul and picks 64-bit multiplies for the unpacked form.
// ---------------------------------------------------------------------------
constexpr int kLut128Bytes = kLutEntries * 128;

__device__ __forceinline__ void build_lut128(uint32_t* lut, const uint32_t* __restrict__ tlut,
                                             int tid, int nthreads) {
  // thread handles (entry, quarter): 32 bytes x 4 quarters... one u32x4 per step
  for (int i = tid; i < kLutEntries * 8; i += nthreads) {
    const int e = i >> 3;
    uint32_t w = tlut[e & 511] ^ ((uint32_t)(e >> 9) << 15);
    u32x4 v = {w, w, w, w};
    reinterpret_cast<u32x4*>(lut)[i] = v;
  }
}

// p.lo = s.lo*s.lo + s.lo, p.hi = s.hi*s.hi + s.hi (mod 2^16 each)
__device__ __forceinline__ uint32_t pk_hash(uint32_t s) {
  uint32_t r;
  asm("v_pk_mad_u16 %0, %1, %1, %1" : "=v"(r) : "v"(s));
  return r;
}
// per half: a * c + b (mod 2^16); cst holds the same 16-bit constant in both halves
__device__ __forceinline__ uint32_t pk_mad_const(uint32_t a, uint32_t cst, uint32_t b) {
  uint32_t r;
  asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(cst), "v"(b));
  return r;
}
__device__ __forceinline__ uint32_t pk_shr(uint32_t a, int sh) {
  typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
  u16x2 v = __builtin_bit_cast(u16x2, a);
  v = v >> (u16x2)(uint16_t)sh;
  return __builtin_bit_cast(uint32_t, v);
}
// unpacked hash (only the low 16 bits of s and of the result are meaningful)
__device__ __forceinline__ uint32_t hash24(uint32_t s) {
  uint32_t r;
  asm("v_mad_u32_u24 %0, %1, %1, %1" : "=v"(r) : "v"(s));
  return r;
}
// LDS byte address of the entry selected by the low / high half of q = p & 0xFFC0FFC0
__device__ __forceinline__ uint32_t lut128_addr_lo(uint32_t q, uint32_t slot4) {
  uint32_t r;
  asm("v_mad_u32_u16 %0, %1, 2, %2 op_sel:[0,0,0,0]" : "=v"(r) : "v"(q), "v"(slot4));
  return r;
}
__device__ __forceinline__ uint32_t lut128_addr_hi(uint32_t q, uint32_t slot4) {
  uint32_t r;
  asm("v_mad_u32_u16 %0, %1, 2, %2 op_sel:[1,0,0,0]" : "=v"(r) : "v"(q), "v"(slot4));
  return r;
}
// ---------------------------------------------------------------------------
// Packed state extraction: 16 registers per lane per wave-load, two 16-bit
// states in each.  Register i and half h (0 = low) stand for
//   K = 2,3:  i = (R*2 + kh)*4 + j,  half h -> tile row half mh = h
//   K = 4:    i = (R*4 + 2*kh + mh)*2 + u,  half h -> j = 2*(1-h) + u
// (R = ref lane A/B, j = state inside the chunk = 2*jh + rh).  pk_meta gives
// the x pair (2*kh + jh) and the accumulator (2*mh + rh) of a half.
// ---------------------------------------------------------------------------
template <int K>
struct PkMeta {
  static constexpr __device__ int R(int i) { return K == 4 ? (i >> 3) : (i >> 3); }
  static constexpr __device__ int xq(int i, int h) {
    if (K == 4) {
      const int kh = (i >> 2) & 1, u = i & 1, j = 2 * (1 - h) + u;
      return 2 * kh + (j >> 1);
    }
    const int kh = (i >> 2) & 1, j = i & 3;
    return 2 * kh + (j >> 1);
  }
  static constexpr __device__ int acc(int i, int h) {
    if (K == 4) {
      const int mh = (i >> 1) & 1, u = i & 1, j = 2 * (1 - h) + u;
      return 2 * mh + (j & 1);
    }
    const int j = i & 3;
    return 2 * h + (j & 1);
  }
};

__device__ __forceinline__ uint32_t perm(uint32_t hi_src, uint32_t lo_src, uint32_t sel) {
  // result byte b = selector byte b: 0..3 -> lo_src byte, 4..7 -> hi_src byte
  return __builtin_amdgcn_perm(hi_src, lo_src, sel);
}

template <int K>
__device__ __forceinline__ void packed_states(const LaneData<K>& ld, uint32_t P[16]) {
  if constexpr (K == 2) {
    // dword R*2+kh = chunk(mh=0) | chunk(mh=1) << 16; a chunk is 4 states of 4 bits
    const uint32_t nb0 = from_next_lane16(ld.d[0]);
    const uint32_t nb1 = from_next_lane16(ld.d[1]);
#pragma unroll
    for (int R = 0; R < 2; ++R)
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        const uint32_t d = ld.d[R * 2 + kh];
        const uint32_t n = R == 0 ? ld.d[2 + kh] : (kh == 0 ? nb0 : nb1);
        uint32_t* o = &P[(R * 2 + kh) * 4];
        o[0] = d;
        o[1] = pk_mad_const(d, 0x00100010u, pk_shr(n, 12));  // d<<4 | n>>12
        o[2] = perm(d, n, 0x06030401u);                       // d<<8 | n>>8
        o[3] = pk_mad_const(d, 0x10001000u, pk_shr(n, 4));   // d<<12 | n>>4
      }
  } else if constexpr (K == 3) {
    // 24-bit chunks c at byte 3t of the ref lane's 12 bytes.  Per tile pair:
    // X1 = c[23:8] (= state 0), X2 = c[15:0], NX = X1 of the successor.
    uint32_t X1[2][2], X2[2][2];
#pragma unroll
    for (int R = 0; R < 2; ++R) {
      const uint32_t e0 = ld.d[3 * R], e1 = ld.d[3 * R + 1], e2 = ld.d[3 * R + 2];
      X1[R][0] = perm(e0, e1, 0x01000605u);
      X2[R][0] = perm(e0, e1, 0x00070504u);
      X1[R][1] = perm(e1, e2, 0x03020007u);
      X2[R][1] = perm(e1, e2, 0x02010706u);
    }
    const uint32_t nb0 = from_next_lane16(X1[0][0]);
    const uint32_t nb1 = from_next_lane16(X1[0][1]);
#pragma unroll
    for (int R = 0; R < 2; ++R)
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        const uint32_t x1 = X1[R][kh], x2 = X2[R][kh];
        const uint32_t nx = R == 0 ? X1[1][kh] : (kh == 0 ? nb0 : nb1);
        uint32_t* o = &P[(R * 2 + kh) * 4];
        o[0] = x1;                                                      // c[23:8]
        o[1] = pk_mad_const(pk_shr(x1, 8), 0x40004000u, pk_shr(x2, 2));  // c[17:2]
        o[2] = pk_mad_const(x2, 0x00100010u, pk_shr(nx, 12));           // c[11:0] | nx[15:12]
        o[3] = pk_mad_const(x2, 0x04000400u, pk_shr(nx, 6));            // c[5:0] | nx[15:6]
      }
  } else {
    // 32-bit chunk c: states c[31:16], c[23:8], c[15:0], c[7:0] | next[31:24]
    uint32_t nb[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) nb[t] = from_next_lane16(ld.d[t]);
#pragma unroll
    for (int R = 0; R < 2; ++R)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t c = ld.d[R * 4 + t];
        const uint32_t cn = R == 0 ? ld.d[4 + t] : nb[t];
        P[(R * 4 + t) * 2] = c;                             // hi = state 0, lo = state 2
        P[(R * 4 + t) * 2 + 1] = perm(c, cn, 0x06050403u);  // hi = state 1, lo = state 3
      }
  }
}

// 32-bit LDS address of a __shared__ object and a load from such an address:
// with the table base folded into the per-lane slot offset, the address that
// v_mad_u32_u16 produces feeds ds_read_b32 directly (no per-lookup add).
typedef __attribute__((address_space(3))) const uint32_t lds_u32_t;
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ uint32_t lds_word_abs(uint32_t lds_addr) {
  return *(lds_u32_t*)(uintptr_t)lds_addr;
}

// index into W[32] (lookup order of the packed hashes) of state (R, t, j)
template <int K>
__device__ __forceinline__ constexpr int w_index(int R, int t, int j) {
  if (K == 4) return 2 * ((R * 4 + t) * 2 + (j & 1)) + (1 - (j >> 1));
  return 2 * ((R * 2 + (t >> 1)) * 4 + j) + (t & 1);
}


// 32 states of one wave-load.  All hashes, addresses and the 32 table reads are issued first, so
// a read has the rest of the address arithmetic (a few hundred cycles) to come back from LDS;
// the products run on the matrix core, which leaves the vector ALU to the decode (a v_dot2c per
// state measured 5 % slower end to end).  The four table words of a
// (tile row half mh, row half rh, kh) group are a v_mfma_f32_16x16x32_f16 B operand (N = the 16
// lanes `a` of a DPP row, K group = g), the lane's own eight x values of that kh are the A operand
// row `a`: D[i][j] = sum over (g, 8 halves) of x(lane i) * W(lane j), which is the wanted dot
// product whenever lanes i and j read the same columns, i.e. i % 2 == j % 2.  Lane (g, a) keeps
// D[4g + r][a] in element r, so element a % 2 of the accumulator is the lane's row sum over all
// four blocks of the wave-load (the cross-block reduction happens inside the MFMA).
//
// RH = 0 / 1 decodes only the states of row half rh = RH (rows 8*RH .. 8*RH + 7 of either tile
// row half): the registers P[i] with i % 2 == RH at every bit width, half the hashes, lookups and
// MFMAs and - the extraction of the others being dead code - about half the vector work.  The
// accumulators of the other row half stay untouched.
template <int K, int RH = -1>
__device__ __forceinline__ void matvec_accumulate(const LaneData<K>& ld, const u32x2 xv[4],
                                                       uint32_t slot4, float4_t acc[4]) {
  uint32_t P[16], W[32];
  packed_states<K>(ld, P);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    if (RH >= 0 && (i & 1) != RH) continue;
    const uint32_t q = pk_hash(P[i]) & 0xFFC0FFC0u;
    W[2 * i] = lds_word_abs(lut128_addr_lo(q, slot4));
    W[2 * i + 1] = lds_word_abs(lut128_addr_hi(q, slot4));
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int kh = 0; kh < 2; ++kh) {
    const u32x4 xa = {xv[2 * kh][0], xv[2 * kh][1], xv[2 * kh + 1][0], xv[2 * kh + 1][1]};
#pragma unroll
    for (int mh = 0; mh < 2; ++mh)
#pragma unroll
      for (int rh = 0; rh < 2; ++rh) {
        if (RH >= 0 && rh != RH) continue;
        const int tt = 2 * kh + mh;
        const u32x4 wv = {W[w_index<K>(0, tt, rh)], W[w_index<K>(1, tt, rh)],
                          W[w_index<K>(0, tt, 2 + rh)], W[w_index<K>(1, tt, 2 + rh)]};
        acc[2 * mh + rh] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            __builtin_bit_cast(half8_t, xa), __builtin_bit_cast(half8_t, wv), acc[2 * mh + rh], 0, 0, 0);
      }
  }
}

}  // namespace qtip
