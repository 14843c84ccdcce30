// Walsh-Hadamard building blocks shared by the transform kernels and the matvec prologue:
// cross-lane exchanges of a wave64, butterflies over lane bits and over a thread's registers,
// and the vector loads / stores of EPT consecutive elements.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qtip_wht {

typedef float float4w __attribute__((ext_vector_type(4)));

// value of lane ^ (1 << b) for b = 0..5
__device__ __forceinline__ float lane_xor(float v, int b) {
  const int u = __builtin_bit_cast(int, v);
  int r;
  switch (b) {
    case 0: r = __builtin_amdgcn_update_dpp(0, u, 0xB1, 0xF, 0xF, false); break;  // quad_perm 1,0,3,2
    case 1: r = __builtin_amdgcn_update_dpp(0, u, 0x4E, 0xF, 0xF, false); break;  // quad_perm 2,3,0,1
    // xor 4 and xor 16 go through the LDS crossbar: one instruction outside the vector pipe (two
    // bank-masked row rotations do xor 4 as well, but cost two vector instructions that cannot
    // ride on the addition; the transforms are bound by vector issue)
    case 2: r = __builtin_amdgcn_ds_swizzle(u, 0x101F); break;                    // xor 4
    case 3: r = __builtin_amdgcn_update_dpp(0, u, 0x128, 0xF, 0xF, false); break;  // xor 8 = row_ror:8
    case 4: r = __builtin_amdgcn_ds_swizzle(u, 0x401F); break;                    // xor 16
    default: {
      auto sw = __builtin_amdgcn_permlane32_swap((uint32_t)u, (uint32_t)u, false, false);
      r = (int)((threadIdx.x & 32) ? sw[0] : sw[1]);
    }
  }
  return __builtin_bit_cast(float, r);
}

// One butterfly over lane bit b: lanes with the bit clear get v + partner, the others partner - v.
// Written as partner + (v with its sign flipped where the bit is set): an xor and an addition (the
// exchange rides on the addition as a DPP operand) instead of an addition, a subtraction and a
// select; the sums are the same floating-point operations on the same operands.
__device__ __forceinline__ float wht_stage(float v, int b, int lane) {
  const uint32_t flip = ((uint32_t)lane << (31 - b)) & 0x80000000u;
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  if (b == 5) {
    // the swap exchanges the upper half of its first operand with the lower half of its second:
    // with (v, flipped v) the first result holds the lower half's values in either half and the
    // second the upper half's, negated where they stayed at home - their sum is the butterfly
    auto sw = __builtin_amdgcn_permlane32_swap(u, u ^ flip, false, false);
    return __builtin_bit_cast(float, (uint32_t)sw[0]) + __builtin_bit_cast(float, (uint32_t)sw[1]);
  }
  return lane_xor(v, b) + __builtin_bit_cast(float, u ^ flip);
}

// Walsh-Hadamard butterflies over lane bits lo .. nbits-1 (natural order)
__device__ __forceinline__ float wht_lanes(float v, int nbits, int lane, int lo = 0) {
#pragma unroll
  for (int b = 0; b < 6; ++b) {
    if (b >= lo && b < nbits) v = wht_stage(v, b, lane);
  }
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int b = 0; b < 6; ++b) v += lane_xor(v, b);
  return v;
}

// EPT consecutive elements as floats, with the widest loads the alignment (EPT elements) allows
template <int EPT>
__device__ __forceinline__ void ld_f32(const float* p, float v[EPT]) {
  if constexpr (EPT == 2) {
    const float2 t = *reinterpret_cast<const float2*>(p);
    v[0] = t.x;
    v[1] = t.y;
  } else {
#pragma unroll
    for (int q = 0; q < EPT / 4; ++q) {
      const float4w t = *reinterpret_cast<const float4w*>(p + 4 * q);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[4 * q + e] = t[e];
    }
  }
}
template <int EPT>
__device__ __forceinline__ void ld_f16(const _Float16* p, float v[EPT]) {
  typedef _Float16 hvec __attribute__((ext_vector_type(EPT)));
  const hvec t = *reinterpret_cast<const hvec*>(p);
#pragma unroll
  for (int e = 0; e < EPT; ++e) v[e] = (float)t[e];
}
template <int EPT>
__device__ __forceinline__ void st_f16(_Float16* p, const _Float16 v[EPT]) {
  typedef _Float16 hvec __attribute__((ext_vector_type(EPT)));
  hvec t;
#pragma unroll
  for (int e = 0; e < EPT; ++e) t[e] = v[e];
  *reinterpret_cast<hvec*>(p) = t;
}

template <int EPT>
__device__ __forceinline__ void wht_regs(float v[EPT]) {
#pragma unroll
  for (int h = 1; h < EPT; h <<= 1)
#pragma unroll
    for (int i = 0; i < EPT; ++i)
      if (!(i & h)) {
        const float a = v[i], b = v[i + h];
        v[i] = a + b;
        v[i + h] = a - b;
      }
}

// exchange buffer index of element e: one pad block of EPT floats per 64 lanes keeps the strided reads apart
template <int EPT>
__device__ __forceinline__ int xidx(int e) {
  return e + EPT * (e / (64 * EPT));
}


}  // namespace qtip_wht
