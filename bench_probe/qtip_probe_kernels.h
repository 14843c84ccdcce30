// Measurement aids for the 2-bit matvec: the issue rate of the instructions its decode is made
// of, and the decode loop by itself.  Included by qtip_probe.hip; the decode steps
// (matvec_accumulate, the table builders) come from the product's own device header, so the
// probe times the code the kernel runs.  Nothing here is part of libqtip_hip.so.
//
// issue_probe_kernel<KIND>: one workgroup of 16 waves per CU (4 waves per SIMD, as in the
// matvec); every wave executes `iters` x 88 instructions of one kind on 8 independent registers,
// so launch time / (iters * 88 * 4) is the time one wave-instruction occupies a SIMD.
// loop_probe_kernel<MODE>: the same workgroup decodes `iters` synthetic wave-loads per wave from
// registers (no global memory in the loop) against the real 128 KiB table in LDS; launch time /
// (iters * 4) is the time of one wave-load on a SIMD.  MODE 0 runs matvec_accumulate as the
// kernel does, MODE 1 only its vector-ALU part (extraction, hash, mask, address).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../qtip_amd/csrc/qtip_device.h"

namespace {

enum ProbeKind {
  kProbeAnd = 0,       // v_and_b32 (VOP2, register operands)
  kProbeAddU32,        // v_add_u32
  kProbeLshrImm,       // v_lshrrev_b32 by a constant
  kProbeLshlImm,       // v_lshlrev_b32 by a constant
  kProbePkMad,         // v_pk_mad_u16 (the hash)
  kProbeMadU32U16,     // v_mad_u32_u16 with op_sel (the table address)
  kProbePerm,          // v_perm_b32
  kProbePkLshr,        // v_pk_lshrrev_b16
  kProbeMovDpp,        // v_mov_b32_dpp row_ror:15
  kProbeDot2c,         // v_dot2c_f32_f16
  kProbeDsRead,        // ds_read_b32, 64 different entries of the 32-replica table
  kProbeMfma,          // v_mfma_f32_16x16x32_f16, independent accumulators
  kProbeIssueKinds,
  kProbeLoop = 100,    // the decode loop of the 2-bit matvec
  kProbeLoopValu = 101 // its vector-ALU part alone
};
constexpr int kProbeOpsPerIter = 88;  // 11 rounds over 8 registers

template <int KIND>
__global__ __launch_bounds__(1024, 1) void issue_probe_kernel(int iters, const uint32_t* __restrict__ tlut,
                                                              uint32_t* __restrict__ sink) {
  using namespace qtip;
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  uint32_t v[8];
  const uint32_t w = threadIdx.x * 3u + 1u;
  const int lane = threadIdx.x & 63;
  if constexpr (KIND == kProbeDsRead) {
    build_lut128(lut, tlut, threadIdx.x, 1024);
    __syncthreads();
    // fixed addresses: a different entry per lane and register, the lane's own replica
    for (int i = 0; i < 8; ++i)
      v[i] = lds_address(lut) + (((threadIdx.x * 2654435761u + i * 40503u) >> 7) & 1023u) * 128u + ((lane & 31) << 2);
  } else {
    for (int i = 0; i < 8; ++i) v[i] = threadIdx.x * 7u + i;
  }
  typedef _Float16 half8 __attribute__((ext_vector_type(8)));
  typedef float float4v __attribute__((ext_vector_type(4)));
  float4v acc[8];
  half8 ha, hb;
  if constexpr (KIND == kProbeMfma) {
    for (int i = 0; i < 8; ++i) acc[i] = float4v{0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < 8; ++i) {
      ha[i] = (_Float16)(float)((threadIdx.x + i) & 3);
      hb[i] = (_Float16)(float)((threadIdx.x * 5 + i) & 3);
    }
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < kProbeOpsPerIter / 8; ++r) {
      if constexpr (KIND == kProbeDsRead) {
        uint32_t t0, t1, t2, t3, t4, t5, t6, t7;
        asm volatile(
            "ds_read_b32 %0, %8\n ds_read_b32 %1, %9\n ds_read_b32 %2, %10\n ds_read_b32 %3, %11\n"
            "ds_read_b32 %4, %12\n ds_read_b32 %5, %13\n ds_read_b32 %6, %14\n ds_read_b32 %7, %15\n"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3), "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
            : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
      } else if constexpr (KIND == kProbeMfma) {
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ha, hb, acc[n], 0, 0, 0);
      } else {
#pragma unroll
        for (int n = 0; n < 8; ++n) {
          if constexpr (KIND == kProbeAnd) asm volatile("v_and_b32 %0, %1, %0" : "+v"(v[n]) : "v"(w));
          else if constexpr (KIND == kProbeAddU32) asm volatile("v_add_u32 %0, %1, %0" : "+v"(v[n]) : "v"(w));
          else if constexpr (KIND == kProbeLshrImm) asm volatile("v_lshrrev_b32 %0, 6, %0" : "+v"(v[n]));
          else if constexpr (KIND == kProbeLshlImm) asm volatile("v_lshlrev_b32 %0, 1, %0" : "+v"(v[n]));
          else if constexpr (KIND == kProbePkMad) asm volatile("v_pk_mad_u16 %0, %0, %0, %0" : "+v"(v[n]));
          else if constexpr (KIND == kProbeMadU32U16)
            asm volatile("v_mad_u32_u16 %0, %0, 2, %1 op_sel:[1,0,0,0]" : "+v"(v[n]) : "v"(w));
          else if constexpr (KIND == kProbePerm) asm volatile("v_perm_b32 %0, %0, %1, %1" : "+v"(v[n]) : "v"(w));
          else if constexpr (KIND == kProbePkLshr)
            asm volatile("v_pk_lshrrev_b16 %0, 4, %0 op_sel_hi:[0,1]" : "+v"(v[n]));
          else if constexpr (KIND == kProbeMovDpp)
            asm volatile("v_mov_b32_dpp %0, %1 row_ror:15 row_mask:0xf bank_mask:0xf" : "+v"(v[n]) : "v"(w));
          else if constexpr (KIND == kProbeDot2c) asm volatile("v_dot2c_f32_f16 %0, %1, %1" : "+v"(v[n]) : "v"(w));
        }
      }
    }
  }
  uint32_t s = 0;
  for (int i = 0; i < 8; ++i) s += v[i];
  if constexpr (KIND == kProbeMfma)
    for (int i = 0; i < 8; ++i) s += __builtin_bit_cast(uint32_t, acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3]);
  sink[(size_t)blockIdx.x * 1024 + threadIdx.x] = s;
}

template <int MODE>
__global__ __launch_bounds__(1024, 1) void loop_probe_kernel(int iters, const uint32_t* __restrict__ tlut,
                                                             uint32_t* __restrict__ sink) {
  using namespace qtip;
  constexpr int K = 2;
  extern __shared__ __align__(16) uint8_t smem[];
  uint32_t* lut = reinterpret_cast<uint32_t*>(smem);
  build_lut128(lut, tlut, threadIdx.x, 1024);
  uint8_t* xs = smem + kLut128Bytes;  // 16 KiB of activations
  for (int i = threadIdx.x; i < 4096; i += 1024) reinterpret_cast<uint32_t*>(xs)[i] = 0x3C003C00u + (i & 255);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t slot4 = lds_address(lut) + ((uint32_t)(lane & 31) << 2);
  const uint32_t xa0 = lds_address(xs) + (lane >> 4) * 64 + (lane & 1) * 8 + wave * 256;
  LaneData<K> ld;
  for (int i = 0; i < 2 * K; ++i) ld.d[i] = threadIdx.x * 2654435761u + i * 40503u;
  float4_t acc[4];
  for (int i = 0; i < 4; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
  uint32_t fold = 0;
  typedef __attribute__((address_space(3))) const u32x2 lds_u32x2_t;
  for (int it = 0; it < iters; ++it) {
    // fresh stream words every item: one full-rate multiply-add per register stands in for the load
#pragma unroll
    for (int i = 0; i < 2 * K; ++i) ld.d[i] = ld.d[i] * 3u + 0x9E3779B9u;
    if constexpr (MODE == 0) {
      u32x2 xv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) xv[q] = *(lds_u32x2_t*)(uintptr_t)(xa0 + 16u * q);
      matvec_accumulate<K>(ld, xv, slot4, acc);
    } else {
      uint32_t P[16];
      packed_states<K>(ld, P);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const uint32_t q = pk_hash(P[i]) & 0xFFC0FFC0u;
        const uint32_t a0 = lut128_addr_lo(q, slot4), a1 = lut128_addr_hi(q, slot4);
        asm volatile("" ::"v"(a0), "v"(a1));
      }
    }
  }
  for (int i = 0; i < 4; ++i) fold += __builtin_bit_cast(uint32_t, acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3]);
  sink[(size_t)blockIdx.x * 1024 + threadIdx.x] = fold + ld.d[0];
}

constexpr size_t kProbeLds = qtip::kLut128Bytes + 16384;

}  // namespace
