// libqtip_probe.so: the measurement aids declared in qtip_probe.h (stream-read ceiling,
// instruction issue rates, the 2-bit decode loop without memory).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qtip_probe.h"
#include "qtip_probe_kernels.h"

namespace {

// Read `n16` 16-byte words once with the loads of the matvec's stream (non-temporal dwordx4,
// one per lane, persistent workgroups) and fold them into one word per wave.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(1024) void stream_read_probe_kernel(uint32_t* __restrict__ sink,
                                                                 const probe_u32x4* __restrict__ src, size_t n16) {
  const size_t nthreads = (size_t)gridDim.x * blockDim.x;
  uint32_t acc = 0;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * nthreads < n16; i += 4 * nthreads) {
    const probe_u32x4 a = __builtin_nontemporal_load(src + i);
    const probe_u32x4 b = __builtin_nontemporal_load(src + i + nthreads);
    const probe_u32x4 c = __builtin_nontemporal_load(src + i + 2 * nthreads);
    const probe_u32x4 d = __builtin_nontemporal_load(src + i + 3 * nthreads);
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < n16; i += nthreads) {
    const probe_u32x4 a = __builtin_nontemporal_load(src + i);
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc ^= __shfl_xor(acc, o);
  if ((threadIdx.x & 63) == 0) sink[(size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)] = acc;
}

int cu_count(int* cus) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || *cus < 1)
    return (int)hipErrorInvalidDevice;
  return 0;
}

template <typename F>
hipError_t allow_lds(F* fn, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                             (int)bytes);
}

}  // namespace

extern "C" {

int qtip_probe_stream_read(void* sink_u32, const void* src, size_t bytes, void* stream) {
  if (!sink_u32 || !src || bytes < 16 || (reinterpret_cast<uintptr_t>(src) & 15u)) return QTIP_PROBE_E_ARG;
  int cus = 0;
  if (const int rc = cu_count(&cus)) return rc;
  stream_read_probe_kernel<<<cus, 1024, 0, (hipStream_t)stream>>>((uint32_t*)sink_u32, (const probe_u32x4*)src,
                                                                  bytes / 16);
  return (int)hipGetLastError();
}

int qtip_probe_issue(int kind, int iters, const void* tlut, void* sink_u32, void* stream) {
  if (!tlut || !sink_u32 || iters < 1 || iters > (1 << 20)) return QTIP_PROBE_E_ARG;
  int cus = 0;
  if (const int rc = cu_count(&cus)) return rc;
  // the kernels with the 128 KiB table need the LDS opt-in (a host-side attribute, no device work)
  hipError_t e = allow_lds(issue_probe_kernel<kProbeDsRead>, kProbeLds);
  if (e == hipSuccess) e = allow_lds(loop_probe_kernel<0>, kProbeLds);
  if (e == hipSuccess) e = allow_lds(loop_probe_kernel<1>, kProbeLds);
  if (e != hipSuccess) return (int)e;
  hipStream_t st = (hipStream_t)stream;
  const uint32_t* tl = (const uint32_t*)tlut;
  uint32_t* sink = (uint32_t*)sink_u32;
  switch (kind) {
#define QTIP_PROBE(KIND, LDS) \
  case KIND: issue_probe_kernel<KIND><<<cus, 1024, LDS, st>>>(iters, tl, sink); break;
    QTIP_PROBE(kProbeAnd, 0)
    QTIP_PROBE(kProbeAddU32, 0)
    QTIP_PROBE(kProbeLshrImm, 0)
    QTIP_PROBE(kProbeLshlImm, 0)
    QTIP_PROBE(kProbePkMad, 0)
    QTIP_PROBE(kProbeMadU32U16, 0)
    QTIP_PROBE(kProbePerm, 0)
    QTIP_PROBE(kProbePkLshr, 0)
    QTIP_PROBE(kProbeMovDpp, 0)
    QTIP_PROBE(kProbeDot2c, 0)
    QTIP_PROBE(kProbeDsRead, kProbeLds)
    QTIP_PROBE(kProbeMfma, 0)
#undef QTIP_PROBE
    case kProbeLoop: loop_probe_kernel<0><<<cus, 1024, kProbeLds, st>>>(iters, tl, sink); break;
    case kProbeLoopValu: loop_probe_kernel<1><<<cus, 1024, kProbeLds, st>>>(iters, tl, sink); break;
    default: return QTIP_PROBE_E_ARG;
  }
  return (int)hipGetLastError();
}

}  // extern "C"
