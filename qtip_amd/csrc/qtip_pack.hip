// Packing tools of libqtip_hip.so: conversions between the natural (per-tile bitstream) packing,
// the kernel packing and explicit trellis states, and a dense decode of the natural packing for
// every decode mode (the caller supplies the expanded 2^16-entry table).
// All of it is integer / byte work, bound by HBM traffic; one thread per output element group.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/qtip_hip.h"

namespace {

constexpr int kBlock = 256;

// ---- natural <-> kernel packing ------------------------------------------------------------
// Natural: tile t = (tile row)*(k/16) + (tile column) owns 32*K bytes; its big-endian bitstream
// is stored as little-endian uint16 words, so stream byte b sits at stored byte b ^ 1.
// Kernel: bytes [m/32][k/32][lane 32][kh 2][mh 2][K], where (lane, c) is stream byte
// lane*K + (K-1-c) of tile (2*i0 + mh, 2*i1 + kh).
// A thread moves the 4*K bytes of one (i0, i1, lane): contiguous on the kernel side.
template <int K, bool TO_KERNEL>
__global__ __launch_bounds__(kBlock) void repack_kernel(uint8_t* __restrict__ out,
                                                        const uint8_t* __restrict__ in, int m, int k) {
  const long total = (long)(m >> 5) * (k >> 5) * 32;
  const long idx = (long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int lane = (int)(idx & 31);
  const long blk = idx >> 5;
  const int nb1 = k >> 5;
  const int i0 = (int)(blk / nb1), i1 = (int)(blk - (long)i0 * nb1);
  const long kbase = idx * 4 * K;
#pragma unroll
  for (int kh = 0; kh < 2; ++kh)
#pragma unroll
    for (int mh = 0; mh < 2; ++mh) {
      const long tile = (long)(2 * i0 + mh) * (k >> 4) + (2 * i1 + kh);
#pragma unroll
      for (int c = 0; c < K; ++c) {
        const int b = lane * K + (K - 1 - c);
        const long nat = tile * 32 * K + (b ^ 1);
        const long ker = kbase + (kh * 2 + mh) * K + c;
        if (TO_KERNEL) out[ker] = in[nat];
        else out[nat] = in[ker];
      }
    }
}

// 16-bit big-endian window at bit offset pos of a tile's circular stream of nw uint16 words
__device__ __forceinline__ uint32_t window16(const uint16_t* __restrict__ tile, int nw, int pos) {
  const int w = pos >> 4, off = pos & 15;
  const uint32_t cur = tile[w];
  const uint32_t nxt = tile[w + 1 == nw ? 0 : w + 1];
  return (((cur << 16) | nxt) >> (16 - off)) & 0xFFFFu;
}

// ---- natural packing -> states ---------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void unpack_states_kernel(int32_t* __restrict__ states,
                                                               const uint16_t* __restrict__ packed,
                                                               long ntiles, int ns, int nw, int kv) {
  const long idx = (long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= ntiles * ns) return;
  const long t = idx / ns;
  const int i = (int)(idx - t * ns);
  states[idx] = (int32_t)window16(packed + t * nw, nw, i * kv);
}

// ---- states -> natural packing ---------------------------------------------------------------
// Stream bit b < 16 is bit (15 - b) of state 0; bit b >= 16 is one of the kv fresh (low) bits of
// state 1 + (b - 16) / kv.  The bits past ns*kv repeat the head of a tail-biting walk and are
// not stored.  A thread assembles one uint16 word; `violations` counts state pairs that do not
// overlap by 16 - kv bits.
__global__ __launch_bounds__(kBlock) void pack_states_kernel(uint16_t* __restrict__ packed,
                                                             const int32_t* __restrict__ states,
                                                             long ntiles, int ns, int nw, int kv,
                                                             int* __restrict__ violations) {
  const long idx = (long)blockIdx.x * kBlock + threadIdx.x;
  if (idx < ntiles * ns) {
    const long t = idx / ns;
    const int i = (int)(idx - t * ns);
    if (i > 0) {
      const uint32_t prev = (uint32_t)states[idx - 1], cur = (uint32_t)states[idx];
      if ((prev & ((1u << (16 - kv)) - 1u)) != ((cur & 0xFFFFu) >> kv)) atomicAdd(violations, 1);
    }
  }
  if (idx >= ntiles * nw) return;
  const long t = idx / nw;
  const int w = (int)(idx - t * nw);
  const int32_t* st = states + t * ns;
  uint32_t word = 0;
#pragma unroll 4
  for (int e = 0; e < 16; ++e) {
    const int b = 16 * w + e;
    uint32_t bit;
    if (b < 16) {
      bit = ((uint32_t)st[0] >> (15 - b)) & 1u;
    } else {
      const int j = 1 + (b - 16) / kv, r = (b - 16) % kv;
      bit = ((uint32_t)st[j] >> (kv - 1 - r)) & 1u;
    }
    word = (word << 1) | bit;
  }
  packed[idx] = (uint16_t)word;
}

// ---- natural packing -> dense matrix -----------------------------------------------------------
// out[row][col .. col+V) = lut[v][state] for state i of tile (ti, tj): sequence position i*V + v is
// the row-major element of the td_x x td_y tile.  T = float (fp32 table) or uint16_t (fp16 bits).
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void decode_natural_kernel(T* __restrict__ out,
                                                                const uint16_t* __restrict__ packed,
                                                                const T* __restrict__ lut, int m, int n,
                                                                int td_x, int td_y, int ns, int nw, int kv) {
  const long ntiles = (long)(m / td_x) * (n / td_y);
  const long idx = (long)blockIdx.x * kBlock + threadIdx.x;
  if (idx >= ntiles * ns) return;
  const long t = idx / ns;
  const int i = (int)(idx - t * ns);
  const uint32_t s = window16(packed + t * nw, nw, i * kv);
  const int tn = n / td_y;
  const long ti = t / tn, tj = t - ti * tn;
  const int p = i * V;
  const long row = ti * td_x + p / td_y;
  const long col = tj * td_y + p % td_y;
#pragma unroll
  for (int v = 0; v < V; ++v) out[row * n + col + v] = lut[(size_t)v * 65536 + s];
}

bool aligned(const void* p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int grid_for(long items) { return (int)((items + kBlock - 1) / kBlock); }

// shared checks of the natural-packing entry points
int check_natural(long ntiles, int T, int K, int V) {
  if (ntiles <= 0 || T <= 0 || K < 1 || K > 8 || (V != 1 && V != 2)) return QTIP_E_SHAPE;
  if (K * V > 16 || T % V || (T * K) % 16) return QTIP_E_SHAPE;
  if (ntiles * (long)(T / V) >= (1L << 38)) return QTIP_E_SHAPE;  // grid size stays below 2^31
  return QTIP_OK;
}

}  // namespace

extern "C" {

int qtip_repack(void* out, const void* in, int m, int k, int bits, int to_kernel, void* stream) {
  if (!out || !in) return QTIP_E_NULL;
  if (out == in) return QTIP_E_SHAPE;  // not an in-place permutation
  if (bits < 2 || bits > 4 || m <= 0 || k <= 0 || (m & 31) || (k & 31)) return QTIP_E_SHAPE;
  const long items = (long)(m >> 5) * (k >> 5) * 32;
  const int grid = grid_for(items);
  hipStream_t st = (hipStream_t)stream;
  auto* o = (uint8_t*)out;
  auto* i = (const uint8_t*)in;
#define QTIP_REPACK(KB)                                                        \
  if (to_kernel) repack_kernel<KB, true><<<grid, kBlock, 0, st>>>(o, i, m, k); \
  else repack_kernel<KB, false><<<grid, kBlock, 0, st>>>(o, i, m, k);
  switch (bits) {
    case 2: QTIP_REPACK(2) break;
    case 3: QTIP_REPACK(3) break;
    default: QTIP_REPACK(4) break;
  }
#undef QTIP_REPACK
  return (int)hipGetLastError();
}

int qtip_unpack_trellis(int32_t* states, const void* packed, long ntiles, int T, int K, int V,
                        void* stream) {
  if (!states || !packed) return QTIP_E_NULL;
  int rc = check_natural(ntiles, T, K, V);
  if (rc) return rc;
  if (!aligned(states, 4) || !aligned(packed, 2)) return QTIP_E_ALIGN;
  const int ns = T / V, nw = T * K / 16;
  unpack_states_kernel<<<grid_for(ntiles * ns), kBlock, 0, (hipStream_t)stream>>>(
      states, (const uint16_t*)packed, ntiles, ns, nw, K * V);
  return (int)hipGetLastError();
}

int qtip_pack_trellis(void* packed, const int32_t* states, long ntiles, int T, int K, int V,
                      int* violations, void* stream) {
  if (!states || !packed || !violations) return QTIP_E_NULL;
  int rc = check_natural(ntiles, T, K, V);
  if (rc) return rc;
  if (!aligned(states, 4) || !aligned(packed, 2) || !aligned(violations, 4)) return QTIP_E_ALIGN;
  const int ns = T / V, nw = T * K / 16;
  const long items = ntiles * (ns > nw ? ns : nw);
  pack_states_kernel<<<grid_for(items), kBlock, 0, (hipStream_t)stream>>>(
      (uint16_t*)packed, states, ntiles, ns, nw, K * V, violations);
  return (int)hipGetLastError();
}

int qtip_decode_natural(void* out, const void* packed, const void* lut, int lut_dtype, int m, int n,
                        int td_x, int td_y, int K, int V, void* stream) {
  if (!out || !packed || !lut) return QTIP_E_NULL;
  if (m <= 0 || n <= 0 || td_x <= 0 || td_y <= 0 || m % td_x || n % td_y) return QTIP_E_SHAPE;
  const int T = td_x * td_y;
  const long ntiles = (long)(m / td_x) * (n / td_y);
  int rc = check_natural(ntiles, T, K, V);
  if (rc) return rc;
  if (td_y % V) return QTIP_E_SHAPE;
  if (lut_dtype != QTIP_F16 && lut_dtype != QTIP_F32) return QTIP_E_DTYPE;
  if (!aligned(out, 4) || !aligned(packed, 2) || !aligned(lut, 4)) return QTIP_E_ALIGN;
  const int ns = T / V, nw = T * K / 16, kv = K * V;
  const int grid = grid_for(ntiles * ns);
  hipStream_t st = (hipStream_t)stream;
  auto* pk = (const uint16_t*)packed;
#define QTIP_DN(TY, VV) \
  decode_natural_kernel<TY, VV><<<grid, kBlock, 0, st>>>((TY*)out, pk, (const TY*)lut, m, n, td_x, td_y, ns, nw, kv)
  if (lut_dtype == QTIP_F16) {
    if (V == 1) QTIP_DN(uint16_t, 1); else QTIP_DN(uint16_t, 2);
  } else {
    if (V == 1) QTIP_DN(float, 1); else QTIP_DN(float, 2);
  }
#undef QTIP_DN
  return (int)hipGetLastError();
}


}  // extern "C"
