/* CPU oracle in plain C for the QTIP decode / decompress-matvec path.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py as the checker.  Nothing in qtip_amd/ links or
 * loads it.
 *
 * Restates, one state at a time, what a lane of the reference CUDA kernel
 * computes (qtip-kernels/src/inference.cu:94-166 load + neighbour fix-up,
 * :340-359 window shift, hash, table lookup and sign flip), with the packed
 * layout of lib/algo/finetune.py:196-201:
 *   bytes [m/32][k/32][lane 32][kh 2][mh 2][K], each K-byte chunk little-endian
 *   = big-endian integer of 8K stream bits; window = chunk || top 16 bits of
 *   lane+1's chunk (mod 32); state j = 16 bits starting 2K*j bits from the top;
 *   p = s*(s+1); index (p>>6)&511; element 0 negated if bit 15 of p is set;
 *   lane l, state j -> row l/4 + 8*(j%2), columns 2*(l%4) + 8*(j/2) + {0,1}.
 * Pinned by tests/test_oracle.py against the numpy restatements of the other
 * two descriptions of the layout in the reference and its known-answer tests.
 */
#include <stdint.h>
#include <string.h>

static double half_bits_to_double(uint16_t h) {
  const int sign = h >> 15, exp = (h >> 10) & 31, man = h & 1023;
  double v;
  if (exp == 0) {
    v = (double)man * 5.9604644775390625e-08; /* 2^-24 */
  } else if (exp == 31) {
    v = man ? (0.0 / 0.0) : (1.0 / 0.0);
  } else {
    uint64_t bits = ((uint64_t)(exp - 15 + 1023) << 52) | ((uint64_t)man << 42);
    memcpy(&v, &bits, 8);
  }
  return sign ? -v : v;
}

static inline uint32_t chunk_at(const uint8_t* blk, int lane, int kh, int mh, int K) {
  const uint8_t* p = blk + ((lane * 2 + kh) * 2 + mh) * K;
  uint32_t v = 0;
  for (int b = 0; b < K; ++b) v |= (uint32_t)p[b] << (8 * b);
  return v;
}

/* state j of (lane, kh, mh) of the 2x2 tile block at blk */
static inline uint32_t state_at(const uint8_t* blk, int lane, int kh, int mh, int j, int K) {
  const uint64_t own = chunk_at(blk, lane, kh, mh, K);
  const uint64_t nxt = chunk_at(blk, (lane + 1) & 31, kh, mh, K) >> (8 * K - 16);
  const uint64_t win = (own << 16) | nxt;
  return (uint32_t)((win >> (8 * K - 2 * K * j)) & 0xFFFF);
}

static inline void lookup(const uint16_t* tlut, uint32_t s, uint16_t w[2]) {
  const uint32_t p = s * (s + 1);
  const uint32_t q = (p >> 6) & 511;
  w[0] = tlut[2 * q] ^ (uint16_t)(p & 0x8000);
  w[1] = tlut[2 * q + 1];
}

/* out[m][k] fp16 bit patterns */
int qtip_oracle_decode(const uint8_t* packed, const uint16_t* tlut, int m, int k, int K,
                       uint16_t* out) {
  if (m % 32 || k % 32 || K < 2 || K > 4) return -1;
  /* 32-row blocks are independent of each other (OpenMP only spreads them over the host cores) */
#pragma omp parallel for schedule(static)
  for (int i0 = 0; i0 < m / 32; ++i0)
    for (int i1 = 0; i1 < k / 32; ++i1) {
      const uint8_t* blk = packed + ((size_t)i0 * (k / 32) + i1) * 128 * K;
      for (int lane = 0; lane < 32; ++lane)
        for (int kh = 0; kh < 2; ++kh)
          for (int mh = 0; mh < 2; ++mh)
            for (int j = 0; j < 4; ++j) {
              uint16_t w[2];
              lookup(tlut, state_at(blk, lane, kh, mh, j, K), w);
              const size_t row = (size_t)32 * i0 + 16 * mh + lane / 4 + 8 * (j % 2);
              const size_t col = (size_t)32 * i1 + 16 * kh + 2 * (lane % 4) + 8 * (j / 2);
              out[row * k + col] = w[0];
              out[row * k + col + 1] = w[1];
            }
    }
  return 0;
}

/* out[m] = decode(packed) . x in double (products of two fp16 values are exact) */
int qtip_oracle_matvec(const uint8_t* packed, const uint16_t* tlut, const uint16_t* x, int m, int k,
                       int K, double* out) {
  if (m % 32 || k % 32 || K < 2 || K > 4) return -1;
  for (int i = 0; i < m; ++i) out[i] = 0.0;
  /* a row block owns its 32 outputs; the sum over a row keeps its serial order */
#pragma omp parallel for schedule(static)
  for (int i0 = 0; i0 < m / 32; ++i0)
    for (int i1 = 0; i1 < k / 32; ++i1) {
      const uint8_t* blk = packed + ((size_t)i0 * (k / 32) + i1) * 128 * K;
      for (int lane = 0; lane < 32; ++lane)
        for (int kh = 0; kh < 2; ++kh)
          for (int mh = 0; mh < 2; ++mh)
            for (int j = 0; j < 4; ++j) {
              uint16_t w[2];
              lookup(tlut, state_at(blk, lane, kh, mh, j, K), w);
              const size_t row = (size_t)32 * i0 + 16 * mh + lane / 4 + 8 * (j % 2);
              const size_t col = (size_t)32 * i1 + 16 * kh + 2 * (lane % 4) + 8 * (j / 2);
              out[row] += half_bits_to_double(w[0]) * half_bits_to_double(x[col]) +
                          half_bits_to_double(w[1]) * half_bits_to_double(x[col + 1]);
            }
    }
  return 0;
}
