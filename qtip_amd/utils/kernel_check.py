"""Which codebook configurations the HIP kernels cover.

Same gate as the reference (lib/utils/kernel_check.py:1-14): HYB code only
(quantlut_sym), L=16, V=2, 2..4 bits, 9-bit tunable LUT, 16x16 tiles.
"""


def has_kernel(decode_mode, L, K, V, tlut_bits, td_x, td_y):
    return (decode_mode == 'quantlut_sym' and L == 16 and V == 2 and 2 <= K <= 4 and tlut_bits == 9
            and td_x == 16 and td_y == 16)
