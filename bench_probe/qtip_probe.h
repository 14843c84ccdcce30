/* C ABI of libqtip_probe.so: measurement aids that bench.py prints beside the kernels' own
 * figures.  Not part of the library that replaces the reference (libqtip_hip.so exports none of
 * this); no counterpart in the reference.  Return 0 or a negative QTIP_PROBE_E_* / positive
 * hipError_t code.  Every call runs on the given stream of the current device and allocates
 * nothing. */
#ifndef QTIP_PROBE_H
#define QTIP_PROBE_H
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QTIP_PROBE_E_ARG (-1)

/* Reads `bytes` of device memory once with the matvec's kind of loads (persistent workgroups,
 * one non-temporal 16-byte load per lane) and writes one folded word per wave to sink_u32
 * (16 * #CUs words).  Its duration is the stream-read ceiling of the box. */
int qtip_probe_stream_read(void* sink_u32, const void* src, size_t bytes, void* stream);

/* What the instructions of the 2-bit decode cost on this box.  One workgroup of 16 waves per CU
 * (4 waves per SIMD, as in the matvec).
 * kind 0..11: every wave executes iters * QTIP_PROBE_OPS_PER_ITER instructions of one kind on
 * eight independent registers - 0 v_and_b32, 1 v_add_u32, 2 v_lshrrev_b32 by a constant,
 * 3 v_lshlrev_b32 by a constant, 4 v_pk_mad_u16, 5 v_mad_u32_u16 with op_sel, 6 v_perm_b32,
 * 7 v_pk_lshrrev_b16, 8 v_mov_b32_dpp row_ror, 9 v_dot2c_f32_f16, 10 ds_read_b32 of 64
 * different entries of the 32-replica table, 11 v_mfma_f32_16x16x32_f16 - so the launch's
 * duration / (iters * QTIP_PROBE_OPS_PER_ITER * 4) is the time one wave-instruction occupies a
 * SIMD.  kind 100: every wave decodes iters synthetic 2-bit wave-loads from registers with the
 * matvec's own loop body against the real table in LDS (no global memory in the loop); kind 101:
 * the vector-ALU part of that body alone; duration / (iters * 4) is the time of one wave-load on
 * a SIMD.  tlut: 512 x (fp16, fp16) as for the matvec; sink_u32 receives 1024 * #CUs words. */
#define QTIP_PROBE_OPS_PER_ITER 88
int qtip_probe_issue(int kind, int iters, const void* tlut, void* sink_u32, void* stream);

#ifdef __cplusplus
}
#endif
#endif
