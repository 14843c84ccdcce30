/* C ABI of libqtip_hip.so: MI355X (gfx950) kernels for QTIP's quantized-linear
 * inference path (HYB code: L=16, 9-bit tunable LUT, V=2, 16x16 trellis tiles,
 * 2/3/4 bits per weight).
 *
 * Conventions for every launcher
 *   - all pointers are DEVICE pointers on the current HIP device, plain C types;
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream);
 *   - asynchronous: the call enqueues work and returns; it never synchronises,
 *     allocates or frees, so it may be recorded into a HIP graph.  The first
 *     launcher call on a device runs that device's one-time set-up
 *     (qtip_init: CU count, LDS opt-in per kernel) if qtip_init has not been
 *     called there - unless its stream is being captured: then nothing is
 *     recorded and the call returns QTIP_E_NOT_INIT, so a caller whose first
 *     call would be inside a stream capture calls qtip_init() beforehand;
 *   - returns 0 on success, a negative QTIP_E_* code for rejected arguments
 *     (nothing was launched), or a positive hipError_t from the launch.  It
 *     never terminates the process (the reference's launcher exits on error,
 *     qtip-kernels/src/inference.h:10-18).
 *
 * Packed layout (`packed`): the reference's kernel packing, m*k*bits/8 bytes,
 * bytes indexed [m/32][k/32][lane 32][kh 2][mh 2][bits] (produced by
 * lib/algo/finetune.py:196-201, consumed by qtip-kernels/src/inference.cu:94-166).
 * `tlut` is the raw tunable table, 512 x (fp16, fp16), 2 KiB.
 */
#ifndef QTIP_HIP_H
#define QTIP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define QTIP_OK 0
#define QTIP_E_SHAPE (-1)     /* m % 32, k % 32, bits, batch or n out of range */
#define QTIP_E_NULL (-2)      /* a required pointer is NULL */
#define QTIP_E_ALIGN (-3)     /* a pointer is not 16-byte aligned */
#define QTIP_E_WORKSPACE (-4) /* workspace smaller than qtip_matvec_workspace_bytes */
#define QTIP_E_DTYPE (-5)     /* unknown dtype code */
#define QTIP_E_SCRATCH (-6)   /* partial sums larger than the library's static scratch */
#define QTIP_E_NOT_INIT (-7)  /* first call on this device came inside a stream capture */

#define QTIP_F16 0
#define QTIP_F32 1

/* Library ABI version (bumped when a signature changes). */
int qtip_abi_version(void);

/* One-time set-up for the CURRENT device: reads the CU count, opts every kernel into its LDS
 * size and looks up the device's copy of the library's static scratch.  Allocates nothing and
 * does not synchronise.  Idempotent and thread-safe; returns 0 or a hipError_t.  Every launcher
 * runs it on first use of a device, so calling it is only required before a stream capture
 * whose first recorded call would otherwise be the library's first call on that device.
 * No counterpart in the reference (its templates need no run-time set-up). */
int qtip_init(void);

/* Text for a return code of any launcher below (static storage). */
const char* qtip_error_string(int code);

/* Dense decode of the kernel-packed stream: out[m][k] fp16, row-major.
 * Replaces decode_compressed(L,S,R,V,m,k,compressed,expanded_lut)
 * (lib/utils/kernel_decompress.py:4-55) and BitshiftLinear.get_hatW_kernel
 * (lib/codebook/bitshift.py:383-387); takes the raw 512x2 table and applies
 * the quantlut_sym expansion (lib/codebook/bitshift.py:72-80) on the fly.
 * Bit-exact with the reference decode. */
int qtip_decode(void* out_f16, const void* packed, const void* tlut,
                int m, int k, int bits, void* stream);

/* Number of k splits S (>= 1) recommended for qtip_decompress_matvec_parts on this shape and
 * device: small m cannot fill 256 CUs with 32-row blocks alone, so the k dimension is cut into
 * S ranges whose partial sums the consumer adds in a fixed order.  Returns 0 for an
 * unsupported shape. */
int qtip_matvec_split(int m, int k, int bits);

/* Bytes of scratch qtip_decompress_matvec wants for this shape: S'*m floats when it splits k,
 * else 0 (S' is chosen with the cost of the extra summing launch included, so it is 1 for most
 * shapes).  The scratch needs no initialisation.  Calls that share one scratch buffer must not
 * overlap in time. */
size_t qtip_matvec_workspace_bytes(int m, int k, int bits);

/* bs=1 decompress + matvec: out[m] (fp32) = hatW[m][k] . x[k] (fp16), fp32
 * accumulate, deterministic summation order, `out` fully overwritten.
 * Replaces decompress_matvec_ptr<16,9,R,1,M,1,K>(float*, const uint32_t*,
 * const half2*, const half2*, CUstream_st*) (qtip-kernels/src/inference.h:48-55,
 * inference.cu:432-471) and the 64 pybind entry points
 * decompress_matvec_16_9_{R}_1_{M}_1_{K} (qtip-kernels/src/wrapper.cpp:489-564).
 * Shapes are run-time arguments: m % 32 == 0, k % 32 == 0, bits in {2,3,4}.
 * With a workspace and S > 1 this is two launches (partial sums, then their
 * sum); `workspace` may be NULL, then k is never split (one launch, less
 * parallelism on small m). */
int qtip_decompress_matvec(float* out, const void* packed, const void* x_f16,
                           const void* tlut, int m, int k, int bits,
                           void* workspace, size_t workspace_bytes, void* stream);

/* qtip_decompress_matvec for callers that cannot allocate device memory and have no workspace
 * to pass (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  The split-k partial sums live in a 256 KiB array in the
 * library's own device image (one copy per GPU, held until the process ends), so the call
 * allocates nothing: no hipMalloc / hipFree, no workspace argument.
 *   nparts = 0: the library's choice of k split (the one qtip_decompress_matvec makes with a
 *               workspace, halved until its partial sums fit the array: never an error);
 *               1..16: that many k ranges.
 * Results are bit-identical to qtip_decompress_matvec with the same split.
 * Limit for a split the caller asks for: nparts * m <= 65536 floats, else QTIP_E_SCRATCH
 * (nothing launched; nparts = 1 never needs the scratch).  The partial sums are all written before they are read, so nothing has to
 * be cleared between calls; but every call on a GPU uses that GPU's one array: calls that
 * overlap in time on one GPU (different streams, or graphs replayed concurrently) race. */
int qtip_decompress_matvec_noalloc(float* out, const void* packed, const void* x_f16,
                                   const void* tlut, int m, int k, int bits, int nparts,
                                   void* stream);

/* Same kernel, but leaves the nparts partial vectors parts[nparts][m] for the
 * consumer to add (qtip_rht does so on load through its in_parts argument),
 * which saves the second launch inside BitshiftLinear.forward.
 * 1 <= nparts <= 16; normally nparts = qtip_matvec_split(m, k, bits). */
int qtip_decompress_matvec_parts(float* parts, const void* packed, const void* x_f16,
                                 const void* tlut, int m, int k, int bits, int nparts,
                                 void* stream);

/* qtip_decompress_matvec_parts with the input transform of the layer inside the kernel:
 *   x_t = fp16(scale * H_k (su * x_raw)),  parts = hatW . x_t
 * i.e. matmul_hadUt_cuda + the SU multiply + the fp16 cast of BitshiftLinear.forward
 * (lib/codebook/bitshift.py:428-441, lib/utils/matmul_had.py:92-119) and the matvec in one
 * launch.  k in {2048, 4096, 8192} (power-of-two transform, order 1); x_raw and su are
 * fp16[k], 16-byte aligned; scale is 1/sqrt(k)/32 in the forward pass.  Every workgroup
 * computes the whole transform while its first weight loads are in flight. */
int qtip_decompress_matvec_parts_rht(float* parts, const void* packed, const void* x_raw_f16,
                                     const void* su_f16, float scale, const void* tlut, int m, int k,
                                     int bits, int nparts, void* stream);

/* qtip_decompress_matvec_parts with the whole boundary between two linear layers of a decoder
 * in front of it (k in {2048, 4096, 8192}):
 *   x_new = residual + fp16(scale_out * post * H_k (prev_parts[0] + prev_parts[1] + ...))
 *   x_t   = fp16(scale_in * H_k (su * (norm_w * fp16(x_new * rsqrt(mean(x_new^2) + eps)))))
 *   parts = hatW . x_t,   x_out = x_new
 * i.e. the output transform of the previous QuantizedLinear (lib/codebook/bitshift.py:465-472) with
 * the residual addition (model/llama.py:964,979), the RMSNorm (model/llama.py:129-135) and this
 * layer's input transform (bitshift.py:428-441) and matvec in one launch: what qtip_rht_chain
 * followed by qtip_decompress_matvec_parts computes.  prev_parts: prev_nparts vectors of k fp32,
 * prev_part_stride floats apart; post fp32[k]; residual, norm_w, su fp16[k]; x_out fp16[k], not
 * the residual buffer (every workgroup reads residual, one writes x_out); all 16-byte aligned. */
int qtip_decompress_matvec_parts_chain(float* parts, const void* packed, const void* tlut, int m, int k,
                                       int bits, int nparts, const float* prev_parts, int prev_nparts,
                                       size_t prev_part_stride, const float* post, float scale_out,
                                       const void* residual_f16, const void* norm_w_f16, float eps,
                                       const void* su_f16, float scale_in, void* x_out_f16,
                                       void* stream);

/* qtip_decompress_matvec_parts_chain for up to three matrices that share their input and
 * differ in everything else - the separate q / k / v (or gate / up) projections of the published
 * checkpoints (model/llama.py:246-262 q_proj, k_proj, v_proj; :389-400 gate_proj, up_proj), each a
 * QuantizedLinear with its own trellis, table and sign vectors - in ONE launch: the workgroups
 * are shared out among the matrices in proportion to their rows.  packed / tlut / su_f16 / m are
 * HOST arrays of ngroups (1..3) device pointers / row counts; parts is [nparts][sum of m] fp32,
 * matrix g's rows following those of matrix g - 1; the boundary arguments are those of
 * qtip_decompress_matvec_parts_chain (one residual stream, one x_out). */
int qtip_decompress_matvec_group_chain(float* parts, int ngroups, const void* const* packed,
                                       const void* const* tlut, const void* const* su_f16, const int* m,
                                       int k, int bits, int nparts, const float* prev_parts,
                                       int prev_nparts, size_t prev_part_stride, const float* post_f32,
                                       float scale_out, const void* residual_f16, const void* norm_weight_f16,
                                       float eps, float scale_in, void* x_out_f16, void* stream);

/* The plain form of the grouped launch: matrix g multiplies its own fp16 input x_f16[g] (the
 * separate projections of a layer whose hidden size is not a power of two, where the input
 * transforms are launches of their own).  Same layout of `parts`; every k range of x must fit the
 * kernel's LDS staging area (k / nparts <= 14336). */
int qtip_decompress_matvec_group(float* parts, int ngroups, const void* const* packed,
                                 const void* const* x_f16, const void* const* tlut, const int* m, int k,
                                 int bits, int nparts, void* stream);

/* Bytes of scratch qtip_decompress_gemm wants for this shape (0 when it does not split k). */
size_t qtip_gemm_workspace_bytes(int m, int k, int bits, int batch);

/* Batched decompress + GEMM on the matrix cores:
 * out[batch][m] = x[batch][k] (fp16) . hatW[m][k]^T, fp32 accumulate.
 * If round_f16 != 0 every result is rounded to fp16 and widened again, which
 * is what the reference's fp16 GEMM output followed by .float() yields.
 * Replaces BitshiftLinearKernelAG.forward = decode_compressed + input.half() @ hatW.T
 * (lib/codebook/bitshift.py:476-489).  1 <= batch <= 65535.
 * Matrices with few rows are also cut along k; the fp32 partial results then pass through
 * `workspace` (qtip_gemm_workspace_bytes, no initialisation needed, 16-byte aligned) and one
 * more small launch adds them in a fixed order.  workspace may be NULL: k is then never split. */
int qtip_decompress_gemm(float* out, const void* packed, const void* x_f16,
                         const void* tlut, int m, int k, int bits, int batch,
                         int round_f16, void* workspace, size_t workspace_bytes, void* stream);

/* Randomised Hadamard transform of `rows` vectors of length n = order * p
 * (p a power of two, order 1 or a table order):
 *   out[r][:] = post[:] * scale * (H_order (x) H_p) (pre[:] * in[r][:])
 * with H_p the Sylvester (natural order) Walsh-Hadamard matrix.
 *   in_dtype/out_dtype  QTIP_F16 or QTIP_F32
 *   pre   fp16[n] or NULL (input sign vector SU)
 *   post  fp32[n] or NULL (output scale vector SV)
 *   had_bits  order*order sign bits, column-major: bit (j*order+i) of a
 *             little-endian uint32 array is set when H[i][j] == -1 (H already
 *             transposed by the caller for the "Ut" form); ignored (may be
 *             NULL) when order == 1
 *   in_parts  > 1: `in` holds in_parts arrays of rows*n elements that are
 *             summed on load (split-k partial sums); normally 1.
 * Replaces matmul_hadU_cuda / matmul_hadUt_cuda and the hadamard::hadamard
 * op (lib/utils/matmul_had.py:92-119; third-party fast_hadamard_transform
 * kernel + dense hadK matmul) together with the elementwise SU / SV / scale
 * steps of BitshiftLinear.forward (lib/codebook/bitshift.py:428-441,469-472). */
int qtip_rht(void* out, int out_dtype, const void* in, int in_dtype, int in_parts,
             int rows, int n, int order, const uint32_t* had_bits,
             const void* pre_f16, const float* post_f32, float scale, void* stream);

/* qtip_rht with one `post` vector per row (post_rows_f32 is [rows][n]): the output transforms of
 * several QuantizedLinear layers of the same size in one launch - the separate gate / up
 * projections of a decoder layer, whose raw matvec results lie side by side in one partial-sum
 * buffer ([in_parts][rows][n]) and whose outputs [gate | up] feed the SiLU * up transform. */
int qtip_rht_post_rows(void* out, int out_dtype, const void* in, int in_dtype, int in_parts, int rows, int n,
                       int order, const uint32_t* had_bits, const float* post_rows_f32, float scale,
                       void* stream);

/* The output transforms of the gate and up projections and the SiLU-gated product after them, in
 * one launch:  out = fp16(fp16(silu(gate)) * up)  (model/llama.py:399-400) with
 * [gate | up] = fp16(post * scale * (H_order (x) H_p)(sum over in_parts of in))
 * (lib/codebook/bitshift.py:465-472), bit-identical to qtip_rht / qtip_rht_post_rows followed by
 * the element-wise step of qtip_rht_fused's pre_mode 2.
 *   two_vectors == 0: one transformed vector of length n whose halves are gate and up (the fused
 *     up/gate projection of model/llama.py:382-390); order must be even; in fp32[in_parts][n],
 *     post fp32[n], out fp16[n / 2].
 *   two_vectors != 0: gate and up are vectors of length n with a transform each (separate
 *     projections); in fp32[in_parts][2][n], post fp32[2][n], out fp16[n].
 * n / order must be a power of two >= 8; n > 4096 is what it is meant for. */
int qtip_rht_silu_pair(void* out_f16, const float* in_f32, int in_parts, int two_vectors, int n, int order,
                       const uint32_t* had_bits, const float* post_f32, float scale, void* stream);

/* The input transforms of several QuantizedLinear layers that read the same vector, in one launch:
 * row r of out = fp16(scale * (H_order^T (x) H_p)(pre_rows[r] * rmsnorm(in))) with the RMSNorm of
 * qtip_rht_fused (model/llama.py:129-135) - q / k / v (or gate / up) of a decoder layer, each with
 * its own sign vector SU (lib/codebook/bitshift.py:428-441).  in fp16[n], pre_rows fp16[rows][n]. */
int qtip_rht_fused_pre_rows(void* out_f16, const void* in_f16, int rows, int n, int order,
                            const uint32_t* had_bits, const void* pre_rows_f16, float scale,
                            const void* norm_weight_f16, float eps, void* stream);

/* qtip_rht with the element-wise work of the layers around a QTIP linear folded in
 * (used by the end-to-end decode loop; each mode cites what it replaces):
 *   pre_mode 0  none
 *   pre_mode 1  RMSNorm of the input row: fp16(w * fp16(x * rsqrt(mean(x^2) + eps)))
 *               (model/llama.py:129-135); needs norm_weight_f16[n], in must be fp16
 *   pre_mode 2  SiLU-gated product: row of `in` is [gate(n) | up(n)], the transform input is
 *               fp16(fp16(silu(gate)) * up) (model/llama.py:399-400)
 *   residual_f16 != NULL: out = fp16(residual + fp16(result)), the decoder layer's
 *               residual addition (model/llama.py:964,979); out_dtype must be QTIP_F16.
 * in_parts > 1 is only allowed with pre_mode 0. */
int qtip_rht_fused(void* out, int out_dtype, const void* in, int in_dtype, int in_parts,
                   int rows, int n, int order, const uint32_t* had_bits,
                   const void* pre_f16, const float* post_f32, float scale,
                   int pre_mode, const void* norm_weight_f16, float eps,
                   const void* residual_f16, void* stream);

/* Output transform of one linear layer, residual addition, RMSNorm and the input transform of the
 * next linear layer for one hidden-size vector per row, in one launch (one workgroup per row):
 *   x_out  = fp16(residual + fp16(post * scale_out * H_n (sum over in_parts of parts)))
 *   xt_out = fp16(scale_in * H_n (pre * fp16(w * fp16(x_out * rsqrt(mean(x_out^2) + eps)))))
 * i.e. qtip_rht_fused(residual) followed by qtip_rht_fused(pre_mode 1) (model/llama.py:129-135,
 * 964-979 between two BitshiftLinear.forward calls, lib/codebook/bitshift.py:428-472).
 * n in {2048, 4096, 8192} (both transforms of order 1); parts is [in_parts][rows][n] fp32,
 * post fp32[n] or NULL, pre fp16[n] or NULL, residual / x_out / xt_out fp16 [rows][n]. */
int qtip_rht_chain(void* xt_out_f16, void* x_out_f16, const float* parts, int in_parts, int rows, int n,
                   const float* post_f32, float scale_out, const void* residual_f16,
                   const void* norm_weight_f16, float eps, const void* pre_f16, float scale_in,
                   void* stream);

/* Single-token decode attention for the end-to-end loop, one launch: rotary embedding of q and
 * k in fp16 arithmetic (model/llama.py:264-295), write of k and v into the static cache at the
 * token's position (model/cache_utils.py:1173-1193), softmax(q K^T / sqrt(d)) V over cache slots
 * 0..pos (model/llama.py:866-880).  qkv_f16 = [heads*d | kv_heads*d | kv_heads*d] of the new token,
 * caches are [kv_heads][max_len][d] fp16, pos_i64 points to the position in DEVICE memory (a
 * recorded graph then follows the position), inv_freq[d/2] fp32.  out_f16 = [heads*d].
 * key_splits (1..16): 1 = one workgroup per head walks the whole context (right up to a few
 * hundred keys: 6 us at 128, 10 us at 1024, 28 us at 4095); > 1 = the cache slots are cut into
 * key_splits equal ranges of max_len / key_splits slots, one workgroup per head and range, and a
 * second small launch combines the ranges' softmax shares, which pass through split_workspace:
 * heads * key_splits * (head_dim + 2) floats, 16-byte aligned, no initialisation needed (may be
 * NULL when key_splits == 1).  The caller picks key_splits from the longest context the call (or
 * the graph it records) will see. */
int qtip_decode_attention(void* out_f16, const void* qkv_f16, void* k_cache_f16, void* v_cache_f16,
                          const void* pos_i64, const float* inv_freq, int heads, int kv_heads,
                          int head_dim, int max_len, int key_splits, float* split_workspace, void* stream);

/* qtip_decode_attention on the qkv projection's raw matvec result: the output transform of
 * BitshiftLinear.forward (lib/codebook/bitshift.py:465-472: H_R, then * SV * 32) runs in the
 * kernel's prologue, each workgroup producing the three head-sized slices it needs, so the
 * [q | k | v] vector never exists in memory and the transform is no launch of its own.
 *   qkv = post * scale * (H_order (x) H_{n/order}) (parts[0] + ... + parts[in_parts-1]),
 * n = (heads + 2 kv_heads) * head_dim, n / order a power of two >= head_dim; had_bits = the packed
 * sign bits of the order x order table as qtip_rht takes them (NULL when order == 1); parts 16-byte
 * aligned fp32, part_stride (elements) a multiple of 4; head_dim 64 or 128.  Values are rounded to
 * fp16 where the layer's output is (the transform's sums are taken in another order than
 * qtip_rht's, so results agree to fp32 rounding before that cast, not bit for bit). */
int qtip_decode_attention_rht(void* out_f16, const float* parts, int in_parts, size_t part_stride,
                              const float* post_f32, float scale, const uint32_t* had_bits, int order,
                              void* k_cache_f16, void* v_cache_f16, const void* pos_i64,
                              const float* inv_freq, int heads, int kv_heads, int head_dim, int max_len,
                              int key_splits, float* split_workspace, void* stream);

/* qtip_decode_attention_rht for separate q / k / v projections: three raw matvec results, each
 * with the output transform of its own QuantizedLinear (q: heads * head_dim elements, k and v:
 * kv_heads * head_dim).  parts / post_f32 / had_bits are HOST arrays of three device pointers
 * (had_bits[i] NULL where order[i] == 1), scale / order host arrays of three values; the three
 * results share in_parts and part_stride (they are column ranges of one partial-sum buffer, as
 * qtip_decompress_matvec_group_chain writes it). */
int qtip_decode_attention_rht3(void* out_f16, const float* const* parts, int in_parts, size_t part_stride,
                               const float* const* post_f32, const float* scale,
                               const uint32_t* const* had_bits, const int* order, void* k_cache_f16,
                               void* v_cache_f16, const void* pos_i64, const float* inv_freq, int heads,
                               int kv_heads, int head_dim, int max_len, int key_splits,
                               float* split_workspace, void* stream);

/* Final RMSNorm of the decoder for one vector: out = weight * fp16(x * rsqrt(mean(x^2) + eps))
 * (model/llama.py:129-135), n <= 16384, one launch instead of the module's six. */
int qtip_rmsnorm(void* out_f16, const void* x_f16, const void* weight_f16, float eps, int n, void* stream);

/* Greedy token pick of the generation loop (eval/interactive_gen.py:43-69: argmax of the last
 * position's logits, copy into the next step's input, position + 1), all in device memory so a
 * recorded graph decodes token after token: tok_i64[0] = argmax(logits_f16[0..vocab)) (first index
 * among equal maxima; NaNs never win), history_i64[pos - history_base] = that token when the slot
 * lies in [0, history_len) (history may be NULL), pos_i64[0] += 1.  logits 16-byte aligned. */
int qtip_greedy_pick(const void* logits_f16, int vocab, void* tok_i64, void* pos_i64, void* history_i64,
                     long history_len, long history_base, void* stream);

/* Sampled token pick of the generation loop (eval/interactive_gen.py:15-40: logits / max(temperature,
 * 1e-5), entries below the top_k-th largest logit removed, softmax, a draw by the exponential race
 * argmax(p / q), q ~ Exp(1)) with the bookkeeping of qtip_greedy_pick, one launch.  top_k 0 keeps
 * the whole vocabulary, at most 64.  The race is evaluated as argmax(logit / T - log q) with q from
 * a counter-based generator keyed by (seed, counter_i64[0], entry); the counter is device memory
 * and advances by one per launch, so a recorded graph draws fresh numbers at every replay.  The
 * distribution is the reference's; the random stream is this library's own. */
int qtip_sample_pick(const void* logits_f16, int vocab, float temperature, int top_k, unsigned seed,
                     void* counter_i64, void* tok_i64, void* pos_i64, void* history_i64, long history_len,
                     long history_base, void* stream);

/* ---- packing tools (natural packing = one circular big-endian bitstream per tile, stored as
 * T*K/16 little-endian uint16 words; state i is the 16-bit window at bit i*K*V) ---------------- */

/* Byte permutation between the natural packing and the kernel packing of a 16x16-tile, V=2
 * matrix, m*k*bits/8 bytes each way; out and in must not overlap.
 * to_kernel != 0: natural -> kernel, the re-pack of lib/algo/finetune.py:196-201;
 * to_kernel == 0: kernel -> natural, lib/utils/kernel_decompress.py:19-24. */
int qtip_repack(void* out, const void* in, int m, int k, int bits, int to_kernel, void* stream);

/* Natural packing -> explicit states, states[ntiles][T/V] (int32, values < 65536).
 * Replaces bitshift_codebook.unpack_trellis (lib/codebook/bitshift.py:329-353).
 * L = 16; T = weights per tile; needs T % V == 0, (T*K) % 16 == 0, V in {1,2}, K*V <= 16. */
int qtip_unpack_trellis(int32_t* states, const void* packed, long ntiles, int T, int K, int V,
                        void* stream);

/* States -> natural packing (packed[ntiles][T*K/16] uint16).  Replaces
 * bitshift_codebook.pack_trellis (lib/codebook/bitshift.py:294-327).  *violations (device int,
 * zeroed by the caller) receives the number of consecutive state pairs that do not overlap by
 * 16 - K*V bits; the reference asserts that there are none (:307-309). */
int qtip_pack_trellis(void* packed, const int32_t* states, long ntiles, int T, int K, int V,
                      int* violations, void* stream);

/* Natural packing -> dense (m, n) matrix for any decode mode: lut is the expanded table
 * [V][65536] (cb.lut of the reference, QTIP_F16 or QTIP_F32), out has the table's dtype.
 * Replaces BitshiftLinear.get_hatW(cb.unpack_trellis(...)) (lib/codebook/bitshift.py:199-201,
 * 329-353, 378-381), the path taken when has_kernel is false. */
int qtip_decode_natural(void* out, const void* packed, const void* lut, int lut_dtype, int m, int n,
                        int td_x, int td_y, int K, int V, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QTIP_HIP_H */
