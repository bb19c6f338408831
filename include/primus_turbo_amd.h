/*
 * primus_turbo_amd — C ABI of the gfx950 low-precision compute path
 * (FP8 / MXFP8 / MXFP4 quantizers and the scaled GEMMs that consume them).
 *
 * Conventions shared by every entry point:
 *   - All tensor arguments are raw DEVICE pointers to contiguous row-major
 *     storage; sizes are int64 element counts; dtypes are PT_DTYPE_* codes.
 *   - The library never allocates or frees device memory, never synchronises
 *     and launches only on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream). Outputs and workspaces are owned by the caller.
 *   - Return value 0 = success, negative = PT_ERR_*; pt_last_error() returns a
 *     thread-local message for the last failure on the calling thread.
 *   - "Replaces" comments cite the interface of AMD-AGI/Primus-Turbo that the
 *     entry point stands in for (paths relative to that repository).
 */
#ifndef PRIMUS_TURBO_AMD_H
#define PRIMUS_TURBO_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PT_API __attribute__((visibility("default")))

/* element type codes */
enum {
    PT_DTYPE_BF16 = 0,
    PT_DTYPE_F16  = 1,
    PT_DTYPE_F32  = 2,
    PT_DTYPE_E4M3 = 3, /* OCP float8_e4m3fn, max 448   */
    PT_DTYPE_E5M2 = 4, /* OCP float8_e5m2,   max 57344 */
    PT_DTYPE_E2M1X2 = 5, /* two OCP E2M1 values per byte, even element in the low nibble */
    PT_DTYPE_E8M0 = 6  /* biased power-of-two exponent byte */
};

/* status codes */
enum {
    PT_OK                   = 0,
    PT_ERR_INVALID_ARGUMENT = -1,
    PT_ERR_UNSUPPORTED      = -2,
    PT_ERR_WORKSPACE        = -3,
    PT_ERR_LAUNCH           = -4
};

/* Library / error plumbing ------------------------------------------------ */

/* Message for the last non-zero status returned on this thread ("" if none). */
PT_API const char *pt_last_error(void);
/* ABI version of this header (bumped on any signature change). */
PT_API int pt_abi_version(void);
/* Number of compute units of the current device (cached per device). */
PT_API int pt_device_cu_count(void);

/* FP8 tensorwise ------------------------------------------------------------
 *
 * Replaces torch.ops.primus_turbo_cpp_extension.quantize_fp8_tensorwise
 * (csrc/pytorch/bindings_pytorch.cpp:34, csrc/pytorch/quantization/quantization.cpp:44-90;
 * kernels csrc/kernels/reduce/reduce_row.cuh:16-88,
 * csrc/include/primus_turbo/device/quant_utils.cuh:62-74,
 * csrc/kernels/quantization/quantization_tensorwise.cu:51-111).
 *
 *   amax      = max |x|                        (fp32, NaN ignored)
 *   scale     = qmax / max(amax, 1e-12)        (IEEE fp32 division)
 *   scale_inv = 1.0f / scale
 *   q[i]      = fp8_rne(clamp(float(x[i]) * scale, -qmax, +qmax))
 *
 * One launch: every workgroup keeps its slice of x in registers across a
 * grid-wide amax exchange, so x is read from HBM once.
 *
 * scale_in  : optional device pointer to a precomputed fp32 scale (1 element);
 *             when non-NULL no amax is taken and scale_inv = 1.0f / *scale_in.
 * scale_inv : device fp32[1] output.
 * workspace : device memory of at least pt_quantize_fp8_tensorwise_workspace_bytes()
 *             bytes, 16-byte aligned, ZERO-FILLED before its first use. The
 *             kernels keep a generation counter and generation-tagged per-workgroup
 *             slots in it and maintain them from then on, so one buffer serves any
 *             number of successive calls on one stream (HIP-graph replays included)
 *             without being cleared again; calls that may overlap (different
 *             streams) need separate buffers. Unused when scale_in is given.
 *
 * The exchange waits for every workgroup of the launch with a bounded number of
 * probes. The launch is sized so that all its workgroups are resident (one per CU), so
 * the bound is only reached when something outside the library takes CUs away (CU
 * masking, a long kernel on another stream). Every wave still exits; the launch then
 * writes NaN into scale_inv, so that everything de-quantized or multiplied from the
 * result is NaN rather than plausible, and the _ex form raises *status.
 */
PT_API size_t pt_quantize_fp8_tensorwise_workspace_bytes(void);
PT_API int    pt_quantize_fp8_tensorwise(const void *x, int x_dtype, int64_t numel, void *q,
                                         int q_dtype, const float *scale_in, float *scale_inv,
                                         void *workspace, size_t workspace_bytes, void *stream);
/* Same operation with the exchange's failure handling exposed.
 * status         : optional device int32; every workgroup that gives up waiting stores 1
 *                  (never cleared by the library; NULL = not reported).
 * max_probes     : probe bound of the wait, 0 = the library's default (2^21).
 * phantom_blocks : number of additional, never-published slots the launch waits for;
 *                  0 in production. Tests pass 1 with a small max_probes to drive the
 *                  wait to its bound from the host while every wave exits normally. */
PT_API int pt_quantize_fp8_tensorwise_ex(const void *x, int x_dtype, int64_t numel, void *q,
                                         int q_dtype, const float *scale_in, float *scale_inv,
                                         void *workspace, size_t workspace_bytes, int32_t *status,
                                         uint32_t max_probes, int64_t phantom_blocks, void *stream);

/* pt_quantize_fp8_tensorwise without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc). It has no counterpart in Primus-Turbo. The exchange words live
 * in a static device array inside the library (66 KB per GPU, zero-initialised when the
 * code object loads, held until the process ends); neither this entry point nor anything
 * it calls allocates or frees memory. Same kernels and results as
 * pt_quantize_fp8_tensorwise.
 *
 * Each stream HANDLE that calls it on a device is given its own slot set and keeps it until
 * pt_tensorwise_static_release (the limit counts handles that have called and not released,
 * not streams in use at a time), at most PT_TENSORWISE_STATIC_MAX_STREAMS per device; one
 * more is rejected with PT_ERR_WORKSPACE, and numel above PT_TENSORWISE_STATIC_MAX_NUMEL
 * with PT_ERR_INVALID_ARGUMENT. Calls on one stream are ordered and share that stream's slot
 * set; the set keeps the last call's words (they are generation-tagged, so nothing has
 * to be cleared). Work that overlaps on one GPU while using ONE slot set races: a graph
 * captured on stream S and replayed on another stream while S is also calling, or the
 * same graph replayed concurrently on two streams.
 * status : as in pt_quantize_fp8_tensorwise_ex (optional). */
#define PT_TENSORWISE_STATIC_MAX_STREAMS 8
#define PT_TENSORWISE_STATIC_MAX_NUMEL (1LL << 37)
PT_API int pt_quantize_fp8_tensorwise_static(const void *x, int x_dtype, int64_t numel, void *q,
                                             int q_dtype, const float *scale_in, float *scale_inv,
                                             int32_t *status, void *stream);

/* Gives the slot set that pt_quantize_fp8_tensorwise_static keeps for `stream` on the current
 * device back, so that another stream handle can take it (a process that cycles through
 * stream handles would otherwise run out of the PT_TENSORWISE_STATIC_MAX_STREAMS sets). Every
 * call made on `stream` through the static entry point must have completed. A stream that
 * holds no set is not an error. Allocates nothing. No counterpart in Primus-Turbo. */
PT_API int pt_tensorwise_static_release(void *stream);

/* The same quantizer in two launches with no exchange between workgroups: per-workgroup
 * abs-max into the workspace, then every workgroup of the second launch reduces those, forms
 * the scale and casts. This is the launch structure of Primus-Turbo's own op
 * (csrc/pytorch/quantization/quantization.cpp:44-90: reduce, compute scale, cast; kernels
 * csrc/kernels/reduce/reduce_row.cuh:16-88, quantization_tensorwise.cu:51-111). Results are
 * bit-identical with pt_quantize_fp8_tensorwise. Nothing in it depends on all workgroups
 * of a launch being resident at once, so it is the form to use when other streams, CU
 * masks or graph replays beside eager work may hold compute units; x is read twice.
 * workspace : as for pt_quantize_fp8_tensorwise in size and alignment, but it needs NO
 *             zero-fill and carries nothing from call to call; calls that may overlap
 *             need separate buffers. */
PT_API int pt_quantize_fp8_tensorwise_two_pass(const void *x, int x_dtype, int64_t numel, void *q,
                                               int q_dtype, float *scale_inv, void *workspace,
                                               size_t workspace_bytes, void *stream);

/* Replaces torch.ops.primus_turbo_cpp_extension.dequantize_fp8_tensorwise
 * (csrc/pytorch/bindings_pytorch.cpp:38, quantization.cpp:211-230,
 * quantization_tensorwise.cu:113-154):  y[i] = T(float(q[i]) * scale_inv[0]). */
PT_API int pt_dequantize_fp8_tensorwise(const void *q, int q_dtype, int64_t numel,
                                        const float *scale_inv, void *y, int y_dtype,
                                        void *stream);

/* FP8 rowwise ---------------------------------------------------------------
 *
 * Replaces torch.ops.primus_turbo_cpp_extension.quantize_fp8_rowwise /
 * dequantize_fp8_rowwise (bindings_pytorch.cpp:36,40; quantization.cpp:110-208,232-282;
 * kernels quantization_rowwise.cu:59-183,188-286,288-503, reduce/reduce_col.cuh).
 *
 * The tensor is viewed as [B, M, N] with M the reduced axis: B = product of the
 * dimensions before it, N = product of those after it (N == 1 when the reduced
 * axis is the last, contiguous one). One scale per (b, n): scale_inv holds B*N
 * floats; numerics per scale as tensorwise (eps 1e-12).
 *
 * scale_in : optional precomputed scales (B*N floats); NULL = dynamic amax.
 */
PT_API int pt_quantize_fp8_rowwise(const void *x, int x_dtype, int64_t B, int64_t M, int64_t N,
                                   void *q, int q_dtype, const float *scale_in, float *scale_inv,
                                   void *stream);
PT_API int pt_dequantize_fp8_rowwise(const void *q, int q_dtype, int64_t B, int64_t M, int64_t N,
                                     const float *scale_inv, void *y, int y_dtype, void *stream);

/* FP8 128-blockwise (fp32 scales, eps 1e-4) -----------------------------------
 *
 * Numerics per block: scale = qmax / max(amax, 1e-4); the stored scale is
 * 1.0f / scale; q = fp8_rne(clamp(float(x) * scale, -qmax, qmax)). Elements
 * beyond the tensor edge count as zeros.
 *
 * pt_quantize_fp8_blockwise replaces primus_turbo::quant_fp8_blockwise_impl and
 * primus_turbo::quant_fp8_blockwise_dual_impl
 * (primus_turbo/pytorch/kernels/quantization/quantization_impl.py:81-125,236-281;
 * kernels primus_turbo/triton/quantization/quant_blockwise.py:11-112) for block 128.
 * x is [M, N]. Give q_row + scale_inv_row ([M, ceil(N/128)]) for 1 x 128 row
 * blocks, q_col + scale_inv_col ([ceil(M/128), N]) for 128 x 1 column blocks, or
 * both ("dual": x is read once).
 */
PT_API int pt_quantize_fp8_blockwise(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                                     void *q_row, float *scale_inv_row, void *q_col,
                                     float *scale_inv_col, void *stream);
/* The dual form with the column codes (also, or only: q_col may be NULL) emitted transposed,
 * q_col_t [N, ldt] with q_col_t[n, m] = q_col[m, n] and zeros in columns [M, ldt), ldt = M
 * rounded up to 128: the K-contiguous operand of the wgrad product of a linear layer (the
 * reference hands the untransposed codes to backends that read either layout,
 * ops/gemm_fp8.py:477-560). q_row / scale_inv_row are required. */
PT_API int pt_quantize_fp8_blockwise_t(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                                       void *q_row, float *scale_inv_row, void *q_col,
                                       void *q_col_t, int64_t ldt, float *scale_inv_col,
                                       void *stream);
/* The row direction of the above with its scales stored block-major, scale_inv_row_kmajor
 * [N / 128, M] (the value of row m and block kb at kb * M + m): the layout the block-scaled GEMM
 * reads per K slab, so that no transposition of the scale array precedes the product, and the one
 * in which the 128 scale values a workgroup produces per tile are contiguous (whole cache lines
 * instead of 128 masked 4-byte writes). q_col_t / ldt / scale_inv_col as for
 * pt_quantize_fp8_blockwise_t, or NULL / 0 / NULL for the row direction alone. Codes and scale
 * values are those of pt_quantize_fp8_blockwise; the reference has the [M, N / 128] layout only
 * (quantization_impl.py quant_fp8_blockwise_impl). */
PT_API int pt_quantize_fp8_blockwise_kmajor(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                                            void *q_row, float *scale_inv_row_kmajor, void *q_col_t,
                                            int64_t ldt, float *scale_inv_col, void *stream);

/* Replaces torch.ops.primus_turbo_cpp_extension.quantize_fp8_blockwise_for_weight
 * (bindings_pytorch.cpp:52-93, csrc/pytorch/quantization/quantization.cpp:1443-1480,
 * csrc/kernels/quantization/quantization_blockwise.cu:248-346): w is [B, M, N], one
 * scale per 128 x 128 tile, scale_inv is [B, ceil(M/128), ceil(N/128)]. */
PT_API int pt_quantize_fp8_blockwise_weight(const void *w, int w_dtype, int64_t B, int64_t M,
                                            int64_t N, void *q, int q_dtype, float *scale_inv,
                                            void *stream);
/* The same, and from the same read of w also q_t [B, N, ldt]: the codes transposed per batch
 * slice (q_t[b, n, m] = q[b, m, n]; M % 16 == 0, ldt >= M a multiple of 16; columns at and
 * beyond M are not written). It is the operand the dgrad product of a linear layer reads (the
 * reference hands the untransposed codes to backends that read either layout:
 * ops/gemm_fp8.py:477-560, ops/grouped_gemm_fp8.py:190-262); the tile scales serve both. */
PT_API int pt_quantize_fp8_blockwise_weight_dual(const void *w, int w_dtype, int64_t B, int64_t M,
                                                 int64_t N, void *q, void *q_t, int64_t ldt,
                                                 int q_dtype, float *scale_inv, void *stream);

/* Prefix sums of group lengths, each rounded up to `align` first:
 *   padded_lens[i] = round_up(group_lens[i], align)   (optional output, may be NULL)
 *   group_offs[0] = 0, group_offs[i+1] = group_offs[i] + padded_lens[i]
 * align = 1 replaces torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs
 * (bindings_pytorch.cpp:134, csrc/kernels/grouped_gemm/compute_group_offs.cu:15-42);
 * align = 128 replaces compute_padded_group_offs
 * (csrc/kernels/quantization/quantization_blockwise.cu:18-48). All int64, on device. */
PT_API int pt_compute_group_offs(const int64_t *group_lens, int64_t num_groups, int64_t align,
                                 int64_t *padded_lens, int64_t *group_offs, void *stream);

/* Replaces torch.ops.primus_turbo_cpp_extension.quantize_fp8_blockwise_segment_m_row_col
 * (csrc/pytorch/quantization/quantization.cpp:1384-1441,
 * csrc/kernels/quantization/quantization_blockwise.cu:60-232): one read of the
 * packed-M activation x [M, N] gives
 *   q_row [M, N] + scale_inv_row stored transposed [ceil(N/128), M]   (1 x 128 blocks)
 *   q_col_padded [M + G*128, N] + scale_inv_col_padded [(M + G*128)/128, N]
 *     (128 x 1 blocks of the segment-padded tensor: group g starts at row
 *      padded_group_offs[g], its pad rows are zero codes; rows at and beyond
 *      padded_group_offs[G] are left untouched).
 * group_offs / padded_group_offs are device int64 [G+1] (see pt_compute_group_offs). */
PT_API int pt_quantize_fp8_blockwise_segment_m_row_col(
    const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
    const int64_t *padded_group_offs, int64_t num_groups, void *q_row, float *scale_inv_row,
    void *q_col_padded, float *scale_inv_col_padded, void *stream);
/* The same with the column codes (also, or only: q_col_padded may be NULL) emitted transposed,
 * q_col_t [N, ldt] with q_col_t[n, r] = q_col_padded[r, n]: the K-contiguous operand of the
 * variable-K wgrad product. ldt >= M + G*128 rounded up to 128, a multiple of 16; columns at
 * and beyond padded_group_offs[G] are not written. Scales as above. */
PT_API int pt_quantize_fp8_blockwise_segment_m_row_col_t(
    const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
    const int64_t *padded_group_offs, int64_t num_groups, void *q_row, float *scale_inv_row,
    void *q_col_padded, void *q_col_t, int64_t ldt, float *scale_inv_col_padded, void *stream);

/* Gated activation fused into the grouped quantizer above: x is the fc1 output [M, 2 N] (gate
 * columns, then up columns) and what gets quantized is
 *   y[m, n] = T( act(x[m, n]) * x[m, N + n] * probs[m] ),   zero where row_mask[m] == 0,
 * act = 0 SiLU, 1 exact (erf) GELU, T = x's 16-bit type: the value swiglu_with_probs /
 * geglu_with_probs would store (primus_turbo/triton/activation/swiglu_kernel.py:11-248) followed
 * by quantize_fp8_blockwise_segment_m_row_col (csrc/kernels/quantization/quantization_blockwise.cu:
 * 60-232), without y ever travelling through HBM. Bit-identical with running the two steps of
 * this library one after the other. The reference has no fused form. probs is fp32 [M], row_mask
 * optional int64 [M]; give q_col_padded and / or q_col_t (with ldt) as above. */
PT_API int pt_glu_quantize_fp8_blockwise_segment_m_row_col(
    const void *x, int x_dtype, const float *probs, const int64_t *row_mask, int act, int64_t M, int64_t N,
    int q_dtype, const int64_t *group_offs, const int64_t *padded_group_offs, int64_t num_groups, void *q_row,
    float *scale_inv_row, void *q_col_padded, void *q_col_t, int64_t ldt, float *scale_inv_col_padded,
    void *stream);

/* De-quantize with one fp32 scale per (block_m x block_n) block of a [B, M, N] tensor:
 *   y[b, m, n] = T(float(q[b, m, n]) * scale_inv[b, m / block_m, n / block_n]).
 * (1, 128) / (128, 1) replace primus_turbo::dequant_fp8_blockwise_impl, (128, 128)
 * replaces primus_turbo::dequant_fp8_blockwise_for_weight_impl
 * (quantization_impl.py:146-234; quant_blockwise.py:162-234). */
PT_API int pt_dequantize_fp8_block(const void *q, int q_dtype, int64_t B, int64_t M, int64_t N,
                                   const float *scale_inv, int64_t block_m, int64_t block_n,
                                   void *y, int y_dtype, void *stream);

/* MX (microscaling) quantizers ------------------------------------------------
 *
 * pt_quantize_mx replaces the dispatcher ops quantize_mxfp8 / quantize_mxfp8_dual /
 * quantize_mxfp4 / quantize_mxfp4_dual (csrc/pytorch/quantization/quantization.cpp:511-969,
 * schemas csrc/pytorch/bindings_pytorch.cpp:52-93) and the FlyDSL kernels the Python layer
 * prefers for them (primus_turbo/flydsl/quantization/mxfp8_quant_flydsl.py:337-525,
 * mxfp4_quant_kernel.py:354-481), for round-to-nearest-even without RHT, stochastic rounding
 * or output shuffling.
 *
 * x is [B, M, N] bf16 / fp16 (B = 1 for a matrix). q_dtype: PT_DTYPE_E4M3, PT_DTYPE_E5M2
 * (MXFP8) or PT_DTYPE_E2M1X2 (MXFP4, two codes per byte). One E8M0 byte per 32 elements:
 *   e = clamp((((bits(amax) + R) >> 23) & 0x1FF) - 127 - T, -127, 128),  byte = e + 127,
 *   q = rne_sat(clamp(x * 2^-e, +-qmax));  (R, T) = (1<<19, 8) E4M3, (1<<20, 15) E5M2,
 *   (1<<21, 2) E2M1.
 * Row direction (blocks of 32 along N): row_q [B, M, Npad] codes (FP4: Npad / 2 bytes per
 * row), row_scale [B, M, Npad / 32]; Npad = N rounded up to 128, the padding is zero data
 * with scale byte 0. Column direction (blocks of 32 along M), emitted transposed:
 * col_q [B, N, Mpad], col_scale [B, N, Mpad / 32]. Either pair may be NULL. row_flags /
 * col_flags: bit 0 shares one exponent per 32 x 32 tile (weights); bit 1 (MXFP4 only, not with
 * bit 0) quantizes the Hadamard-transformed values: every 16 consecutive elements along the
 * direction (of the zero-padded tensor) are replaced by (H4 (x) H4) / 4 times themselves, in fp32
 * with the operation order of flydsl/quantization/mxfp4_quant_kernel.py:92-118 -- the recipe's
 * "RHT" of the two wgrad operands, which cancels in their product. Bit 2 (MXFP4 only) rounds
 * the codes stochastically (unbiased; scales unchanged) from sr_seed, which the caller changes
 * from launch to launch (mxfp4_quant_kernel.py:48-75: random by design, not reproducible bit
 * for bit against the reference).
 *
 * pt_dequantize_mx replaces dequantize_mxfp8 / dequantize_mxfp4 (quantization.cpp:285-359,
 * 436-508; kernels dequantization_mxfp8.cu:29-113, dequantization_mxfp4.cu:28-160):
 *   y[r, c] = T(float(q[r, c]) * bits_to_f32(scale[r, c / 32] << 23))
 * over q [rows, cols] (cols % 32 == 0; FP4 packed), written as y [rows, cols] or, for
 * column-direction data, transposed back as y [cols, rows]. */
PT_API int pt_quantize_mx(const void *x, int x_dtype, int64_t B, int64_t M, int64_t N, int q_dtype,
                          void *row_q, void *row_scale, int row_flags, void *col_q, void *col_scale,
                          int col_flags, uint32_t sr_seed, void *stream);
PT_API int pt_dequantize_mx(const void *q, int q_dtype, const void *scale, int64_t rows,
                            int64_t cols, void *y, int y_dtype, int transpose, void *stream);

/* Scaled FP8 GEMM -------------------------------------------------------------
 *
 * Replaces primus_turbo::gemm_fp8_impl / gemm_fp8_accum_impl
 * (primus_turbo/pytorch/kernels/gemm/gemm_fp8_impl.py:518-585) for the TENSORWISE,
 * ROWWISE and BLOCKWISE granularities, i.e. the Triton kernels of
 * primus_turbo/triton/gemm/gemm_fp8_kernel.py:123-243,446-565,871-1183 and the
 * CK / hipBLASLt instantiations behind the same op.
 *
 *   C[M, N] (+)= scale( op(A) . op(B) ),  fp32 accumulation, C in c_dtype.
 *   trans_a == 0: A is stored [M, K];  trans_a != 0: A is stored [K, M].
 *   trans_b != 0: B is stored [N, K];  trans_b == 0: B is stored [K, N].
 * The MFMA kernel contracts along contiguous K in steps of 128; an operand stored with
 * K as its row axis is transposed into `workspace` first, and when K is not a multiple
 * of 128 both operands are copied there with a zero-filled K tail
 * (pt_gemm_fp8_workspace_bytes(M, N, K, trans_a, trans_b) bytes, 16-byte aligned;
 * zero bytes, and `workspace` may be NULL, for trans_a == 0, trans_b != 0, K % 128 == 0, K >= 512).
 *
 * scale_mode 0 (vector):  C = (A.B) * a_scale[m * sa_m] * b_scale[n * sb_n]
 *     tensorwise: sa_m = sb_n = 0;  rowwise: sa_m = sb_n = 1.
 * scale_mode 1 (128-block along K; kb runs over ceil(K / 128) blocks):
 *     C = sum_kb (A_kb.B_kb) * a_scale[(m / sa_block) * sa_m + kb * sa_k]
 *                            * b_scale[(n / sb_block) * sb_n + kb * sb_k]
 *     sa_block / sb_block are 1 (1 x 128 activation blocks) or 128 (128 x 128 tiles).
 * accumulate != 0 adds into C (beta = 1) instead of overwriting it.
 * tile_cfg: 0 = automatic, 1 = 256x256, 2 = 256x128, 3 = 128x128 workgroup tile,
 *           4 = 256x256 with eight wavefronts (block scales with 128 x 128 B blocks).
 * For large problems the workspace also holds a [K / 128, M] copy of per-row block scales that
 * arrive as [M, K / 128] (sa_block == 1, sa_k == 1): the kernel's scale copies then read
 * contiguous memory. It is made only when the workspace has the size the function reports.
 * Requirements: a, b, c 16-byte aligned.
 */
PT_API size_t pt_gemm_fp8_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a,
                                          int trans_b);
PT_API int pt_gemm_fp8(const void *a, int a_dtype, const float *a_scale, const void *b, int b_dtype,
                       const float *b_scale, void *c, int c_dtype, int64_t M, int64_t N, int64_t K,
                       int trans_a, int trans_b, int scale_mode, int64_t sa_m, int64_t sa_k,
                       int64_t sb_n, int64_t sb_k, int sa_block, int sb_block, int accumulate,
                       void *workspace, size_t workspace_bytes, int tile_cfg, void *stream);

/* MX-scaled GEMM (MXFP8 / MXFP4), NT layout ----------------------------------
 *
 * Replaces primus_turbo::gemm_fp8_impl for the MX_BLOCKWISE granularity
 * (primus_turbo/pytorch/kernels/gemm/gemm_fp8_impl.py:341-496, hipBLASLt / AITER / FlyDSL
 * behind it) and primus_turbo::gemm_fp4_impl (kernels/gemm/gemm_fp4_impl.py:53-319,339-430):
 *
 *   C[m, n] = sum_kb 2^(a_scale[m, kb] - 127) * 2^(b_scale[n, kb] - 127)
 *                    * sum_{k in block kb} A[m, k] * B[n, k],      32-wide K blocks,
 *
 * fp32 accumulation, the block scales applied by the matrix core. A is [M, K] and B is [N, K]
 * (both K-contiguous) with row pitches lda / ldb in BYTES; ab_dtype PT_DTYPE_E4M3 / PT_DTYPE_E5M2
 * selects MXFP8 (a_e5m2 / b_e5m2 give each operand's format), PT_DTYPE_E2M1X2 selects MXFP4 (two
 * codes per byte, K counts codes). a_scale [M, >= K / 32] and b_scale [N, >= K / 32] are E8M0
 * bytes with row pitches sa_ld / sb_ld. K % 32 == 0; bytes of a row behind K must be zero
 * codes, as the MX quantizers leave them. Rows that are not whole 128-byte slabs (at least
 * four) are first copied into `workspace` (16-byte aligned); a workspace of
 * pt_gemm_mx_workspace_bytes also receives, for large problems, a copy of both scale arrays with
 * the 32-bit words of one K position of all rows contiguous, which is what the kernel's scale
 * copies then read (faster; with a smaller workspace, or none when no row copy is needed, the
 * scales are read in place).
 * accumulate != 0 adds into C (beta = 1). tile_cfg as for pt_gemm_fp8; 4 = 256 x 256 tile with
 * eight wavefronts (the automatic choice for MXFP4 with M, N >= 2048), bit-identical results. */
PT_API size_t pt_gemm_mx_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                                         int fp4);
PT_API int pt_gemm_mx(const void *a, const void *a_scale, const void *b, const void *b_scale,
                      int ab_dtype, int a_e5m2, int b_e5m2, void *c, int c_dtype, int64_t M,
                      int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t sa_ld, int64_t sb_ld,
                      int accumulate, void *workspace, size_t workspace_bytes, int tile_cfg,
                      void *stream);

/* MoE grouped FP8 GEMM, 128-blockwise scales -------------------------------
 *
 * pt_grouped_gemm_fp8 replaces primus_turbo::grouped_gemm_fp8_impl
 * (primus_turbo/pytorch/kernels/grouped_gemm/grouped_gemm_fp8_impl.py:888-930; Triton kernels
 * primus_turbo/triton/grouped_gemm/grouped_gemm_fp8_kernel.py:1405-1556,1809-1944) for the
 * BLOCKWISE granularity, the forward and dgrad product of a grouped linear layer:
 *
 *   out[offs[g] : offs[g+1], :] = A[offs[g] : offs[g+1], :] . W_g^T      g = 0 .. G-1
 *   out[offs[G] : out_rows, :]  = 0
 *
 * A is [M, K] fp8 with one scale per row and 128-wide K block stored K-block major,
 * a_scale[kb * M + m] (the "pre-shuffled" row scales of
 * pt_quantize_fp8_blockwise_segment_m_row_col). trans_b != 0: W is [G, N, K] with tile scales
 * [G, ceil(N/128), ceil(K/128)]; trans_b == 0: W is [G, K, N] with [G, ceil(K/128), ceil(N/128)].
 * group_offs: device int64 [G + 1] prefix sums of the per-group row counts (no host sync; groups
 * may be empty). The workspace (pt_grouped_gemm_fp8_workspace_bytes) holds the K-contiguous
 * copy of W when trans_b == 0 and zero-padded copies when K % 128 != 0 or K < 512.
 *
 * pt_grouped_gemm_fp8_variable_k replaces primus_turbo::grouped_gemm_fp8_variable_k_impl and
 * ..._variable_k_accum_impl (grouped_gemm_fp8_impl.py:933-1022; Triton
 * grouped_gemm_fp8_kernel.py:1656-1802,1951-2103), the wgrad product:
 *
 *   C[g] (+)= LHS[p[g] : p[g+1], :]^T . RHS[p[g] : p[g+1], :]     ([Ml, Nr]; [Nr, Ml] if trans_c)
 *
 * LHS [Mp, Ml] and RHS [Mp, Nr] are the segment-padded column quantizations (each group's rows
 * rounded up to a multiple of 128, pad rows zero) with scales [Mp / 128, cols]; p = padded
 * group offsets (device int64 [G + 1], multiples of 128). An empty group yields C[g] = 0
 * (or leaves it unchanged when accumulating). The workspace holds both transposed operands.
 * operands_kmajor != 0: LHS and RHS arrive transposed already, [Ml, Mp] and [Nr, Mp] (the
 * q_col_t output of pt_quantize_fp8_blockwise_segment_m_row_col_t, scales unchanged); no
 * workspace is used. tile_cfg 4 (the automatic choice for outputs of 1024 x 1024 and more) is a
 * 256 x 256 tile with eight wavefronts that streams through the K ranges of consecutive groups
 * without restarting its pipeline, writing one result tile per group on the way.
 */
PT_API size_t pt_grouped_gemm_fp8_workspace_bytes(int64_t G, int64_t M, int64_t N, int64_t K,
                                                  int trans_b);
PT_API int pt_grouped_gemm_fp8(const void *a, int a_dtype, const float *a_scale, const void *b,
                               int b_dtype, const float *b_scale, void *c, int c_dtype,
                               const int64_t *group_offs, int64_t G, int64_t M, int64_t out_rows,
                               int64_t N, int64_t K, int trans_b, void *workspace,
                               size_t workspace_bytes, int tile_cfg, void *stream);
PT_API size_t pt_grouped_gemm_fp8_variable_k_workspace_bytes(int64_t Mp, int64_t Ml, int64_t Nr);
PT_API int pt_grouped_gemm_fp8_variable_k(const void *lhs, int lhs_dtype, const float *lhs_scale,
                                          const void *rhs, int rhs_dtype, const float *rhs_scale,
                                          void *c, int c_dtype, const int64_t *group_offs, int64_t G,
                                          int64_t Mp, int64_t Ml, int64_t Nr, int trans_c,
                                          int accumulate, int operands_kmajor, void *workspace,
                                          size_t workspace_bytes, int tile_cfg, void *stream);

/* Grouped GEMM with vector scales (TENSORWISE / ROWWISE granularities) -----------------
 *
 * pt_grouped_gemm_fp8_vec replaces primus_turbo::grouped_gemm_fp8_impl for TENSORWISE and
 * ROWWISE (kernels/grouped_gemm/grouped_gemm_fp8_impl.py:888-930; callers
 * ops/grouped_gemm_fp8.py:265-603), forward and dgrad:
 *   out[offs[g] : offs[g+1], n] = (A[offs[g] : offs[g+1]] . op(B[g]))[., n]
 *                                 * a_scale[m * sa_stride] * b_scale[g * sb_gstride + n * sb_stride]
 *   out[offs[G] : out_rows] = 0
 * A [M, K] fp8; trans_b != 0: B [G, N, K], else [G, K, N]. Strides in floats: 0 = one scalar
 * (TENSORWISE), 1 = one per row / column (ROWWISE). The workspace
 * (pt_grouped_gemm_fp8_vec_workspace_bytes) holds the K-contiguous copy of B when trans_b == 0
 * and zero-padded copies when K % 128 != 0 or K < 512.
 *
 * pt_grouped_gemm_fp8_vec_variable_k replaces primus_turbo::grouped_gemm_fp8_variable_k_impl for
 * the same granularities (grouped_gemm_fp8_impl.py:933-1022), wgrad over tightly packed groups:
 *   C[g][i, j] (+)= (L[offs[g] : offs[g+1]]^T . R[offs[g] : offs[g+1]])[i, j]
 *                   * lhs_scale[i * sl_stride] * rhs_scale[j * sr_stride]
 * L [M, Ml], R [M, Nr] fp8, C [G, Ml, Nr] (trans_c: [G, Nr, Ml]). The workspace holds the padded
 * group offsets and both operands copied K-contiguous with every group padded to a multiple of
 * 128 rows of zeros. */
PT_API size_t pt_grouped_gemm_fp8_vec_workspace_bytes(int64_t G, int64_t M, int64_t N, int64_t K,
                                                      int trans_b);
PT_API int pt_grouped_gemm_fp8_vec(const void *a, int a_dtype, const float *a_scale, int64_t sa_stride,
                                   const void *b, int b_dtype, const float *b_scale, int64_t sb_stride,
                                   int64_t sb_gstride, void *c, int c_dtype, const int64_t *group_offs,
                                   int64_t G, int64_t M, int64_t out_rows, int64_t N, int64_t K,
                                   int trans_b, void *workspace, size_t workspace_bytes, int tile_cfg,
                                   void *stream);
PT_API size_t pt_grouped_gemm_fp8_vec_variable_k_workspace_bytes(int64_t G, int64_t M, int64_t Ml,
                                                                 int64_t Nr);
PT_API int pt_grouped_gemm_fp8_vec_variable_k(const void *lhs, int lhs_dtype, const float *lhs_scale,
                                              int64_t sl_stride, const void *rhs, int rhs_dtype,
                                              const float *rhs_scale, int64_t sr_stride, void *c,
                                              int c_dtype, const int64_t *group_offs, int64_t G,
                                              int64_t M, int64_t Ml, int64_t Nr, int trans_c,
                                              int accumulate, void *workspace, size_t workspace_bytes,
                                              int tile_cfg, void *stream);

/* Grouped MXFP8 path (MoE experts with E8M0 block scales) ------------------------------
 *
 * pt_grouped_quantize_mx replaces the dispatcher ops grouped_quantize_mxfp8 /
 * grouped_quantize_mxfp8_dual (csrc/pytorch/quantization/quantization.cpp:971-1378; Python
 * quantization_impl.py:572-700, FlyDSL mxfp8_quant_flydsl.py:982-1045) for round-to-nearest-even
 * without output shuffling: x [M, N] bf16 / fp16 holds the rows of G groups (group_offs, device
 * int64 [G + 1]); numerics per 32-element block as pt_quantize_mx.
 *   Row direction: row_q [*, Npad] codes and row_scale [*, Npad / 32] with the rows of group g
 *   at row_offs_padded[g] (every group padded to a multiple of 32 rows; pad rows are not
 *   written); row_offs_padded == NULL keeps the rows where they are in x.
 *   Column direction, emitted transposed: col_q [N, col_ld], col_scale [N, col_ld / 32] with
 *   the rows of group g at columns col_offs_padded[g] ... (every group padded to a multiple of
 *   128 rows with zero data, scale byte 0); col_ld is a multiple of 128 >= col_offs_padded[G];
 *   columns from col_offs_padded[G] on are not written.
 * Either pair may be NULL. The padded offsets come from pt_compute_group_offs (align 32 / 128).
 * With q_dtype e2m1x2 it is the grouped MXFP4 quantizer (grouped_quantize_mxfp4[_dual],
 * quantization.cpp:1209-1378; default dispatch flydsl/quantization/mxfp4_grouped_quant.py:320-349):
 * two codes per byte, rows kept tight (row_offs_padded NULL) and column groups padded to 256;
 * row_flags / col_flags / sr_seed as for pt_quantize_mx; a direction's 32 x 32 blocks (bit 0) are
 * counted from its group's first row, the rows behind the group's end being zeros.
 *
 * pt_grouped_gemm_mx replaces primus_turbo::grouped_gemm_fp8_impl for MX_BLOCKWISE
 * (kernels/grouped_gemm/grouped_gemm_fp8_impl.py:888-930 with group_offs_out; caller
 * ops/grouped_gemm_fp8.py:726-741,786-801) and primus_turbo::grouped_gemm_fp4_impl
 * (kernels/grouped_gemm/grouped_gemm_fp4_impl.py; caller ops/grouped_gemm_fp4.py:226-240,
 * 279-293), forward and dgrad:
 *   out[oo[g] : oo[g] + len_g, :] = A[o[g] : o[g] + len_g, :] . B[g]^T,   out[oo[G] : out_rows] = 0
 * A [a_rows, lda bytes] MXFP8 (or, both operands, packed MXFP4) codes with scale bytes
 * [a_rows, sa_ld], B [G, N, ldb bytes] with [G, N, sb_ld]; o = group_offs (rows of A, e.g. the
 * padded row layout above), oo = group_offs_out (rows of the output, packed tight; NULL = the
 * same as o); len_g = oo[g + 1] - oo[g] when oo is given. K counts elements (a multiple of 32);
 * lda == ldb is a multiple of 128 bytes, at least 512, and the bytes of a row behind its K
 * codes are zero.
 *
 * pt_grouped_gemm_mx_variable_k replaces primus_turbo::grouped_gemm_fp8_variable_k_impl for
 * MX_BLOCKWISE (grouped_gemm_fp8_impl.py:933-974; caller ops/grouped_gemm_fp8.py:809-825) and
 * primus_turbo::grouped_gemm_fp4_variable_k[_accum]_impl (caller ops/grouped_gemm_fp4.py:56-98,
 * 296-312), wgrad:
 *   C[g] (+)= L[:, p[g] : p[g+1]] . R[:, p[g] : p[g+1]]^T      C is [G, Ml, Nr]
 * L [Ml, ld] and R [Nr, ld] (ld in elements) are transposed column-direction outputs of
 * pt_grouped_quantize_mx with scale bytes [rows, ld / 32]; p = the group offsets in elements,
 * padded to whole 128-byte slabs (128 elements, MXFP4: 256). An empty group yields C[g] = 0 (or
 * leaves it unchanged when accumulating). Both operands are read in place.
 *
 * workspace (both entry points; optional, NULL = none): room for word-major copies of the two
 * scale arrays (pt_grouped_gemm_mx_workspace_bytes / ..._variable_k_workspace_bytes, 16-byte
 * aligned), which turn the kernel's scale copies into contiguous reads; without it the scale
 * arrays are read where they are. */
PT_API int pt_grouped_quantize_mx(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                                  const int64_t *group_offs, const int64_t *row_offs_padded,
                                  const int64_t *col_offs_padded, int64_t G, void *row_q,
                                  void *row_scale, int row_flags, void *col_q, void *col_scale,
                                  int col_flags, int64_t col_ld, uint32_t sr_seed, void *stream);
/* Gated activation fused into pt_grouped_quantize_mx: x is the fc1 output [M, 2 N] (gate
 * columns, then up columns) and what gets quantized is
 *   y[m, n] = T( act(x[m, n]) * x[m, N + n] * probs[m] ),   zero where row_mask[m] == 0,
 * act = 0 SiLU, 1 exact (erf) GELU, T = x's 16-bit type: the value swiglu_with_probs /
 * geglu_with_probs would store (primus_turbo/triton/activation/swiglu_kernel.py:11-248) followed
 * by grouped_quantize_mxfp8[_dual] / grouped_quantize_mxfp4[_dual] (quantization.cpp:971-1378),
 * without y travelling through HBM; bit-identical with running the two steps of this library one
 * after the other. The reference has no fused form. Round to nearest, 1-D blocks; row_q /
 * row_scale are required (fc2's forward operand), col_q / col_scale (its wgrad operand) optional;
 * col_flags: 0, or 2 = Hadamard-transformed column direction (MXFP4's wgrad recipe). probs is
 * fp32 [M], row_mask optional int64 [M]. */
PT_API int pt_glu_grouped_quantize_mx(const void *x, int x_dtype, const float *probs, const int64_t *row_mask,
                                      int act, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
                                      const int64_t *row_offs_padded, const int64_t *col_offs_padded, int64_t G,
                                      void *row_q, void *row_scale, void *col_q, void *col_scale, int col_flags,
                                      int64_t col_ld, void *stream);
PT_API int pt_grouped_gemm_mx(const void *a, int a_dtype, const void *a_scale, int64_t lda,
                              int64_t sa_ld, const void *b, int b_dtype, const void *b_scale,
                              int64_t ldb, int64_t sb_ld, void *c, int c_dtype,
                              const int64_t *group_offs, const int64_t *group_offs_out, int64_t G,
                              int64_t a_rows, int64_t out_rows, int64_t N, int64_t K, void *workspace,
                              size_t workspace_bytes, int tile_cfg, void *stream);
PT_API size_t pt_grouped_gemm_mx_workspace_bytes(int64_t G, int64_t a_rows, int64_t N, int64_t K);
PT_API size_t pt_grouped_gemm_mx_variable_k_workspace_bytes(int64_t Ml, int64_t Nr, int64_t ld);
PT_API int pt_grouped_gemm_mx_variable_k(const void *lhs, int lhs_dtype, const void *lhs_scale,
                                         const void *rhs, int rhs_dtype, const void *rhs_scale, void *c,
                                         int c_dtype, const int64_t *group_offs, int64_t G, int64_t Ml,
                                         int64_t Nr, int64_t ld, int accumulate, void *workspace,
                                         size_t workspace_bytes, int tile_cfg, void *stream);

/* Gated activation of an MoE expert MLP with the router probability folded in -------------
 *
 * Replaces swiglu_fwd_with_probs / swiglu_bwd_with_probs and geglu_fwd_with_probs /
 * geglu_bwd_with_probs (primus_turbo/pytorch/kernels/activation/swiglu_impl.py:20-117,
 * geglu_impl.py; Triton kernels primus_turbo/triton/activation/swiglu_kernel.py:11-248):
 *   out[t, c]     = act(x[t, c]) * x[t, H + c] * probs[t]                      x [rows, 2 H]
 *   grad_x[t, c]     = grad_out[t, c] * probs[t] * x[t, H + c] * act'(x[t, c])
 *   grad_x[t, H + c] = grad_out[t, c] * probs[t] * act(x[t, c])
 *   grad_probs[t]    = sum_c grad_out[t, c] * act(x[t, c]) * x[t, H + c]
 * act: 0 = SiLU, 1 = exact (erf) GELU; x / out / grad in bf16 or fp16, probs and grad_probs fp32,
 * arithmetic in fp32. row_mask (device int64 [rows], may be NULL): rows with 0 produce zeros. */
PT_API int pt_glu_with_probs_fwd(const void *x, int x_dtype, const float *probs,
                                 const int64_t *row_mask, void *out, int64_t rows, int64_t H, int act,
                                 void *stream);
PT_API int pt_glu_with_probs_bwd(const void *grad_out, const void *x, int x_dtype, const float *probs,
                                 const int64_t *row_mask, void *grad_x, float *grad_probs,
                                 int64_t rows, int64_t H, int act, void *stream);

/* Byte-matrix transpose out[b, c, r] = in[b, r, c] (fp8 payloads; replaces the 2-D
 * transpose used for tensorwise `.t()` copies, csrc/kernels/transpose/). */
PT_API int pt_transpose_u8(const void *in, void *out, int64_t batch, int64_t R, int64_t C,
                           void *stream);
/* The same for elements of 1, 2, 4 or 8 bytes. Replaces
 * torch.ops.primus_turbo_cpp_extension.transpose_2d (csrc/pytorch/bindings_pytorch.cpp:44,
 * csrc/pytorch/transpose/transpose.cpp:17-49: last two dimensions of a contiguous 2-D / 3-D
 * tensor of any dtype). */
PT_API int pt_transpose_2d(const void *in, void *out, int64_t batch, int64_t R, int64_t C,
                           int elem_bytes, void *stream);

/* Pre-shuffled MX operand layouts (the (16, 16) tile orders that the reference hands to AITER's
 * a4w4 GEMM). Replaces shuffle_weight / shuffle_e8m0_scale (csrc/include/primus_turbo/shuffle.h:26-32,
 * csrc/kernels/shuffle/shuffle.cu:32-160; index maps csrc/include/primus_turbo/device/shuffle.cuh:39-80)
 * and the shuffle_out / shuffle_scale outputs of the MX quantizers
 * (csrc/pytorch/quantization/quantization.cpp:553-603). `inverse` != 0 brings a shuffled tensor back
 * to the plain row-major layout (no counterpart in the reference, whose GEMMs read the shuffled one).
 *
 * pt_shuffle_mx_codes: [rows, row_bytes] code bytes (FP4 pairs or FP8), rows % 16 == 0,
 *   row_bytes % 32 == 0; every 16-row x 32-byte tile is stored as two contiguous 16 x 16-byte halves.
 * pt_shuffle_e8m0_scale: `batch` matrices [M, N] of E8M0 bytes <-> [M_pad, N_pad] (M_pad % 32 == 0,
 *   N_pad % 8 == 0, the reference pads M to 256 and N to 8), zero outside [M, N]; every 32 x 8 tile is
 *   stored in the order (col % 4, row % 16, (col % 8) / 4, (row % 32) / 16). */
PT_API int pt_shuffle_mx_codes(const void *in, void *out, int64_t rows, int64_t row_bytes, int inverse,
                               void *stream);
PT_API int pt_shuffle_e8m0_scale(const void *in, void *out, int64_t batch, int64_t M, int64_t N,
                                 int64_t M_pad, int64_t N_pad, int inverse, void *stream);

/* MoE token permute / unpermute (the step before and after the grouped GEMMs of an expert bank).
 * Replaces permute_preprocessing_impl / permute_impl / unpermute_impl
 * (csrc/include/primus_turbo/moe_permute.h, csrc/kernels/moe_permute/moe_permute.cu:84-330, :425-510,
 * :553-745; schemas csrc/pytorch/bindings_pytorch.cpp:100-112).
 *
 * pt_moe_permute_preprocess: expert_map is bool [T, E] (map_kind 0) or topk_idx [T, num_topk] of
 *   int32 / int64 (1 / 2; entries outside [0, E) are ignored). Writes row_id_map
 *   [T + pad_multiple, 2 E + 1] (row of a token: [2E] = n routed experts, [0, n) = 1-based destination
 *   rows in ascending expert order, [E, E + n) = expert id, or the top-k slot when
 *   topk_aligned_probs; rows T + i: negative 1-based rows of the i-th zero pad row of every expert that
 *   has one; other entries are left as they are), tokens_per_expert [E] (padded to pad_multiple,
 *   clipped at num_permuted_tokens when that is > 0), overflow_flag (1 when rows were dropped for
 *   that limit), num_dispatched_tokens (tokens routed to at least one local expert). E <= 240.
 *   workspace: pt_moe_permute_workspace_bytes(T, E) bytes, contents irrelevant. Three launches, no host
 *   synchronisation, no inter-block waiting.
 * pt_moe_permute: copies token rows (hidden_bytes each, a multiple of 16) to their destination rows
 *   and writes the zero pad rows; optional per-token scale factors (scale_bytes_per_token raw bytes)
 *   and probs (prob_bytes 2 or 4; source row stride probs_stride elements, column from the map) ride
 *   along. Rows of permuted_tokens that no map entry names are left untouched; map entries at or
 *   beyond num_permuted_rows (the rows the permuted tensors hold) are skipped, also in pt_moe_unpermute.
 * pt_moe_unpermute: tokens[t] = sum over the token's experts of permuted_tokens[row] (fp32
 *   accumulation in map order, bf16 / fp16 storage; zeros for a token routed nowhere); optional probs
 *   scattered back into zero-filled rows of probs_stride elements. */
PT_API size_t pt_moe_permute_workspace_bytes(int64_t num_tokens, int64_t num_local_experts);
PT_API int pt_moe_permute_preprocess(const void *expert_map, int map_kind, int64_t num_tokens,
                                     int64_t num_local_experts, int64_t num_topk, int64_t pad_multiple,
                                     int64_t num_permuted_tokens, int topk_aligned_probs, int *row_id_map,
                                     int64_t *tokens_per_expert, int *overflow_flag,
                                     int *num_dispatched_tokens, void *workspace, size_t workspace_bytes,
                                     void *stream);
PT_API int pt_moe_permute(const void *tokens, void *permuted_tokens, int64_t hidden_bytes,
                          const void *scaling_factor, void *permuted_scaling_factor,
                          int64_t scale_bytes_per_token, const void *probs, void *permuted_probs,
                          int prob_bytes, int64_t probs_stride, const int *row_id_map, int64_t num_tokens,
                          int64_t pad_multiple, int64_t num_local_experts, int64_t num_permuted_rows,
                          void *stream);
PT_API int pt_moe_unpermute(const void *permuted_tokens, void *tokens, int dtype, int64_t hidden,
                            const void *permuted_probs, void *probs, int prob_bytes, int64_t probs_stride,
                            const int *row_id_map, int64_t num_tokens, int64_t num_local_experts,
                            int64_t num_permuted_rows, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PRIMUS_TURBO_AMD_H */
