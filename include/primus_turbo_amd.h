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
 *             kernel leaves it zero-filled on exit, so one buffer can be reused
 *             by successive calls on the same stream without clearing it again;
 *             calls that may overlap (different streams) need separate buffers.
 */
PT_API size_t pt_quantize_fp8_tensorwise_workspace_bytes(void);
PT_API int    pt_quantize_fp8_tensorwise(const void *x, int x_dtype, int64_t numel, void *q,
                                         int q_dtype, const float *scale_in, float *scale_inv,
                                         void *workspace, size_t workspace_bytes, void *stream);

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
 * The tensor is viewed as [B, M, N] with the reduced axis = M when N > 1
 * ("column" scales, one per (b, n)) or as [outer, inner] rows when the reduced
 * axis is the last one (B*M rows of length N... expressed as B = outer, M = inner,
 * N = 1). scale / scale_inv hold B*N floats; numerics per scale as tensorwise
 * (eps 1e-12).
 *
 * scale_in : optional precomputed scales (B*N floats); NULL = dynamic amax.
 */
PT_API int pt_quantize_fp8_rowwise(const void *x, int x_dtype, int64_t B, int64_t M, int64_t N,
                                   void *q, int q_dtype, const float *scale_in, float *scale_inv,
                                   void *stream);
PT_API int pt_dequantize_fp8_rowwise(const void *q, int q_dtype, int64_t B, int64_t M, int64_t N,
                                     const float *scale_inv, void *y, int y_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PRIMUS_TURBO_AMD_H */
