// Pre-shuffled MX operand layouts: the (16, 16) tile orders in which Primus-Turbo hands MXFP4 / MXFP8
// codes and their E8M0 scales to AITER's a4w4 GEMM (csrc/include/primus_turbo/device/shuffle.cuh:39-80,
// csrc/kernels/shuffle/shuffle.cu:32-115, host side csrc/pytorch/shuffle/shuffle.cpp:15-83).
//
//   codes  [R, W bytes], R % 16 == 0, W % 32 == 0: every 16-row x 32-byte tile becomes two
//          16 x 16-byte halves, each contiguous:
//            byte (r, c) -> (r / 16) * 16 W + (c / 32) * 512 + ((c % 32) / 16) * 256 + (r % 16) * 16 + c % 16
//   scales [M, N] bytes -> [Mp, Np] (Mp % 32 == 0, Np % 8 == 0, zero outside [M, N]): every 32 x 8 tile
//          is stored as (col % 4, row % 16, (col % 8) / 4, (row % 32) / 16):
//            byte (r, c) -> (r / 32) * 32 Np + (c / 8) * 256 + (c % 4) * 64 + (r % 16) * 4 + ((c % 8) / 4) * 2 + (r % 32) / 16
//
// The GEMM kernels of this library read plain row-major operands; these passes exist so that callers who
// produce or hold the shuffled layouts get the same bytes, and to bring such operands back.
// Pure byte movement, HBM-bound: 16-byte accesses for codes, one 4-byte word per thread for scales.
#include "pt_common.h"

namespace pt {

// one thread per 16-byte chunk, numbered in shuffled order (contiguous on the shuffled side)
template <bool INVERSE>
__global__ __launch_bounds__(256) void shuffle_codes_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                            const int64_t chunks, const int64_t W) {
    const int64_t per_band = W; // 16 rows x W bytes = W chunks of 16 bytes
    for (int64_t s = blockIdx.x * 256L + threadIdx.x; s < chunks; s += gridDim.x * 256L) {
        const int64_t band = s / per_band, within = s - band * per_band;
        const int64_t kblk = within >> 5;      // 32-byte column block
        const int     half = (within >> 4) & 1;
        const int     r16  = within & 15;
        const int64_t plain = ((band * 16 + r16) * W + kblk * 32 + half * 16) >> 4;
        if constexpr (INVERSE)
            st128(out + plain * 16, ld128(in + s * 16));
        else
            st128(out + s * 16, ld128(in + plain * 16));
    }
}

// one thread per 4-byte word of the shuffled side: bytes (i4, i1) = (0,0) (0,1) (1,0) (1,1)
template <bool INVERSE>
__global__ __launch_bounds__(256) void shuffle_scale_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                            const int64_t B, const int64_t M, const int64_t Nn,
                                                            const int64_t Mp, const int64_t Np) {
    const int64_t tiles_n = Np >> 3, words_b = (Mp * Np) >> 2, words = B * words_b;
    for (int64_t d = blockIdx.x * 256L + threadIdx.x; d < words; d += gridDim.x * 256L) {
        const int64_t b = d / words_b, w = d - b * words_b;
        const int64_t tile = w >> 6;
        const int     i5 = (w >> 4) & 3, i2 = w & 15;
        const int64_t i0 = tile / tiles_n, i3 = tile - i0 * tiles_n;
        const uint8_t *src = in + b * (INVERSE ? Mp * Np : M * Nn);
        uint8_t       *dst = out + b * (INVERSE ? M * Nn : Mp * Np);
        uint32_t       word = INVERSE ? *reinterpret_cast<const uint32_t *>(src + w * 4) : 0u;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t row = i0 * 32 + (j & 1) * 16 + i2, col = i3 * 8 + (j >> 1) * 4 + i5;
            const bool    ok  = row < M && col < Nn;
            if constexpr (INVERSE) {
                if (ok)
                    dst[row * Nn + col] = static_cast<uint8_t>(word >> (8 * j));
            } else {
                word |= ok ? static_cast<uint32_t>(src[row * Nn + col]) << (8 * j) : 0u;
            }
        }
        if constexpr (!INVERSE)
            *reinterpret_cast<uint32_t *>(dst + w * 4) = word;
    }
}

static unsigned grid_for(int64_t items) {
    const int64_t want = cdiv(items, 256), cap = 64L * device_cu_count();
    return static_cast<unsigned>(want < cap ? (want > 0 ? want : 1) : cap);
}

} // namespace pt

using namespace pt;

extern "C" {

int pt_shuffle_mx_codes(const void *in, void *out, int64_t rows, int64_t row_bytes, int inverse, void *stream) {
    PT_REQUIRE(rows >= 0 && row_bytes >= 0, "dimensions must be non-negative");
    PT_REQUIRE(rows % 16 == 0, "rows must be divisible by 16 for the shuffled layout, got rows=" + std::to_string(rows));
    PT_REQUIRE(row_bytes % 32 == 0,
               "row bytes must be divisible by 32 for the shuffled layout, got " + std::to_string(row_bytes));
    if (rows == 0 || row_bytes == 0)
        return PT_OK;
    PT_REQUIRE(in && out && in != out, "NULL or aliased tensor pointer");
    PT_REQUIRE(aligned_to(in, 16) && aligned_to(out, 16), "tensors must be 16-byte aligned");
    const int64_t chunks = rows * row_bytes / 16;
    auto          st     = static_cast<hipStream_t>(stream);
    if (inverse)
        shuffle_codes_kernel<true><<<grid_for(chunks), 256, 0, st>>>(static_cast<const uint8_t *>(in),
                                                                     static_cast<uint8_t *>(out), chunks, row_bytes);
    else
        shuffle_codes_kernel<false><<<grid_for(chunks), 256, 0, st>>>(static_cast<const uint8_t *>(in),
                                                                      static_cast<uint8_t *>(out), chunks, row_bytes);
    return check_launch("shuffle_codes_kernel");
}

int pt_shuffle_e8m0_scale(const void *in, void *out, int64_t batch, int64_t M, int64_t N, int64_t M_pad, int64_t N_pad,
                          int inverse, void *stream) {
    PT_REQUIRE(batch >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    PT_REQUIRE(M_pad >= M && N_pad >= N && M_pad % 32 == 0 && N_pad % 8 == 0,
               "padded scale shape must cover [M, N] in whole 32 x 8 tiles");
    if (batch == 0 || M_pad == 0 || N_pad == 0)
        return PT_OK;
    PT_REQUIRE(in && out && in != out, "NULL or aliased tensor pointer");
    PT_REQUIRE(aligned_to(inverse ? in : out, 4), "the shuffled tensor must be 4-byte aligned");
    const int64_t words = batch * M_pad * N_pad / 4;
    auto          st    = static_cast<hipStream_t>(stream);
    if (inverse)
        shuffle_scale_kernel<true><<<grid_for(words), 256, 0, st>>>(static_cast<const uint8_t *>(in),
                                                                    static_cast<uint8_t *>(out), batch, M, N, M_pad, N_pad);
    else
        shuffle_scale_kernel<false><<<grid_for(words), 256, 0, st>>>(static_cast<const uint8_t *>(in),
                                                                     static_cast<uint8_t *>(out), batch, M, N, M_pad, N_pad);
    return check_launch("shuffle_scale_kernel");
}

} // extern "C"
