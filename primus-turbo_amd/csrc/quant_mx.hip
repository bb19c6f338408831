// MX (microscaling) quantizers and de-quantizers for gfx950: MXFP8 (E4M3 / E5M2) and MXFP4
// (E2M1), one E8M0 shared exponent per 32 elements.
//
// Numerics (Primus-Turbo's MX quantizers: flydsl/quantization/mxfp8_quant_flydsl.py:44-66,
// flydsl/quantization/mxfp4_quant_kernel.py:78-89,121-149; de-quantizers
// csrc/kernels/quantization/dequantization_mxfp8.cu:29-113, dequantization_mxfp4.cu:28-160):
//   amax  = max |x| over the block (NaN ignored)
//   e     = clamp((((bits(amax) + R) >> 23) & 0x1FF) - 127 - T, -127, 128)   (integers)
//           (R, T) = (1 << 19, 8) E4M3, (1 << 20, 15) E5M2, (1 << 21, 2) E2M1
//   scale byte = e + 127;  q = rne_sat(clamp(x * 2^-e, +-qmax))  (NaN -> +qmax)
//   FP4: element 2p in the low nibble, 2p + 1 in the high nibble of byte p
//   de-quantize: y = T(float(q) * bits_to_f32(byte << 23))
//
// One workgroup handles a 128 x 128 tile: it is read once into LDS (raw 16-bit), then
// quantized along rows (blocks of 32 columns) and/or along columns (blocks of 32 rows, output
// transposed), so the dual quantizer reads HBM once. The "2-D block" variants share one
// exponent per 32 x 32 tile.
#include "pt_activation.h"
#include "pt_common.h"

namespace pt {

enum : int { MX_E4M3 = 0, MX_E5M2 = 1, MX_E2M1 = 2 };

template <int FMT> struct MxFmt;
template <> struct MxFmt<MX_E4M3> {
    static constexpr uint32_t R = 1u << 19;
    static constexpr int      T = 8;
    static constexpr float    QMAX = 448.f;
};
template <> struct MxFmt<MX_E5M2> {
    static constexpr uint32_t R = 1u << 20;
    static constexpr int      T = 15;
    static constexpr float    QMAX = 57344.f;
};
template <> struct MxFmt<MX_E2M1> {
    static constexpr uint32_t R = 1u << 21;
    static constexpr int      T = 2;
    static constexpr float    QMAX = 6.f;
};

// shared exponent of a block (unbiased) from its abs-max
template <int FMT> __device__ __forceinline__ int mx_exponent(float amax) {
    const uint32_t b = __float_as_uint(amax);
    int            e = static_cast<int>(((b + MxFmt<FMT>::R) >> 23) & 0x1FFu) - 127 - MxFmt<FMT>::T;
    e                = e < -127 ? -127 : e;
    return e > 128 ? 128 : e;
}

// 2^-e as a float; e stays within [-127, 126] for every finite or infinite abs-max
__device__ __forceinline__ float mx_inv_scale(int e) {
    return __uint_as_float(static_cast<uint32_t>(127 - e) << 23);
}

// clamp(x * scale, +-qmax) in two instructions for an x that is not NaN (same value as scale_clamp)
__device__ __forceinline__ float scale_clamp_no_nan(float x, float scale, float qmax) {
    return __builtin_amdgcn_fmed3f(x * scale, -qmax, qmax);
}

// N scaled values (N = 8 or 32) -> packed codes. FP8: N / 4 dwords, FP4: N / 8 dwords. `no_nan`: the
// caller knows that no value is NaN (the short clamp serves).
template <int FMT, int N, int W> __device__ __forceinline__ void mx_encode(const float (&v)[N], float inv, uint32_t (&out)[W], bool no_nan) {
    constexpr float Q = MxFmt<FMT>::QMAX;
    if (no_nan) {
        if constexpr (FMT == MX_E2M1) {
#pragma unroll
            for (int d = 0; d < N / 8; ++d) {
                uint32_t w = 0;
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp_no_nan(v[8 * d + 0], inv, Q), scale_clamp_no_nan(v[8 * d + 1], inv, Q), 1.0f, 0);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp_no_nan(v[8 * d + 2], inv, Q), scale_clamp_no_nan(v[8 * d + 3], inv, Q), 1.0f, 1);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp_no_nan(v[8 * d + 4], inv, Q), scale_clamp_no_nan(v[8 * d + 5], inv, Q), 1.0f, 2);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp_no_nan(v[8 * d + 6], inv, Q), scale_clamp_no_nan(v[8 * d + 7], inv, Q), 1.0f, 3);
                out[d] = w;
            }
        } else {
#pragma unroll
            for (int d = 0; d < N / 4; ++d)
                out[d] = cvt4_fp8<FMT == MX_E5M2>(scale_clamp_no_nan(v[4 * d], inv, Q), scale_clamp_no_nan(v[4 * d + 1], inv, Q),
                                                  scale_clamp_no_nan(v[4 * d + 2], inv, Q), scale_clamp_no_nan(v[4 * d + 3], inv, Q));
        }
        return;
    }
    if constexpr (FMT == MX_E2M1) {
#pragma unroll
        for (int d = 0; d < N / 8; ++d) {
            uint32_t w = 0;
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp(v[8 * d + 0], inv, Q), scale_clamp(v[8 * d + 1], inv, Q), 1.0f, 0);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp(v[8 * d + 2], inv, Q), scale_clamp(v[8 * d + 3], inv, Q), 1.0f, 1);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp(v[8 * d + 4], inv, Q), scale_clamp(v[8 * d + 5], inv, Q), 1.0f, 2);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, scale_clamp(v[8 * d + 6], inv, Q), scale_clamp(v[8 * d + 7], inv, Q), 1.0f, 3);
            out[d] = w;
        }
    } else {
#pragma unroll
        for (int d = 0; d < N / 4; ++d)
            out[d] = cvt4_fp8<FMT == MX_E5M2>(scale_clamp(v[4 * d], inv, Q), scale_clamp(v[4 * d + 1], inv, Q),
                                              scale_clamp(v[4 * d + 2], inv, Q), scale_clamp(v[4 * d + 3], inv, Q));
    }
}

// The abs-max of 16-bit floats taken on their bit patterns, two at a time: with the sign bit
// cleared, floats order like unsigned integers. A NaN shows as a value above the infinity
// pattern; the caller then takes the abs-max that ignores NaN from the float values.
template <typename T> struct Bits16;
template <> struct Bits16<bf16_t> {
    static constexpr uint32_t INF = 0x7F80u;
    static __device__ __forceinline__ float to_f32(uint32_t b) { return __uint_as_float(b << 16); }
};
template <> struct Bits16<f16_t> {
    static constexpr uint32_t INF = 0x7C00u;
    static __device__ __forceinline__ float to_f32(uint32_t b) {
        return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(b)));
    }
};
__device__ __forceinline__ uint32_t pk_absmax16(uint32_t acc, uint32_t w) {
    typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, acc),
                                                                  __builtin_bit_cast(u16x2, w & 0x7FFF7FFFu)));
}

// Stochastic rounding (MXFP4 gradients): the hardware converter adds the seed's bits below the
// kept mantissa before truncating, so a value lands on its upper neighbour with a probability
// equal to its position between the two neighbours (unbiased; measured on uniform seeds). The
// scale stays the deterministic one. Every pair of values gets its own seed; the converter's
// destination bytes other than the selected one are not preserved, hence byte 0 and a mask.
// (Primus-Turbo's recipe: flydsl/quantization/mxfp4_quant_kernel.py:48-75,120-150.)
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t sr_hash(uint32_t s) {
    s = (s ^ 61u) ^ (s >> 16);
    s *= 9u;
    s ^= s >> 4;
    s *= 0x27D4EB2Du;
    s ^= s >> 15;
    return s;
}
__device__ __forceinline__ void mx_encode32_fp4_sr(const float (&v)[32], float inv, uint32_t seed, uint32_t (&out)[8]) {
    constexpr float Q = MxFmt<MX_E2M1>::QMAX;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        uint32_t w = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const f32x2_t pair = {scale_clamp(v[8 * d + 2 * k], inv, Q), scale_clamp(v[8 * d + 2 * k + 1], inv, Q)};
            seed += 0x9E3779B9u;
            const uint32_t b = __builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, pair, seed, 1.0f, 0) & 0xffu;
            w |= b << (8 * k);
        }
        out[d] = w;
    }
}

// A build for timing studies may define this to record a time stamp per workgroup and phase
#ifndef PT_MX_TRACE
#define PT_MX_TRACE(id)
#endif

constexpr int MX_TILE  = 128;
constexpr int MX_PITCH = MX_TILE + 8; // 16-bit elements per LDS row (272 B: 16-byte aligned rows)

struct MxArgs {
    const void *x; // [B, M, N] bf16 / fp16
    int64_t     B, M, N, Mpad, Npad;
    uint8_t    *row_q; // [B, M, Npad] (FP4: Npad / 2 bytes per row) or NULL
    uint8_t    *row_s; // [B, M, Npad / 32] or NULL
    uint8_t    *col_q; // [B, N, Mpad] (FP4: Mpad / 2) or NULL
    uint8_t    *col_s; // [B, N, Mpad / 32] or NULL
    // Grouped mode (B = 1, group_offs != NULL): the rows of x belong to G groups; the tile grid
    // runs over the row space in which every group is padded to a multiple of 128 rows
    // (col_offs_pad, Mpad = its allocated extent): the column-direction output lives there, pad
    // rows are zero data. The row-direction output puts the rows of group g at row_offs_pad[g]
    // (NULL: at their place in x); its pad rows are not written.
    const int64_t *group_offs;   // [G + 1]
    const int64_t *row_offs_pad; // [G + 1] or NULL
    const int64_t *col_offs_pad; // [G + 1]
    int            G;
    // MXFP4 stochastic rounding: bit 0 / bit 1 = row / column direction; one seed per launch
    int      sr_mask;
    uint32_t sr_seed;
    // Gated input (the GLU kernels): x is [M, 2 N], gate half then up half of every row; the
    // tile holds T(act(gate) * up * probs[m]), zeros for rows whose row_mask entry is 0.
    const float   *probs;    // [M]
    const int64_t *row_mask; // [M] or NULL
};

// The MXFP4 recipe's fixed 16-point Hadamard transform of v[base .. base + 16), in place:
// (H4 (x) H4) / 4 with the operation order of Primus-Turbo's
// primus_turbo/flydsl/quantization/mxfp4_quant_kernel.py:92-118 (an H4 butterfly inside each run
// of four, one across the four runs, then * 0.25). Additions only and one exact scaling: there is
// nothing here for the compiler to contract.
__device__ __forceinline__ void h4(float &v0, float &v1, float &v2, float &v3) {
    const float a0 = v0 + v1, a1 = v0 - v1, a2 = v2 + v3, a3 = v2 - v3;
    v0 = a0 + a2;
    v1 = a1 + a3;
    v2 = a0 - a2;
    v3 = a1 - a3;
}
__device__ __forceinline__ void hadamard16(float (&v)[32], int base) {
#pragma unroll
    for (int b = 0; b < 4; ++b)
        h4(v[base + 4 * b], v[base + 4 * b + 1], v[base + 4 * b + 2], v[base + 4 * b + 3]);
#pragma unroll
    for (int l = 0; l < 4; ++l) {
        h4(v[base + l], v[base + 4 + l], v[base + 8 + l], v[base + 12 + l]);
#pragma unroll
        for (int b = 0; b < 4; ++b)
            v[base + 4 * b + l] *= 0.25f;
    }
}

// fabsf(x) with NaN mapped to 0 (fmaxf-style abs-max ignores NaN)
__device__ __forceinline__ float abs_or_zero(float x) {
    const float a = fabsf(x);
    return a == a ? a : 0.f;
}

// RHT: bit 0 / bit 1 = the row / column direction quantizes the Hadamard-transformed values
// (16 consecutive elements along the direction; never together with 2-D blocks).
// GLU: 0 = x is the tile source itself; 1 + ACT_SILU / 1 + ACT_GELU = x holds gate and up halves
// and the tile is the gated activation, rounded to T as the stand-alone activation kernel rounds
// it (grouped mode only).
template <typename T, int FMT, bool ROW, bool COL, bool ROW2D, bool COL2D, int RHT = 0, int GLU = 0>
__global__ __launch_bounds__(256) void mx_quant_kernel(const MxArgs a) {
    constexpr bool ANY2D = (ROW && ROW2D) || (COL && COL2D);
    static_assert(RHT == 0 || !ANY2D, "the Hadamard transform is not combined with 2-D blocks");
    static_assert(GLU == 0 || !ANY2D, "the gated input is not combined with 2-D blocks");
    __shared__ __attribute__((aligned(16))) uint16_t tile[MX_TILE * MX_PITCH];
    __shared__ float                                 amax_rc[ANY2D ? MX_TILE * 4 : 1]; // [row][32-col block]
    __shared__ float                                 amax_blk[ROW && ROW2D ? 16 : 1];  // [32-row block][32-col block]
    __shared__ __attribute__((aligned(4))) uint8_t   sbytes[MX_TILE * 4]; // E8M0 bytes of the tile, [row or column][block]
    const int     tid = threadIdx.x;
    // (tile order: blocks of 8 x 8 tiles per XCD, see xcd_block_tile)
    uint32_t tile_x, tile_y;
    xcd_block_tile(tile_x, tile_y);
    const uint32_t tile_z = blockIdx.z, gx = gridDim.x, gy = gridDim.y;
    const uint32_t wg = (tile_z * gy + tile_y) * gx + tile_x; // the tile's number (batch, row tile, column tile)
    const int64_t  n0 = static_cast<int64_t>(tile_x) * MX_TILE, m0 = static_cast<int64_t>(tile_y) * MX_TILE;
    const int64_t  b  = tile_z;
    const uint16_t *x = static_cast<const uint16_t *>(a.x) + b * a.M * a.N;
    // tile row r holds input row in_m0 + r (while below in_end) and goes to row row_dst0 + r of
    // the row-direction output (while r < row_cnt: in the padded layout that includes the zero
    // rows that round the group up to a multiple of 32)
    int64_t in_m0 = m0, in_end = a.M, row_dst0 = b * a.M + m0, row_cnt = a.M - m0;
    if (a.group_offs != nullptr) {
        if (m0 >= a.col_offs_pad[a.G])
            return;
        const int g = find_group(a.col_offs_pad, a.G, m0);
        in_m0    = a.group_offs[g] + (m0 - a.col_offs_pad[g]);
        in_end   = a.group_offs[g + 1];
        const int64_t done = in_m0 - a.group_offs[g]; // rows of the group in earlier tiles
        row_dst0 = a.row_offs_pad != nullptr ? a.row_offs_pad[g] + done : in_m0;
        row_cnt  = (a.row_offs_pad != nullptr ? a.row_offs_pad[g + 1] - a.row_offs_pad[g] : in_end - a.group_offs[g]) - done;
    }

    PT_MX_TRACE(0);
    // (the row direction is taken from the registers of the loads where that is possible)
    constexpr bool EARLY_ROW = ROW && (RHT & 1) == 0;
    bool           row_done  = false;
    // ---- tile -> LDS (zeros outside the matrix) ----
    // Whole 16-byte pieces (the common case) are all requested before the first is used: a piece
    // outside the matrix reads the matrix's first bytes instead and is replaced by zeros, so that
    // no branch separates the loads.
    const bool vec = (a.N & 7) == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
    if (vec) {
        u32x4 piece[8];
        bool  inside[8];
        if constexpr (GLU != 0) {
            u32x4   up[8];
            float   pr[8];
            int64_t ms[8];
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const int     r = p * 16 + (tid >> 4), c = (tid & 15) * 8;
                const int64_t m = in_m0 + r, n = n0 + c;
                inside[p]       = m < in_end && n < a.N;
                ms[p]           = inside[p] ? m : 0;
                const uint16_t *gp = static_cast<const uint16_t *>(a.x) + ms[p] * 2 * a.N + (inside[p] ? n : 0);
                piece[p]           = ld128_nt(gp);
                up[p]              = ld128_nt(gp + a.N);
                pr[p]              = a.probs[ms[p]];
            }
            if (a.row_mask != nullptr) {
                int64_t keep[8];
#pragma unroll
                for (int p = 0; p < 8; ++p)
                    keep[p] = a.row_mask[ms[p]];
#pragma unroll
                for (int p = 0; p < 8; ++p)
                    inside[p] = inside[p] && keep[p] != 0;
            }
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const uint32_t gw[4] = {piece[p].x, piece[p].y, piece[p].z, piece[p].w};
                const uint32_t uw[4] = {up[p].x, up[p].y, up[p].z, up[p].w};
                uint32_t       o[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float g0, g1, u0, u1;
                    unpack2<T>(gw[k], g0, g1);
                    unpack2<T>(uw[k], u0, u1);
                    o[k] = pack2<T>(act_fwd<GLU - 1>(g0) * u0 * pr[p], act_fwd<GLU - 1>(g1) * u1 * pr[p]);
                }
                piece[p] = u32x4{o[0], o[1], o[2], o[3]};
            }
        } else {
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const int     r = p * 16 + (tid >> 4), c = (tid & 15) * 8;
                const int64_t m = in_m0 + r, n = n0 + c;
                inside[p]       = m < in_end && n < a.N;
                piece[p]        = ld128_nt(x + (inside[p] ? m * a.N + n : 0));
            }
        }
#pragma unroll
        for (int p = 0; p < 8; ++p)
            piece[p] = inside[p] ? piece[p] : u32x4{0u, 0u, 0u, 0u};
        // The row direction with 1-D blocks needs no transposition: it is encoded straight from the
        // registers the loads arrived in (a lane holds a quarter of a block, the block's abs-max is
        // a reduction over four neighbouring lanes), 8 code bytes per lane and 128 per row segment.
        if constexpr (EARLY_ROW) {
            float am8[8];  // abs-max of this lane's block in piece p (the same in the four lanes of a block)
            bool  nan8[8]; // a NaN somewhere in that block
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const uint32_t ww[4] = {piece[p].x, piece[p].y, piece[p].z, piece[p].w};
                uint32_t       m2 = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    m2 = pk_absmax16(m2, ww[i]);
                uint32_t m16 = max(m2 & 0xffffu, m2 >> 16);
                m16          = max(m16, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, m16, 0xB1, 0xf, 0xf, true)));
                m16          = max(m16, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, m16, 0x4E, 0xf, 0xf, true)));
                nan8[p]      = m16 > Bits16<T>::INF;
                float am     = Bits16<T>::to_f32(m16);
                if (nan8[p]) {
                    am = 0.f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float f0, f1;
                        unpack2<T>(ww[i], f0, f1);
                        am = fmaxf(am, fmaxf(abs_or_zero(f0), abs_or_zero(f1)));
                    }
                    am = fmaxf(am, dpp_f32<0xB1>(am));
                    am = fmaxf(am, dpp_f32<0x4E>(am));
                }
                am8[p] = am;
                if constexpr (ANY2D)
                    if ((tid & 3) == 0)
                        amax_rc[(p * 16 + (tid >> 4)) * 4 + ((tid & 15) >> 2)] = am;
            }
            if constexpr (ROW2D) {
                // the 16 blocks of 32 x 32: sixteen lanes reduce the 32 row values of one block
                __syncthreads();
                {
                    const int blk = tid >> 4, rb = blk >> 2, cb = blk & 3, i = (tid & 15) * 2;
                    const float m = row16_max(fmaxf(amax_rc[(rb * 32 + i) * 4 + cb], amax_rc[(rb * 32 + i + 1) * 4 + cb]));
                    if ((tid & 15) == 0)
                        amax_blk[blk] = m;
                }
                __syncthreads();
#pragma unroll
                for (int p = 0; p < 8; ++p)
                    am8[p] = amax_blk[((p * 16 + (tid >> 4)) >> 5) * 4 + ((tid & 15) >> 2)];
            }
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const int      r = p * 16 + (tid >> 4), cb = (tid & 15) >> 2; // tile row, 32-column block
                const uint32_t ww[4] = {piece[p].x, piece[p].y, piece[p].z, piece[p].w};
                float          f[8];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    unpack2<T>(ww[i], f[2 * i], f[2 * i + 1]);
                const bool  nan = nan8[p];
                const int   e   = mx_exponent<FMT>(am8[p]);
                const float inv = mx_inv_scale(e);
                if ((tid & 3) == 0)
                    sbytes[r * 4 + cb] = static_cast<uint8_t>(e + 127);
                const int64_t n = n0 + (tid & 15) * 8;
                if constexpr (FMT == MX_E2M1) {
                    uint32_t w = 0;
                    if (a.sr_mask & 1) {
                        // the seeds of the LDS row pass: task 4 r + cb of this tile, one step per pair
                        constexpr float Q = MxFmt<MX_E2M1>::QMAX;
                        uint32_t seed = sr_hash(a.sr_seed ^ (wg * 512u + static_cast<uint32_t>(r * 4 + cb))) + 4u * (tid & 3) * 0x9E3779B9u;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const f32x2_t pair = {scale_clamp(f[2 * i], inv, Q), scale_clamp(f[2 * i + 1], inv, Q)};
                            seed += 0x9E3779B9u;
                            w |= (__builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, pair, seed, 1.0f, 0) & 0xffu) << (8 * i);
                        }
                    } else {
                        uint32_t c[1];
                        mx_encode<FMT>(f, inv, c, !nan);
                        w = c[0];
                    }
                    if (r < row_cnt)
                        st32_nt(a.row_q + (row_dst0 + r) * (a.Npad >> 1) + (n >> 1), w);
                } else {
                    uint32_t c[2];
                    mx_encode<FMT>(f, inv, c, !nan);
                    if (r < row_cnt)
                        st64_nt(a.row_q + (row_dst0 + r) * a.Npad + n, u32x2{c[0], c[1]});
                }
            }
            row_done = true;
        }
        if constexpr (COL || !EARLY_ROW) {
#pragma unroll
            for (int p = 0; p < 8; ++p) {
                const int r = p * 16 + (tid >> 4), c = (tid & 15) * 8;
                *reinterpret_cast<u32x4 *>(&tile[r * MX_PITCH + c]) = piece[p];
            }
        }
    } else {
#pragma unroll 1
        for (int p = 0; p < 8; ++p) {
            const int     r = p * 16 + (tid >> 4), c = (tid & 15) * 8;
            const int64_t m = in_m0 + r, n = n0 + c;
            u32x4         v = u32x4{0u, 0u, 0u, 0u};
            if constexpr (GLU != 0) {
                if (m < in_end && n < a.N && (a.row_mask == nullptr || a.row_mask[m] != 0)) {
                    const uint16_t *gp = static_cast<const uint16_t *>(a.x) + m * 2 * a.N + n;
                    const float     pr = a.probs[m];
                    uint32_t        gw[4] = {0u, 0u, 0u, 0u}, uw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        if (n + k < a.N) {
                            gw[k >> 1] |= static_cast<uint32_t>(gp[k]) << (16 * (k & 1));
                            uw[k >> 1] |= static_cast<uint32_t>(gp[a.N + k]) << (16 * (k & 1));
                        }
                    uint32_t o[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        float g0, g1, u0, u1;
                        unpack2<T>(gw[k], g0, g1);
                        unpack2<T>(uw[k], u0, u1);
                        // columns behind N stay +0 whatever probs holds
                        const float r0 = n + 2 * k < a.N ? act_fwd<GLU - 1>(g0) * u0 * pr : 0.f;
                        const float r1 = n + 2 * k + 1 < a.N ? act_fwd<GLU - 1>(g1) * u1 * pr : 0.f;
                        o[k]           = pack2<T>(r0, r1);
                    }
                    v = u32x4{o[0], o[1], o[2], o[3]};
                }
            } else if (m < in_end && n < a.N) {
                uint16_t e[8];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    e[k] = n + k < a.N ? x[m * a.N + n + k] : uint16_t(0);
                v = u32x4{e[0] | (uint32_t(e[1]) << 16), e[2] | (uint32_t(e[3]) << 16), e[4] | (uint32_t(e[5]) << 16),
                          e[6] | (uint32_t(e[7]) << 16)};
            }
            *reinterpret_cast<u32x4 *>(&tile[r * MX_PITCH + c]) = v;
        }
    }
    PT_MX_TRACE(1);
    __syncthreads();
    PT_MX_TRACE(2);

    // ---- row direction: task = (row r, 32-column block c) ----
    float rv[2][32];
    float ram[2];
    bool  rnan[2] = {true, true}; // false: the task's 32 input values are known to hold no NaN
    if constexpr (ROW || ANY2D) {
        if (!row_done) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int t = tid + 256 * p, r = t >> 2, c = t & 3;
            uint32_t  m2 = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u32x4    w    = *reinterpret_cast<const u32x4 *>(&tile[r * MX_PITCH + c * 32 + q * 8]);
                const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    unpack2<T>(ww[k], rv[p][q * 8 + 2 * k], rv[p][q * 8 + 2 * k + 1]);
                    m2 = pk_absmax16(m2, ww[k]);
                }
            }
            const uint32_t m16 = max(m2 & 0xffffu, m2 >> 16);
            rnan[p]            = m16 > Bits16<T>::INF;
            float am           = Bits16<T>::to_f32(m16);
            if constexpr ((RHT & 1) != 0) {
                hadamard16(rv[p], 0);
                hadamard16(rv[p], 16);
                rnan[p] = true; // the transformed values are not looked at
            }
            if (rnan[p]) {
                am = 0.f;
#pragma unroll
                for (int k = 0; k < 32; ++k)
                    am = fmaxf(am, abs_or_zero(rv[p][k]));
            }
            ram[p] = am;
            if constexpr (ANY2D)
                amax_rc[r * 4 + c] = am;
        }
        } // the row pass through the LDS
    }
    if constexpr (ANY2D)
        __syncthreads();
    if constexpr (ROW) {
        if (!row_done) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int     t = tid + 256 * p, r = t >> 2, c = t & 3;
            float         am = ram[p];
            if constexpr (ROW2D) {
                const int rb = r & ~31;
                am           = 0.f;
#pragma unroll 8
                for (int i = 0; i < 32; ++i)
                    am = fmaxf(am, amax_rc[(rb + i) * 4 + c]);
            }
            const int e = mx_exponent<FMT>(am);
            uint32_t  code[8];
            if (FMT == MX_E2M1 && (a.sr_mask & 1)) {
                // a seed per 32-element block: launch seed, tile and task mixed
                const uint32_t id = wg; // the tile's number (batch, row tile, column tile)
                mx_encode32_fp4_sr(rv[p], mx_inv_scale(e), sr_hash(a.sr_seed ^ (id * 512u + t)), code);
            } else {
                mx_encode<FMT>(rv[p], mx_inv_scale(e), code, !rnan[p]);
            }
            sbytes[r * 4 + c] = static_cast<uint8_t>(e + 127);
            if (r < row_cnt) {
                const int64_t nb = (n0 >> 5) + c; // 32-column block index in the padded row
                if constexpr (FMT == MX_E2M1) {
                    uint8_t *q = a.row_q + (row_dst0 + r) * (a.Npad >> 1) + nb * 16;
                    st128(q, u32x4{code[0], code[1], code[2], code[3]});
                } else {
                    uint8_t *q = a.row_q + (row_dst0 + r) * a.Npad + nb * 32;
                    st128(q, u32x4{code[0], code[1], code[2], code[3]});
                    st128(q + 16, u32x4{code[4], code[5], code[6], code[7]});
                }
            }
        }
        __syncthreads();
        } // the row pass through the LDS
        // the four scale bytes of a tile row leave as one word (Npad / 32 is a multiple of 4)
        if (tid < MX_TILE && tid < row_cnt)
            *reinterpret_cast<uint32_t *>(a.row_s + (row_dst0 + tid) * (a.Npad >> 5) + (n0 >> 5)) =
                *reinterpret_cast<const uint32_t *>(&sbytes[tid * 4]);
    }

    PT_MX_TRACE(3);
    // ---- column direction: task = (column n, 32-row block rb); output transposed ----
    // The codes go back through the LDS (over the input tile, once everybody has read it) so that
    // they leave as whole 128-byte (FP4: 64-byte) rows of the transposed output.
    if constexpr (COL) {
        constexpr int CB    = FMT == MX_E2M1 ? 16 : 32;   // code bytes per 32-row block
        constexpr int CROW  = 4 * CB;                     // code bytes per output row of the tile
        constexpr int CPITCH = CROW + 16;                 // LDS pitch of an output row
        static_assert(MX_TILE * CPITCH <= MX_TILE * MX_PITCH * 2, "the staged codes fit over the input tile");
        uint32_t code[2][8];
        if constexpr (ROW)
            __syncthreads(); // the row pass's scale bytes have been read
        // a thread owns two neighbouring columns of one 32-row block: one 32-bit LDS read per row
        // serves both (task p: column c, numbered t = 128 rb + c as the seeds of stochastic rounding expect)
        const int rb = tid >> 6, c0 = (tid & 63) * 2;
        float     v2[2][32];
        uint32_t  m2 = 0; // low half: column c0, high half: column c0 + 1
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const uint32_t w = *reinterpret_cast<const uint32_t *>(&tile[(rb * 32 + i) * MX_PITCH + c0]);
            unpack2<T>(w, v2[0][i], v2[1][i]);
            m2 = pk_absmax16(m2, w);
        }
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int c = c0 + p, t = 128 * rb + c;
            float (&v)[32] = v2[p];
            const uint32_t m16 = p == 0 ? (m2 & 0xffffu) : (m2 >> 16);
            bool           cnan = m16 > Bits16<T>::INF;
            float          am   = Bits16<T>::to_f32(m16);
            if constexpr ((RHT & 2) != 0) {
                hadamard16(v, 0);
                hadamard16(v, 16);
                cnan = true; // the transformed values are not looked at
            }
            if (cnan) {
                am = 0.f;
#pragma unroll
                for (int i = 0; i < 32; ++i)
                    am = fmaxf(am, abs_or_zero(v[i]));
            }
            if constexpr (COL2D) {
                if (ROW && ROW2D && row_done) { // the register row pass has left the blocks' maxima
                    am = amax_blk[rb * 4 + (c >> 5)];
                } else {
                    am = 0.f;
#pragma unroll 8
                    for (int i = 0; i < 32; ++i)
                        am = fmaxf(am, amax_rc[(rb * 32 + i) * 4 + (c >> 5)]);
                }
            }
            const int e = mx_exponent<FMT>(am);
            if (FMT == MX_E2M1 && (a.sr_mask & 2)) {
                const uint32_t id = wg; // the tile's number (batch, row tile, column tile)
                mx_encode32_fp4_sr(v, mx_inv_scale(e), sr_hash(a.sr_seed ^ 0x5BD1E995u ^ (id * 512u + t)), code[p]);
            } else {
                mx_encode<FMT>(v, mx_inv_scale(e), code[p], !cnan);
            }
            sbytes[c * 4 + rb] = static_cast<uint8_t>(e + 127);
        }
        PT_MX_TRACE(4);
        __syncthreads(); // everybody is done with the input tile
        PT_MX_TRACE(5);
        uint8_t *stage = reinterpret_cast<uint8_t *>(tile);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int c = c0 + p;
            uint8_t  *d = stage + c * CPITCH + rb * CB;
            *reinterpret_cast<u32x4 *>(d) = u32x4{code[p][0], code[p][1], code[p][2], code[p][3]};
            if constexpr (FMT != MX_E2M1)
                *reinterpret_cast<u32x4 *>(d + 16) = u32x4{code[p][4], code[p][5], code[p][6], code[p][7]};
        }
        __syncthreads();
        PT_MX_TRACE(6);
        constexpr int CHUNKS = CROW / 16; // 16-byte chunks per output row
#pragma unroll
        for (int p = 0; p < MX_TILE * CHUNKS / 256; ++p) {
            const int     k = tid + 256 * p, c = k / CHUNKS, ch = k % CHUNKS;
            const int64_t n = n0 + c;
            if (n < a.N) {
                const u32x4 w = *reinterpret_cast<const u32x4 *>(stage + c * CPITCH + ch * 16);
                uint8_t    *q = a.col_q + (b * a.N + n) * (FMT == MX_E2M1 ? a.Mpad >> 1 : a.Mpad) + (m0 >> 5) * CB + ch * 16;
                st128(q, w);
            }
        }
        if (tid < MX_TILE && n0 + tid < a.N)
            *reinterpret_cast<uint32_t *>(a.col_s + (b * a.N + n0 + tid) * (a.Mpad >> 5) + (m0 >> 5)) =
                *reinterpret_cast<const uint32_t *>(&sbytes[tid * 4]);
    }
    PT_MX_TRACE(7);
}

// Row direction only, 1-D blocks, nearest or stochastic rounding, rows of whole 16-byte pieces: a
// plain stream without LDS, same bytes as the tile kernel. The padded rows are cut into runs of
// 512 columns; a wavefront takes four consecutive runs, a lane 8 consecutive elements of each (a
// quarter of a block: the block's abs-max is a reduction over four neighbouring lanes). The 64
// scale bytes of a wavefront leave as 16 words.
template <typename T, int FMT>
__global__ __launch_bounds__(256) void mx_quant_rows_kernel(const MxArgs a, const int64_t rows, const int64_t runs_per_row) {
    const int     lane  = threadIdx.x & 63;
    const int64_t total = rows * runs_per_row;
    const int64_t u0    = (static_cast<int64_t>(blockIdx.x) * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6)) * 4;
    if (u0 >= total)
        return;
    const uint16_t *x = static_cast<const uint16_t *>(a.x);
    int64_t         row[4], run[4];
    row[0] = u0 / runs_per_row;
    run[0] = u0 - row[0] * runs_per_row;
#pragma unroll
    for (int k = 1; k < 4; ++k) {
        const bool wrap = run[k - 1] + 1 == runs_per_row;
        row[k]          = wrap ? row[k - 1] + 1 : row[k - 1];
        run[k]          = wrap ? 0 : run[k - 1] + 1;
    }
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int64_t n = run[k] * 512 + lane * 8;
        v[k]            = (u0 + k < total && n < a.N) ? ld128_nt(x + row[k] * a.N + n) : u32x4{0u, 0u, 0u, 0u};
    }
    uint32_t ebytes = 0; // byte k: the scale byte of this lane's block in run k
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t ww[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        float          f[8];
        uint32_t       m2 = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            unpack2<T>(ww[i], f[2 * i], f[2 * i + 1]);
            m2 = pk_absmax16(m2, ww[i]);
        }
        // the block's abs-max: over the four lanes of the quad (quad_perm [1,0,3,2], then [2,3,0,1])
        uint32_t m16 = max(m2 & 0xffffu, m2 >> 16);
        m16          = max(m16, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, m16, 0xB1, 0xf, 0xf, true)));
        m16          = max(m16, static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, m16, 0x4E, 0xf, 0xf, true)));
        const bool nan = m16 > Bits16<T>::INF; // somewhere in the block
        float      am  = Bits16<T>::to_f32(m16);
        if (nan) {
            am = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                am = fmaxf(am, abs_or_zero(f[i]));
            am = fmaxf(am, dpp_f32<0xB1>(am));
            am = fmaxf(am, dpp_f32<0x4E>(am));
        }
        const int   e   = mx_exponent<FMT>(am);
        const float inv = mx_inv_scale(e);
        ebytes |= static_cast<uint32_t>(e + 127) << (8 * k);
        constexpr float Q = MxFmt<FMT>::QMAX;
        const int64_t   n = run[k] * 512 + lane * 8;
        const bool      in = u0 + k < total && n < a.Npad;
        if constexpr (FMT == MX_E2M1) {
            uint32_t w = 0;
            if (a.sr_mask & 1) {
                // the seeds of the tile kernel: tile (batch, row tile, column tile), task 4 r + c
                // of the tile, then one step per pair of the block
                const int64_t  m  = row[k] % a.M, bt = row[k] / a.M, nb = n >> 5;
                const uint32_t id = static_cast<uint32_t>((bt * (a.Mpad >> 7) + (m >> 7)) * (a.Npad >> 7) + (nb >> 2));
                const uint32_t t  = static_cast<uint32_t>((m & 127) * 4 + (nb & 3));
                uint32_t seed = sr_hash(a.sr_seed ^ (id * 512u + t)) + 4u * (lane & 3) * 0x9E3779B9u;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const f32x2_t pair = {scale_clamp(f[2 * i], inv, Q), scale_clamp(f[2 * i + 1], inv, Q)};
                    seed += 0x9E3779B9u;
                    w |= (__builtin_amdgcn_cvt_scalef32_sr_pk_fp4_f32(0u, pair, seed, 1.0f, 0) & 0xffu) << (8 * i);
                }
            } else {
                uint32_t c[1];
                mx_encode<FMT>(f, inv, c, !nan);
                w = c[0];
            }
            if (in)
                st32_nt(a.row_q + row[k] * (a.Npad >> 1) + (n >> 1), w);
        } else {
            uint32_t c[2];
            mx_encode<FMT>(f, inv, c, !nan);
            if (in)
                st64_nt(a.row_q + row[k] * a.Npad + n, u32x2{c[0], c[1]});
        }
    }
    // lane L < 16 writes scale word L & 3 of run L >> 2: the bytes of the blocks 4 (L & 3) .. + 3 of
    // that run, which the lanes 16 (L & 3) + 4 j hold
    uint32_t word = 0;
    const int k_of = (lane >> 2) & 3, j0 = lane & 3;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t wj = static_cast<uint32_t>(__shfl(static_cast<int>(ebytes), 16 * j0 + 4 * j, 64));
        word |= ((wj >> (8 * k_of)) & 0xffu) << (8 * j);
    }
    if (lane < 16) {
        int64_t r = row[0], c = run[0];
#pragma unroll
        for (int k = 1; k < 4; ++k)
            if (k_of == k)
                r = row[k], c = run[k];
        const int64_t sb = c * 16 + j0 * 4; // scale byte index in the padded row
        if (u0 + k_of < total && sb < (a.Npad >> 5))
            *reinterpret_cast<uint32_t *>(a.row_s + r * (a.Npad >> 5) + sb) = word;
    }
}

// The streaming row kernel serves an ungrouped launch when only the row direction is asked for,
// with 1-D blocks and no transform, and the rows are whole 16-byte pieces.
static bool mx_rows_stream_ok(const MxArgs &a, bool row2d, bool rht) {
    return a.col_q == nullptr && a.row_q != nullptr && !row2d && !rht && (a.N & 7) == 0 &&
           (reinterpret_cast<uintptr_t>(a.x) & 15) == 0 && a.group_offs == nullptr;
}
template <typename T> static void launch_mx_rows(const MxArgs &a, int fmt, hipStream_t st) {
    const int64_t rows = a.B * a.M, runs = cdiv(a.Npad, 512);
    const dim3    grid(static_cast<unsigned>(cdiv(rows * runs, 16)));
    if (fmt == MX_E4M3)
        mx_quant_rows_kernel<T, MX_E4M3><<<grid, 256, 0, st>>>(a, rows, runs);
    else if (fmt == MX_E5M2)
        mx_quant_rows_kernel<T, MX_E5M2><<<grid, 256, 0, st>>>(a, rows, runs);
    else
        mx_quant_rows_kernel<T, MX_E2M1><<<grid, 256, 0, st>>>(a, rows, runs);
}

template <typename T, int FMT, bool ROW, bool COL>
static void launch_mx_2d(const MxArgs &a, bool row2d, bool col2d, dim3 grid, hipStream_t st) {
    if (row2d && col2d)
        mx_quant_kernel<T, FMT, ROW, COL, ROW, COL><<<grid, 256, 0, st>>>(a);
    else if (row2d)
        mx_quant_kernel<T, FMT, ROW, COL, ROW, false><<<grid, 256, 0, st>>>(a);
    else if (col2d)
        mx_quant_kernel<T, FMT, ROW, COL, false, COL><<<grid, 256, 0, st>>>(a);
    else
        mx_quant_kernel<T, FMT, ROW, COL, false, false><<<grid, 256, 0, st>>>(a);
}

template <typename T, int FMT>
static void launch_mx_dir(const MxArgs &a, bool row2d, bool col2d, dim3 grid, hipStream_t st) {
    const bool row = a.row_q != nullptr, col = a.col_q != nullptr;
    if (row && col)
        launch_mx_2d<T, FMT, true, true>(a, row2d, col2d, grid, st);
    else if (row)
        launch_mx_2d<T, FMT, true, false>(a, row2d, false, grid, st);
    else
        launch_mx_2d<T, FMT, false, true>(a, false, col2d, grid, st);
}

// MXFP4 with the Hadamard transform in one or both directions (1-D blocks only)
template <typename T> static void launch_mx_rht(const MxArgs &a, bool row_rht, bool col_rht, dim3 grid, hipStream_t st) {
    const bool row = a.row_q != nullptr, col = a.col_q != nullptr;
    if (row && col) {
        if (row_rht && col_rht)
            mx_quant_kernel<T, MX_E2M1, true, true, false, false, 3><<<grid, 256, 0, st>>>(a);
        else if (col_rht)
            mx_quant_kernel<T, MX_E2M1, true, true, false, false, 2><<<grid, 256, 0, st>>>(a);
        else
            mx_quant_kernel<T, MX_E2M1, true, true, false, false, 1><<<grid, 256, 0, st>>>(a);
    } else if (row) {
        mx_quant_kernel<T, MX_E2M1, true, false, false, false, 1><<<grid, 256, 0, st>>>(a);
    } else {
        mx_quant_kernel<T, MX_E2M1, false, true, false, false, 2><<<grid, 256, 0, st>>>(a);
    }
}

// the gated-input quantizers: 1-D blocks, nearest rounding, both directions or rows only; MXFP4
// may transform its column direction (the recipe of the wgrad operand)
template <typename T, int FMT, int GLU> static void launch_mx_glu_dir(const MxArgs &a, bool col_rht, dim3 grid, hipStream_t st) {
    if constexpr (FMT == MX_E2M1) {
        if (a.col_q != nullptr && col_rht) {
            mx_quant_kernel<T, FMT, true, true, false, false, 2, GLU><<<grid, 256, 0, st>>>(a);
            return;
        }
    }
    if (a.col_q != nullptr)
        mx_quant_kernel<T, FMT, true, true, false, false, 0, GLU><<<grid, 256, 0, st>>>(a);
    else
        mx_quant_kernel<T, FMT, true, false, false, false, 0, GLU><<<grid, 256, 0, st>>>(a);
}
template <typename T, int GLU> static void launch_mx_glu(const MxArgs &a, int fmt, bool col_rht, dim3 grid, hipStream_t st) {
    if (fmt == MX_E4M3)
        launch_mx_glu_dir<T, MX_E4M3, GLU>(a, col_rht, grid, st);
    else if (fmt == MX_E5M2)
        launch_mx_glu_dir<T, MX_E5M2, GLU>(a, col_rht, grid, st);
    else
        launch_mx_glu_dir<T, MX_E2M1, GLU>(a, col_rht, grid, st);
}

template <typename T> static void launch_mx_fmt(const MxArgs &a, int fmt, bool row2d, bool col2d, dim3 grid, hipStream_t st) {
    if (fmt == MX_E4M3)
        launch_mx_dir<T, MX_E4M3>(a, row2d, col2d, grid, st);
    else if (fmt == MX_E5M2)
        launch_mx_dir<T, MX_E5M2>(a, row2d, col2d, grid, st);
    else
        launch_mx_dir<T, MX_E2M1>(a, row2d, col2d, grid, st);
}

// ---------------------------------------------------------------------------
// de-quantize: q [rows, cols] codes (FP4 packed) with scales [rows, cols / 32]
//   -> y [rows, cols], or y [cols, rows] when `transpose` (column-direction data)
// One workgroup per 64 x 64 tile through LDS so that both layouts store whole lines.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float e2m1_to_f32(uint32_t nib) {
    // E2M1: 1 sign, 2 exponent, 1 mantissa bits: {0, .5, 1, 1.5, 2, 3, 4, 6}
    const uint32_t mag = nib & 7u;
    const float    f   = mag < 2 ? 0.5f * mag : __uint_as_float(((126u + (mag >> 1)) << 23) | ((mag & 1u) << 22));
    return nib & 8u ? -f : f;
}

template <typename T, int FMT>
__global__ __launch_bounds__(256) void mx_dequant_kernel(const uint8_t *__restrict__ q, const uint8_t *__restrict__ s,
                                                         T *__restrict__ y, const int64_t rows, const int64_t cols,
                                                         const int transpose) {
    __shared__ float t[64][65];
    const int64_t    r0 = static_cast<int64_t>(blockIdx.y) * 64, c0 = static_cast<int64_t>(blockIdx.x) * 64;
    const int        tx = threadIdx.x & 15, ty = threadIdx.x >> 4; // thread: row ty + 16 p, columns 4 tx .. 4 tx + 3
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     r  = ty + 16 * p;
        const int64_t gr = r0 + r, gc = c0 + tx * 4;
        float         v[4] = {0.f, 0.f, 0.f, 0.f};
        if (gr < rows && gc < cols) { // cols is a multiple of 32: a group of 4 is all in or all out
            const float sc = __uint_as_float(static_cast<uint32_t>(s[gr * (cols >> 5) + (gc >> 5)]) << 23);
            if constexpr (FMT == MX_E2M1) {
                const uint16_t w = *reinterpret_cast<const uint16_t *>(q + gr * (cols >> 1) + (gc >> 1));
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v[k] = e2m1_to_f32((w >> (4 * k)) & 0xFu) * sc;
                }
            } else {
                const uint32_t w = *reinterpret_cast<const uint32_t *>(q + gr * cols + gc);
                v[0] = fp8_to_f32<FMT == MX_E5M2>(w, 0) * sc;
                v[1] = fp8_to_f32<FMT == MX_E5M2>(w, 1) * sc;
                v[2] = fp8_to_f32<FMT == MX_E5M2>(w, 2) * sc;
                v[3] = fp8_to_f32<FMT == MX_E5M2>(w, 3) * sc;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
            t[r][tx * 4 + k] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int r = ty + 16 * p; // output row within the tile
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int c = tx * 4 + k;
            if (!transpose) {
                if (r0 + r < rows && c0 + c < cols)
                    y[(r0 + r) * cols + c0 + c] = HP<T>::from_f32(t[r][c]);
            } else {
                if (c0 + r < cols && r0 + c < rows)
                    y[(c0 + r) * rows + r0 + c] = HP<T>::from_f32(t[c][r]);
            }
        }
    }
}

// Row-direction data with 16-byte aligned pointers: a plain stream. A thread takes 8 consecutive
// elements of a row (a quarter of a block, one scale byte): 8 (FP4: 4) code bytes in, 16 or 32
// bytes out, whole lines per wavefront on both sides; four such pieces per round, all of them
// requested before the first is used. `per_row_shift`: log2 of the pieces per row, or -1.
template <typename T, int FMT>
__global__ __launch_bounds__(256) void mx_dequant_stream_kernel(const uint8_t *__restrict__ q, const uint8_t *__restrict__ s,
                                                                T *__restrict__ y, const int64_t rows, const int64_t cols,
                                                                const int per_row_shift) {
    const int64_t per_row = cols >> 3, units = rows * per_row;
    const int64_t stride  = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t u0 = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; u0 < units; u0 += 4 * stride) {
        uint32_t code[4][2];
        uint32_t sbyte[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t u = u0 + k * stride < units ? u0 + k * stride : u0; // (a piece behind the end re-reads the first)
            const int64_t r = per_row_shift >= 0 ? u >> per_row_shift : u / per_row, c = u - r * per_row;
            sbyte[k]        = s[r * (cols >> 5) + (c >> 2)];
            if constexpr (FMT == MX_E2M1) {
                code[k][0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(q + (u << 2)));
                code[k][1] = 0;
            } else {
                const u32x2 w = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(q + (u << 3)));
                code[k][0] = w.x, code[k][1] = w.y;
            }
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t u = u0 + k * stride;
            if (u >= units)
                break;
            const float sc = __uint_as_float(sbyte[k] << 23);
            float       f[8];
            if constexpr (FMT == MX_E2M1) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    f[i] = e2m1_to_f32(code[k][0] >> (4 * i)) * sc;
            } else {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    f[4 * i + 0] = fp8_to_f32<FMT == MX_E5M2>(code[k][i], 0) * sc;
                    f[4 * i + 1] = fp8_to_f32<FMT == MX_E5M2>(code[k][i], 1) * sc;
                    f[4 * i + 2] = fp8_to_f32<FMT == MX_E5M2>(code[k][i], 2) * sc;
                    f[4 * i + 3] = fp8_to_f32<FMT == MX_E5M2>(code[k][i], 3) * sc;
                }
            }
            char *dst = reinterpret_cast<char *>(y + (u << 3));
            if constexpr (sizeof(T) == 4) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    st128_nt(dst + 16 * i, u32x4{__float_as_uint(f[4 * i]), __float_as_uint(f[4 * i + 1]),
                                              __float_as_uint(f[4 * i + 2]), __float_as_uint(f[4 * i + 3])});
            } else {
                st128_nt(dst, u32x4{pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])});
            }
        }
    }
}

template <typename T, int FMT>
static void launch_mx_dequant_t(const uint8_t *q, const uint8_t *s, T *y, int64_t rows, int64_t cols, int transpose,
                                hipStream_t st) {
    if (!transpose && aligned_to(q, 16) && aligned_to(y, 16)) {
        const int64_t units = rows * (cols >> 3), per_row = cols >> 3;
        int64_t       grid  = cdiv(units, 4 * 256);
        const int64_t cap   = 32L * device_cu_count();
        grid                = grid > cap ? cap : grid;
        int shift = -1;
        if ((per_row & (per_row - 1)) == 0)
            for (shift = 0; (int64_t{1} << shift) < per_row; ++shift) {
            }
        mx_dequant_stream_kernel<T, FMT><<<static_cast<unsigned>(grid), 256, 0, st>>>(q, s, y, rows, cols, shift);
        return;
    }
    dim3 grid(static_cast<unsigned>(cdiv(cols, 64)), static_cast<unsigned>(cdiv(rows, 64)));
    mx_dequant_kernel<T, FMT><<<grid, 256, 0, st>>>(q, s, y, rows, cols, transpose);
}

template <int FMT>
static void launch_mx_dequant(const uint8_t *q, const uint8_t *s, void *y, int ydtype, int64_t rows, int64_t cols,
                              int transpose, hipStream_t st) {
    if (ydtype == PT_DTYPE_BF16)
        launch_mx_dequant_t<bf16_t, FMT>(q, s, static_cast<bf16_t *>(y), rows, cols, transpose, st);
    else if (ydtype == PT_DTYPE_F16)
        launch_mx_dequant_t<f16_t, FMT>(q, s, static_cast<f16_t *>(y), rows, cols, transpose, st);
    else
        launch_mx_dequant_t<float, FMT>(q, s, static_cast<float *>(y), rows, cols, transpose, st);
}

static int mx_fmt_of(int dtype) {
    return dtype == PT_DTYPE_E4M3 ? MX_E4M3 : dtype == PT_DTYPE_E5M2 ? MX_E5M2 : dtype == PT_DTYPE_E2M1X2 ? MX_E2M1 : -1;
}

} // namespace pt

using namespace pt;

extern "C" {

// direction flags: bit 0 = 2-D (32 x 32) blocks, bit 1 = Hadamard transform (MXFP4, 1-D blocks),
// bit 2 = stochastic rounding (MXFP4)
static int check_mx_flags(int fmt, int row_flags, int col_flags) {
    PT_REQUIRE((row_flags & ~7) == 0 && (col_flags & ~7) == 0, "unknown direction flags");
    const bool rht = ((row_flags | col_flags) & 2) != 0;
    PT_REQUIRE(!rht || fmt == MX_E2M1, "the Hadamard transform belongs to the MXFP4 recipe");
    PT_REQUIRE(((row_flags | col_flags) & 4) == 0 || fmt == MX_E2M1, "stochastic rounding belongs to the MXFP4 recipe");
    PT_REQUIRE(!rht || ((row_flags | col_flags) & 1) == 0, "the Hadamard transform is not combined with 2-D blocks");
    return PT_OK;
}

int pt_quantize_mx(const void *x, int x_dtype, int64_t B, int64_t M, int64_t N, int q_dtype, void *row_q,
                   void *row_scale, int row_flags, void *col_q, void *col_scale, int col_flags, uint32_t sr_seed,
                   void *stream) {
    PT_REQUIRE(x_dtype == PT_DTYPE_BF16 || x_dtype == PT_DTYPE_F16, "input must be bf16 or fp16");
    const int fmt = mx_fmt_of(q_dtype);
    PT_REQUIRE(fmt >= 0, "q_dtype must be e4m3, e5m2 or e2m1x2");
    PT_REQUIRE(B >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    PT_REQUIRE((row_q != nullptr) == (row_scale != nullptr) && (col_q != nullptr) == (col_scale != nullptr),
               "codes and scales come in pairs");
    PT_REQUIRE(row_q || col_q, "nothing to produce");
    if (const int rc = check_mx_flags(fmt, row_q ? row_flags : 0, col_q ? col_flags : 0))
        return rc;
    const bool rht = (((row_q ? row_flags : 0) | (col_q ? col_flags : 0)) & 2) != 0;
    if (B == 0 || M == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(x, "NULL input");
    PT_REQUIRE(aligned_to(row_q, 16) && aligned_to(col_q, 16), "outputs must be 16-byte aligned");
    PT_REQUIRE(aligned_to(row_scale, 4) && aligned_to(col_scale, 4), "scale outputs must be 4-byte aligned");
    MxArgs a;
    a.x     = x;
    a.B     = B;
    a.M     = M;
    a.N     = N;
    a.Mpad  = cdiv(M, 128) * 128;
    a.Npad  = cdiv(N, 128) * 128;
    a.row_q = static_cast<uint8_t *>(row_q);
    a.row_s = static_cast<uint8_t *>(row_scale);
    a.col_q = static_cast<uint8_t *>(col_q);
    a.col_s = static_cast<uint8_t *>(col_scale);
    a.group_offs = a.row_offs_pad = a.col_offs_pad = nullptr;
    a.G          = 0;
    a.probs      = nullptr;
    a.row_mask   = nullptr;
    a.sr_mask    = ((row_q && (row_flags & 4)) ? 1 : 0) | ((col_q && (col_flags & 4)) ? 2 : 0);
    a.sr_seed    = sr_seed;
    PT_REQUIRE(a.Mpad / 128 < 65536 && B < 65536, "grid dimension out of range");
    dim3 grid(static_cast<unsigned>(a.Npad / 128), static_cast<unsigned>(a.Mpad / 128), static_cast<unsigned>(B));
    auto st = static_cast<hipStream_t>(stream);
    if (mx_rows_stream_ok(a, (row_flags & 1) != 0, rht)) {
        PT_REQUIRE(cdiv(B * M * cdiv(a.Npad, 512), 16) < (1LL << 31), "too many rows");
        if (x_dtype == PT_DTYPE_BF16)
            launch_mx_rows<bf16_t>(a, fmt, st);
        else
            launch_mx_rows<f16_t>(a, fmt, st);
        return check_launch("mx_quant_rows_kernel");
    }
    if (rht) {
        if (x_dtype == PT_DTYPE_BF16)
            launch_mx_rht<bf16_t>(a, (row_flags & 2) != 0, (col_flags & 2) != 0, grid, st);
        else
            launch_mx_rht<f16_t>(a, (row_flags & 2) != 0, (col_flags & 2) != 0, grid, st);
    } else if (x_dtype == PT_DTYPE_BF16) {
        launch_mx_fmt<bf16_t>(a, fmt, (row_flags & 1) != 0, (col_flags & 1) != 0, grid, st);
    } else {
        launch_mx_fmt<f16_t>(a, fmt, (row_flags & 1) != 0, (col_flags & 1) != 0, grid, st);
    }
    return check_launch("mx_quant_kernel");
}

// The shared body of the grouped quantizers; glu = 0 (x is [M, N]) or 1 + ACT_* (x is [M, 2 N]).
static int grouped_quantize_mx(const void *x, int x_dtype, const float *probs, const int64_t *row_mask,
                               int glu, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
                               const int64_t *row_offs_padded, const int64_t *col_offs_padded, int64_t G, void *row_q,
                               void *row_scale, int row_flags, void *col_q, void *col_scale, int col_flags, int64_t col_ld,
                               uint32_t sr_seed, void *stream) {
    PT_REQUIRE(x_dtype == PT_DTYPE_BF16 || x_dtype == PT_DTYPE_F16, "input must be bf16 or fp16");
    const int fmt = mx_fmt_of(q_dtype);
    PT_REQUIRE(fmt >= 0, "q_dtype must be e4m3, e5m2 or e2m1x2");
    PT_REQUIRE(M >= 0 && N >= 0 && G >= 1 && G <= 65535, "bad dimensions");
    PT_REQUIRE((row_q != nullptr) == (row_scale != nullptr) && (col_q != nullptr) == (col_scale != nullptr),
               "codes and scales come in pairs");
    PT_REQUIRE(row_q || col_q, "nothing to produce");
    if (const int rc = check_mx_flags(fmt, row_q ? row_flags : 0, col_q ? col_flags : 0))
        return rc;
    const bool rht = (((row_q ? row_flags : 0) | (col_q ? col_flags : 0)) & 2) != 0;
    PT_REQUIRE(col_ld % 128 == 0 && col_ld >= M, "col_ld must be a multiple of 128 that holds every padded group");
    if (glu != 0) {
        PT_REQUIRE(row_q != nullptr, "the gated quantizer produces the row direction (optionally the column direction too)");
        PT_REQUIRE(((row_flags | col_flags) & 4) == 0 && (row_flags & 2) == 0,
                   "the gated quantizer rounds to nearest; only its column direction may be Hadamard-transformed");
        PT_REQUIRE(((row_flags | col_flags) & 1) == 0, "the gated quantizer has no 2-D blocks");
    }
    if (M == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(x && group_offs && col_offs_padded, "NULL pointer");
    PT_REQUIRE(glu == 0 || probs != nullptr, "NULL probs");
    PT_REQUIRE(aligned_to(row_q, 16) && aligned_to(col_q, 16), "outputs must be 16-byte aligned");
    PT_REQUIRE(aligned_to(row_scale, 4) && aligned_to(col_scale, 4), "scale outputs must be 4-byte aligned");
    MxArgs a;
    a.x            = x;
    a.B            = 1;
    a.M            = M;
    a.N            = N;
    a.Mpad         = col_ld;
    a.Npad         = cdiv(N, 128) * 128;
    a.row_q        = static_cast<uint8_t *>(row_q);
    a.row_s        = static_cast<uint8_t *>(row_scale);
    a.col_q        = static_cast<uint8_t *>(col_q);
    a.col_s        = static_cast<uint8_t *>(col_scale);
    a.group_offs   = group_offs;
    a.row_offs_pad = row_offs_padded;
    a.col_offs_pad = col_offs_padded;
    a.G            = static_cast<int>(G);
    a.sr_mask      = ((row_q && (row_flags & 4)) ? 1 : 0) | ((col_q && (col_flags & 4)) ? 2 : 0);
    a.sr_seed      = sr_seed;
    a.probs        = probs;
    a.row_mask     = row_mask;
    PT_REQUIRE(col_ld / 128 < 65536, "grid dimension out of range");
    dim3 grid(static_cast<unsigned>(a.Npad / 128), static_cast<unsigned>(col_ld / 128), 1);
    auto st = static_cast<hipStream_t>(stream);
    if (glu != 0) {
        const bool bf = x_dtype == PT_DTYPE_BF16;
        if (glu == 1 + ACT_SILU)
            bf ? launch_mx_glu<bf16_t, 1 + ACT_SILU>(a, fmt, rht, grid, st) : launch_mx_glu<f16_t, 1 + ACT_SILU>(a, fmt, rht, grid, st);
        else
            bf ? launch_mx_glu<bf16_t, 1 + ACT_GELU>(a, fmt, rht, grid, st) : launch_mx_glu<f16_t, 1 + ACT_GELU>(a, fmt, rht, grid, st);
    } else if (rht) {
        if (x_dtype == PT_DTYPE_BF16)
            launch_mx_rht<bf16_t>(a, (row_flags & 2) != 0, (col_flags & 2) != 0, grid, st);
        else
            launch_mx_rht<f16_t>(a, (row_flags & 2) != 0, (col_flags & 2) != 0, grid, st);
    } else if (x_dtype == PT_DTYPE_BF16) {
        launch_mx_fmt<bf16_t>(a, fmt, row_q && (row_flags & 1), col_q && (col_flags & 1), grid, st);
    } else {
        launch_mx_fmt<f16_t>(a, fmt, row_q && (row_flags & 1), col_q && (col_flags & 1), grid, st);
    }
    return check_launch("mx_quant_kernel");
}

int pt_grouped_quantize_mx(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
                           const int64_t *row_offs_padded, const int64_t *col_offs_padded, int64_t G, void *row_q,
                           void *row_scale, int row_flags, void *col_q, void *col_scale, int col_flags, int64_t col_ld,
                           uint32_t sr_seed, void *stream) {
    return grouped_quantize_mx(x, x_dtype, nullptr, nullptr, 0, M, N, q_dtype, group_offs,
                               row_offs_padded, col_offs_padded, G, row_q, row_scale, row_flags, col_q, col_scale, col_flags,
                               col_ld, sr_seed, stream);
}

int pt_glu_grouped_quantize_mx(const void *x, int x_dtype, const float *probs, const int64_t *row_mask, int act, int64_t M,
                               int64_t N, int q_dtype, const int64_t *group_offs, const int64_t *row_offs_padded,
                               const int64_t *col_offs_padded, int64_t G, void *row_q, void *row_scale, void *col_q,
                               void *col_scale, int col_flags, int64_t col_ld, void *stream) {
    PT_REQUIRE(act == ACT_SILU || act == ACT_GELU, "act must be 0 (SiLU) or 1 (GELU)");
    return grouped_quantize_mx(x, x_dtype, probs, row_mask, 1 + act, M, N, q_dtype, group_offs,
                               row_offs_padded, col_offs_padded, G, row_q, row_scale, 0, col_q, col_scale, col_flags, col_ld,
                               0u, stream);
}

int pt_dequantize_mx(const void *q, int q_dtype, const void *scale, int64_t rows, int64_t cols, void *y, int y_dtype,
                     int transpose, void *stream) {
    const int fmt = mx_fmt_of(q_dtype);
    PT_REQUIRE(fmt >= 0, "q_dtype must be e4m3, e5m2 or e2m1x2");
    PT_REQUIRE(is_hp_dtype(y_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(rows >= 0 && cols >= 0 && cols % 32 == 0, "cols must be a non-negative multiple of 32");
    if (rows == 0 || cols == 0)
        return PT_OK;
    PT_REQUIRE(q && scale && y, "NULL pointer");
    PT_REQUIRE(cdiv(rows, 64) < 65536, "grid dimension out of range");
    auto           st = static_cast<hipStream_t>(stream);
    const uint8_t *qq = static_cast<const uint8_t *>(q), *ss = static_cast<const uint8_t *>(scale);
    if (fmt == MX_E4M3)
        launch_mx_dequant<MX_E4M3>(qq, ss, y, y_dtype, rows, cols, transpose, st);
    else if (fmt == MX_E5M2)
        launch_mx_dequant<MX_E5M2>(qq, ss, y, y_dtype, rows, cols, transpose, st);
    else
        launch_mx_dequant<MX_E2M1>(qq, ss, y, y_dtype, rows, cols, transpose, st);
    return check_launch("mx_dequant_kernel");
}

} // extern "C"
