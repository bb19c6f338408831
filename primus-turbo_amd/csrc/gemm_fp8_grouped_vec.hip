// MoE grouped FP8 GEMM with vector scales (TENSORWISE: one scale per tensor, ROWWISE: one per row
// / column) on gfx950: forward / dgrad over row groups and the variable-K wgrad.
// Semantics of Primus-Turbo's grouped TENSORWISE / ROWWISE path (primus_turbo/pytorch/ops/
// grouped_gemm_fp8.py:265-603 with kernels/grouped_gemm/grouped_gemm_fp8_impl.py:888-1022):
//   out[offs[g] : offs[g+1]] = (A[offs[g] : offs[g+1]] . op(B[g])) * sA[m] * sB[g, n]
//   C[g] = (L[offs[g] : offs[g+1]]^T . R[offs[g] : offs[g+1]]) * sL[col of L] * sR[col of R]
// The groups of these granularities are packed tight (no per-group padding in the data), so the
// wgrad operands are copied into K-contiguous form with every group padded to whole 128-byte
// slabs of zeros -- the layout the kernel's variable-K mode reads.
#include "gemm_fp8_kernel.h"

namespace pt {

template <int GMODE, int FA, int FB> static int launch_gvec_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 = 256x256, 3 = 128x128 (two workgroups per CU)
    if (tile_cfg == 0) {
        const bool big = GMODE == GROUP_K ? (a.M >= 1024 && a.N >= 1024)
                                          : (a.G > 0 && a.M / a.G >= 512 && a.N >= 1024);
        tile_cfg       = big ? 1 : 3;
    }
    if (tile_cfg == 1 || tile_cfg == 2)
        return launch_gemm_cfg<8, 8, SCALE_VECTOR, false, FA, FB, GMODE>(a, stream);
    return launch_gemm_cfg<4, 4, SCALE_VECTOR, false, FA, FB, GMODE>(a, stream);
}

template <int GMODE> static int launch_gvec(const GemmArgs &a, int fa, int fb, int tile_cfg, hipStream_t stream) {
    if (fa == 0 && fb == 0)
        return launch_gvec_tiles<GMODE, 0, 0>(a, tile_cfg, stream);
    if (fa == 0 && fb == 1)
        return launch_gvec_tiles<GMODE, 0, 1>(a, tile_cfg, stream);
    if (fa == 1 && fb == 0)
        return launch_gvec_tiles<GMODE, 1, 0>(a, tile_cfg, stream);
    return launch_gvec_tiles<GMODE, 1, 1>(a, tile_cfg, stream);
}

// padded[0] = 0, padded[g + 1] = padded[g] + round_up(offs[g + 1] - offs[g], 128)
__global__ void pad_offs128_kernel(const int64_t *offs, int G, int64_t *padded) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        int64_t run = 0;
        padded[0]   = 0;
        for (int g = 0; g < G; ++g) {
            run += (offs[g + 1] - offs[g] + 127) / 128 * 128;
            padded[g + 1] = run;
        }
    }
}

// in [M, C] (rows of G groups, packed) -> out [C, ld]: out[c][padded[g] + i] = in[offs[g] + i][c],
// zeros in the padding of every group; columns from padded[G] on are not written. One workgroup
// per 128 x 128 tile of the padded row space (the byte transpose of the dense case with the rows
// looked up through the group offsets).
__global__ __launch_bounds__(256) void transpose_grouped_pad_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                                    const int64_t *__restrict__ offs,
                                                                    const int64_t *__restrict__ padded, const int G,
                                                                    const int64_t C, const int64_t ld) {
    constexpr int       P = 33;
    __shared__ uint32_t t[128 * P];
    const int64_t       p0 = static_cast<int64_t>(blockIdx.y) * 128, c0 = static_cast<int64_t>(blockIdx.x) * 128;
    if (p0 >= padded[G])
        return;
    const int g = find_group(padded, G, p0);
    const int64_t in0 = offs[g] + (p0 - padded[g]), in_end = offs[g + 1];
    const int     tid = threadIdx.x;
    const bool    vec = (C & 15) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
    {
        const int     cc = tid & 7, rg = tid >> 3;
        const int64_t gc = c0 + cc * 16;
        u32x4         a[4];
        if (vec) {
            // the four pieces are requested together (a piece outside the group re-reads the first
            // bytes of the matrix and is zeroed: no branch between the loads)
            bool ok[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t gr = in0 + rg * 4 + e;
                ok[e]            = gr < in_end && gc < C;
                a[e]             = *reinterpret_cast<const u32x4 *>(in + (ok[e] ? gr * C + gc : 0));
            }
#pragma unroll
            for (int e = 0; e < 4; ++e)
                a[e] = ok[e] ? a[e] : u32x4{0, 0, 0, 0};
        } else {
#pragma unroll 1
            for (int e = 0; e < 4; ++e) {
                const int64_t gr = in0 + rg * 4 + e;
                a[e]             = u32x4{0, 0, 0, 0};
                if (gr < in_end && gc < C) {
                    uint32_t w[4] = {0, 0, 0, 0};
                    for (int k = 0; k < 16; ++k)
                        if (gc + k < C)
                            w[k >> 2] |= static_cast<uint32_t>(in[gr * C + gc + k]) << (8 * (k & 3));
                    a[e] = u32x4{w[0], w[1], w[2], w[3]};
                }
            }
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t t0 = __builtin_amdgcn_perm(a[1][w], a[0][w], 0x05010400u);
            const uint32_t t1 = __builtin_amdgcn_perm(a[1][w], a[0][w], 0x07030602u);
            const uint32_t t2 = __builtin_amdgcn_perm(a[3][w], a[2][w], 0x05010400u);
            const uint32_t t3 = __builtin_amdgcn_perm(a[3][w], a[2][w], 0x07030602u);
            const int      c  = cc * 16 + w * 4;
            t[(c + 0) * P + rg] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
            t[(c + 1) * P + rg] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
            t[(c + 2) * P + rg] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
            t[(c + 3) * P + rg] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
        }
    }
    __syncthreads();
    const int j = tid & 7;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     c  = (tid >> 3) + 32 * p;
        const int64_t gc = c0 + c;
        if (gc < C) { // ld is a multiple of 128: the 16-byte chunk is always inside the row
            u32x4 v;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                v[k] = t[c * P + j * 4 + k];
            *reinterpret_cast<u32x4 *>(out + gc * ld + p0 + j * 16) = v;
        }
    }
}

__global__ __launch_bounds__(256) void zero_rows_from2_kernel(uint8_t *c, const int64_t *offs, int G, int64_t rows,
                                                              int64_t row_bytes) {
    const int64_t first = offs[G];
    if (first >= rows)
        return;
    uint8_t      *p     = c + first * row_bytes;
    const int64_t bytes = (rows - first) * row_bytes;
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, nthr = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t i = tid; i < bytes; i += nthr)
        p[i] = 0;
}

} // namespace pt

using namespace pt;

extern "C" {

size_t pt_grouped_gemm_fp8_vec_workspace_bytes(int64_t G, int64_t M, int64_t N, int64_t K, int trans_b) {
    const int64_t Kp  = padded_k(K);
    const bool    pad = Kp != K;
    size_t        b   = 0;
    if (pad)
        b += static_cast<size_t>(round_up(M * Kp, 256));
    if (!trans_b || pad)
        b += static_cast<size_t>(round_up(G * N * Kp, 256));
    return b;
}

int pt_grouped_gemm_fp8_vec(const void *a, int a_dtype, const float *a_scale, int64_t sa_stride, const void *b, int b_dtype,
                            const float *b_scale, int64_t sb_stride, int64_t sb_gstride, void *c, int c_dtype,
                            const int64_t *group_offs, int64_t G, int64_t M, int64_t out_rows, int64_t N, int64_t K,
                            int trans_b, void *workspace, size_t workspace_bytes, int tile_cfg, void *stream) {
    PT_REQUIRE(is_fp8_dtype(a_dtype) && is_fp8_dtype(b_dtype), "operands must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && M >= 0 && N >= 0 && K >= 0 && out_rows >= M, "bad dimensions");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 3, "tile_cfg must be 0..3");
    PT_REQUIRE(K < (1LL << 24), "K must be below 2^24");
    auto st = static_cast<hipStream_t>(stream);
    if (out_rows == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(c && group_offs, "NULL pointer");
    const int64_t ES = c_dtype == PT_DTYPE_F32 ? 4 : 2;
    if (G > 0 && M > 0 && K > 0) {
        PT_REQUIRE(a && b && a_scale && b_scale, "NULL tensor pointer");
        PT_REQUIRE(aligned_to(a, 16) && aligned_to(b, 16) && aligned_to(c, 16), "operands must be 16-byte aligned");
        const int64_t  Kp  = padded_k(K);
        const bool     pad = Kp != K;
        const uint8_t *A   = static_cast<const uint8_t *>(a);
        const uint8_t *B   = static_cast<const uint8_t *>(b);
        if (!trans_b || pad) {
            const size_t need = pt_grouped_gemm_fp8_vec_workspace_bytes(G, M, N, K, trans_b);
            if (workspace == nullptr || workspace_bytes < need || !aligned_to(workspace, 16))
                return fail(PT_ERR_WORKSPACE, "pt_grouped_gemm_fp8_vec: workspace missing, too small or misaligned");
            uint8_t *ws = static_cast<uint8_t *>(workspace);
            if (pad) {
                launch_pad_rows(A, ws, M, K, Kp, st);
                A = ws;
                ws += round_up(M * Kp, 256);
            }
            if (!trans_b) // stored [G, K, N] -> [G, N, Kp]
                launch_transpose(B, ws, G, K, N, Kp, st);
            else
                launch_pad_rows(B, ws, G * N, K, Kp, st);
            B = ws;
        }
        GemmArgs g{};
        g.A          = A;
        g.B          = B;
        g.C          = c;
        g.sA         = a_scale;
        g.sB         = b_scale;
        g.M          = M;
        g.N          = N;
        g.K          = Kp;
        g.lda        = Kp;
        g.ldb        = Kp;
        g.sa_m       = sa_stride;
        g.sb_n       = sb_stride;
        g.out_dtype  = c_dtype;
        g.G          = static_cast<int>(G);
        g.group_offs = group_offs;
        g.b_gstride  = N * Kp;
        g.sb_gstride = sb_gstride;
        const int rc = launch_gvec<GROUP_ROWS>(g, a_dtype == PT_DTYPE_E5M2, b_dtype == PT_DTYPE_E5M2, tile_cfg, st);
        if (rc != PT_OK)
            return rc;
    } else if (K == 0 && M > 0) {
        zero_rows_from2_kernel<<<256, 256, 0, st>>>(static_cast<uint8_t *>(c), group_offs, 0, M, N * ES); // offs[0] = 0
    }
    zero_rows_from2_kernel<<<256, 256, 0, st>>>(static_cast<uint8_t *>(c), group_offs, static_cast<int>(G), out_rows, N * ES);
    return check_launch("pt_grouped_gemm_fp8_vec");
}

size_t pt_grouped_gemm_fp8_vec_variable_k_workspace_bytes(int64_t G, int64_t M, int64_t Ml, int64_t Nr) {
    const int64_t ld = round_up(M + 128 * G, 128);
    return static_cast<size_t>(round_up((G + 1) * 8, 256) + round_up(Ml * ld, 256) + round_up(Nr * ld, 256));
}

int pt_grouped_gemm_fp8_vec_variable_k(const void *lhs, int lhs_dtype, const float *lhs_scale, int64_t sl_stride,
                                       const void *rhs, int rhs_dtype, const float *rhs_scale, int64_t sr_stride, void *c,
                                       int c_dtype, const int64_t *group_offs, int64_t G, int64_t M, int64_t Ml,
                                       int64_t Nr, int trans_c, int accumulate, void *workspace, size_t workspace_bytes,
                                       int tile_cfg, void *stream) {
    PT_REQUIRE(is_fp8_dtype(lhs_dtype) && is_fp8_dtype(rhs_dtype), "operands must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && G <= 65535 && M >= 0 && Ml >= 0 && Nr >= 0, "bad dimensions");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 3, "tile_cfg must be 0..3");
    PT_REQUIRE(M + 128 * G < (1LL << 24), "at most 2^24 padded rows");
    auto st = static_cast<hipStream_t>(stream);
    if (G == 0 || Ml == 0 || Nr == 0)
        return PT_OK;
    PT_REQUIRE(lhs_scale && rhs_scale && c && group_offs, "NULL pointer");
    PT_REQUIRE(M == 0 || (lhs && rhs), "NULL operand");
    PT_REQUIRE(aligned_to(c, 16), "output must be 16-byte aligned");
    const size_t need = pt_grouped_gemm_fp8_vec_variable_k_workspace_bytes(G, M, Ml, Nr);
    if (workspace == nullptr || workspace_bytes < need || !aligned_to(workspace, 16))
        return fail(PT_ERR_WORKSPACE, "pt_grouped_gemm_fp8_vec_variable_k: workspace missing, too small or misaligned");
    const int64_t ld     = round_up(M + 128 * G, 128);
    uint8_t      *ws     = static_cast<uint8_t *>(workspace);
    int64_t      *padded = reinterpret_cast<int64_t *>(ws);
    uint8_t      *lt     = ws + round_up((G + 1) * 8, 256);
    uint8_t      *rt     = lt + round_up(Ml * ld, 256);
    pad_offs128_kernel<<<1, 64, 0, st>>>(group_offs, static_cast<int>(G), padded);
    const unsigned gy = static_cast<unsigned>(ld / 128);
    transpose_grouped_pad_kernel<<<dim3(static_cast<unsigned>(cdiv(Ml, 128)), gy), 256, 0, st>>>(
        static_cast<const uint8_t *>(lhs), lt, group_offs, padded, static_cast<int>(G), Ml, ld);
    transpose_grouped_pad_kernel<<<dim3(static_cast<unsigned>(cdiv(Nr, 128)), gy), 256, 0, st>>>(
        static_cast<const uint8_t *>(rhs), rt, group_offs, padded, static_cast<int>(G), Nr, ld);

    GemmArgs g{};
    g.A          = trans_c ? rt : lt;
    g.B          = trans_c ? lt : rt;
    g.C          = c;
    g.sA         = trans_c ? rhs_scale : lhs_scale;
    g.sB         = trans_c ? lhs_scale : rhs_scale;
    g.M          = trans_c ? Nr : Ml;
    g.N          = trans_c ? Ml : Nr;
    g.K          = 0; // per group
    g.lda        = ld;
    g.ldb        = ld;
    g.sa_m       = trans_c ? sr_stride : sl_stride;
    g.sb_n       = trans_c ? sl_stride : sr_stride;
    g.out_dtype  = c_dtype;
    g.accumulate = accumulate;
    g.G          = static_cast<int>(G);
    g.group_offs = padded;
    g.c_gstride  = Ml * Nr;
    const int fl = lhs_dtype == PT_DTYPE_E5M2 ? 1 : 0, fr = rhs_dtype == PT_DTYPE_E5M2 ? 1 : 0;
    return launch_gvec<GROUP_K>(g, trans_c ? fr : fl, trans_c ? fl : fr, tile_cfg, st);
}

} // extern "C"
