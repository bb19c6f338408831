// hipcc-flags: -mllvm -amdgpu-mfma-vgpr-form=1
// MoE grouped FP8 GEMM with 128-blockwise scales: the grouped instantiations of the GEMM
// kernel (block-scale mode, compiled like gemm_fp8_block.hip with MFMA results in
// architectural VGPRs) and their C entry points.
//
//   pt_grouped_gemm_fp8             out[offs[g] : offs[g+1]] = A[offs[g] : offs[g+1]] . W_g^T
//                                   (forward and dgrad of a grouped linear layer)
//   pt_grouped_gemm_fp8_variable_k  dW[g] = LHS_g^T . RHS_g over the rows of group g
//                                   (wgrad; the reduction length differs per group)
#include "gemm_fp8_block8_vk.h"



namespace pt {

template <int GMODE, bool SB_VEC, int FA, int FB>
static int launch_grouped_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 / 2 = 256x128, 3 = 128x128 (two workgroups per CU), 4 = 256x256 with
    // eight wavefronts (row groups: gemm_fp8_block8.h; variable K: gemm_fp8_block8_vk.h)
    // (the 256x128 tile leaves LDS for the tile prefix sums of 1024 groups only)
    if (tile_cfg == 0) { // 256-row tiles once the average group fills a couple of them
        tile_cfg = ((GMODE == GROUP_K ? a.M >= 1024 : (a.G > 0 && a.M / a.G >= 512)) && a.N >= 1024) ? 2 : 3;
        if (GMODE == GROUP_ROWS && !SB_VEC && tile_cfg == 2 && a.N >= 2048)
            tile_cfg = 4;
        if (GMODE == GROUP_K && SB_VEC && a.M >= 1024 && a.N >= 1024)
            tile_cfg = 4; // measured 15-20 % faster than the 256x128 tile on 4096 x 7168 and 7168 x 2048 outputs
    }
    if (tile_cfg == 4) {
        if constexpr (GMODE == GROUP_ROWS && !SB_VEC)
            return launch_gemm_block8<FA, FB, GROUP_ROWS>(a, stream);
        else if constexpr (GMODE == GROUP_K && SB_VEC)
            return launch_gemm_block8_vk<FA, FB>(a, stream);
        else
            tile_cfg = 2;
    }
    if (a.G > 1024)
        tile_cfg = 3;
    if (tile_cfg == 3)
        return launch_gemm_cfg<4, 4, SCALE_BLOCK, SB_VEC, FA, FB, GMODE>(a, stream);
    return launch_gemm_cfg<8, 4, SCALE_BLOCK, SB_VEC, FA, FB, GMODE>(a, stream);
}

template <int GMODE, bool SB_VEC>
static int launch_grouped(const GemmArgs &a, int fa, int fb, int tile_cfg, hipStream_t stream) {
    if (fa == 0 && fb == 0)
        return launch_grouped_tiles<GMODE, SB_VEC, 0, 0>(a, tile_cfg, stream);
    if (fa == 0 && fb == 1)
        return launch_grouped_tiles<GMODE, SB_VEC, 0, 1>(a, tile_cfg, stream);
    if (fa == 1 && fb == 0)
        return launch_grouped_tiles<GMODE, SB_VEC, 1, 0>(a, tile_cfg, stream);
    return launch_grouped_tiles<GMODE, SB_VEC, 1, 1>(a, tile_cfg, stream);
}

// rows [offs[G], rows) of a [rows, row_bytes] matrix := 0 (16-byte stores; row_bytes % 16 == 0
// is not required: the tail is a contiguous byte range)
__global__ __launch_bounds__(256) void zero_tail_rows_kernel(uint8_t *c, const int64_t *group_offs, int G,
                                                             int64_t rows, int64_t row_bytes) {
    const int64_t first = group_offs[G];
    if (first >= rows)
        return;
    uint8_t      *p     = c + first * row_bytes;
    const int64_t bytes = (rows - first) * row_bytes;
    const int64_t head  = (16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15; // bytes up to alignment
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, nthr = static_cast<int64_t>(gridDim.x) * 256;
    const int64_t h   = head < bytes ? head : bytes;
    for (int64_t i = tid; i < h; i += nthr)
        p[i] = 0;
    const int64_t n16 = (bytes - h) / 16;
    u32x4        *q   = reinterpret_cast<u32x4 *>(p + h);
    for (int64_t i = tid; i < n16; i += nthr)
        q[i] = u32x4{0u, 0u, 0u, 0u};
    for (int64_t i = h + n16 * 16 + tid; i < bytes; i += nthr)
        p[i] = 0;
}

} // namespace pt

using namespace pt;

extern "C" {

size_t pt_grouped_gemm_fp8_workspace_bytes(int64_t G, int64_t M, int64_t N, int64_t K, int trans_b) {
    const int64_t Kp  = padded_k(K);
    const bool    pad = Kp != K;
    size_t        b   = 0;
    if (pad)
        b += static_cast<size_t>(round_up(M * Kp, 256));
    if (!trans_b || pad)
        b += static_cast<size_t>(round_up(G * N * Kp, 256));
    return b;
}

int pt_grouped_gemm_fp8(const void *a, int a_dtype, const float *a_scale, const void *b, int b_dtype,
                        const float *b_scale, void *c, int c_dtype, const int64_t *group_offs, int64_t G,
                        int64_t M, int64_t out_rows, int64_t N, int64_t K, int trans_b, void *workspace,
                        size_t workspace_bytes, int tile_cfg, void *stream) {
    PT_REQUIRE(is_fp8_dtype(a_dtype) && is_fp8_dtype(b_dtype), "operands must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && M >= 0 && N >= 0 && K >= 0 && out_rows >= M, "bad dimensions");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 4, "tile_cfg must be 0..4");
    PT_REQUIRE(K < (1LL << 24), "K must be below 2^24");
    auto st = static_cast<hipStream_t>(stream);
    if (out_rows == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(c && group_offs, "NULL pointer");
    const int64_t ES = c_dtype == PT_DTYPE_F32 ? 4 : 2;
    PT_REQUIRE(a && b && a_scale && b_scale, "NULL tensor pointer");
    PT_REQUIRE(aligned_to(a, 16) && aligned_to(b, 16) && aligned_to(c, 16), "operands must be 16-byte aligned");
    PT_REQUIRE(K > 0, "K must be positive");

    const int64_t  Kp  = padded_k(K);
    const bool     pad = Kp != K;
    const uint8_t *A   = static_cast<const uint8_t *>(a);
    const uint8_t *B   = static_cast<const uint8_t *>(b);
    if (!trans_b || pad) {
        const size_t need = pt_grouped_gemm_fp8_workspace_bytes(G, M, N, K, trans_b);
        if (workspace == nullptr || workspace_bytes < need || !aligned_to(workspace, 16))
            return fail(PT_ERR_WORKSPACE, "pt_grouped_gemm_fp8: workspace missing, too small or misaligned");
        uint8_t *ws = static_cast<uint8_t *>(workspace);
        if (pad) {
            if (M > 0)
                launch_pad_rows(A, ws, M, K, Kp, st);
            A = ws;
            ws += round_up(M * Kp, 256);
        }
        if (G * N > 0) {
            if (!trans_b) // stored [G, K, N] -> [G, N, Kp]
                launch_transpose(B, ws, G, K, N, Kp, st);
            else
                launch_pad_rows(B, ws, G * N, K, Kp, st);
        }
        B = ws;
    }

    const int64_t kb = cdiv(K, 128), nb = cdiv(N, 128);
    GemmArgs      g{};
    g.A          = A;
    g.B          = B;
    g.C          = c;
    g.sA         = a_scale; // [K/128, M]: one scale per row and K block, K block major
    g.sB         = b_scale; // [G, N/128, K/128] (trans_b) or [G, K/128, N/128]
    g.M          = M;
    g.N          = N;
    g.K          = Kp;
    g.lda        = Kp;
    g.ldb        = Kp;
    g.sa_m       = 1;
    g.sa_k       = M;
    g.sb_n       = trans_b ? kb : 1;
    g.sb_k       = trans_b ? 1 : nb;
    g.sa_shift   = 0;
    g.sb_shift   = 7;
    g.kb_valid   = static_cast<int>(kb);
    g.out_dtype  = c_dtype;
    g.accumulate = 0;
    g.G          = static_cast<int>(G);
    g.group_offs = group_offs;
    g.b_gstride  = N * Kp;
    g.sb_gstride = nb * kb;
    g.c_gstride  = 0;
    const int fa = a_dtype == PT_DTYPE_E5M2 ? 1 : 0, fb = b_dtype == PT_DTYPE_E5M2 ? 1 : 0;
    if (G > 0 && M > 0) {
        const int rc = launch_grouped<GROUP_ROWS, false>(g, fa, fb, tile_cfg, st);
        if (rc != PT_OK)
            return rc;
    }
    // rows past the last routed token (over-allocated outputs) read as zero
    if (out_rows > 0) {
        zero_tail_rows_kernel<<<256, 256, 0, st>>>(static_cast<uint8_t *>(c), group_offs, static_cast<int>(G), out_rows,
                                                   N * ES);
        return check_launch("zero_tail_rows_kernel");
    }
    return PT_OK;
}

size_t pt_grouped_gemm_fp8_variable_k_workspace_bytes(int64_t Mp, int64_t Ml, int64_t Nr) {
    const int64_t ld = round_up(Mp, 128);
    return static_cast<size_t>(round_up(Ml * ld, 256) + round_up(Nr * ld, 256));
}

int pt_grouped_gemm_fp8_variable_k(const void *lhs, int lhs_dtype, const float *lhs_scale, const void *rhs,
                                   int rhs_dtype, const float *rhs_scale, void *c, int c_dtype,
                                   const int64_t *group_offs, int64_t G, int64_t Mp, int64_t Ml, int64_t Nr,
                                   int trans_c, int accumulate, int operands_kmajor, void *workspace,
                                   size_t workspace_bytes, int tile_cfg, void *stream) {
    PT_REQUIRE(is_fp8_dtype(lhs_dtype) && is_fp8_dtype(rhs_dtype), "operands must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && Mp >= 0 && Ml >= 0 && Nr >= 0, "bad dimensions");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 4, "tile_cfg must be 0..4");
    PT_REQUIRE(Mp < (1LL << 24), "at most 2^24 rows");
    auto st = static_cast<hipStream_t>(stream);
    if (G == 0 || Ml == 0 || Nr == 0)
        return PT_OK;
    PT_REQUIRE(lhs && rhs && lhs_scale && rhs_scale && c && group_offs, "NULL pointer");
    PT_REQUIRE(aligned_to(lhs, 16) && aligned_to(rhs, 16) && aligned_to(c, 16), "operands must be 16-byte aligned");
    const int64_t  ld = round_up(Mp, 128);
    const uint8_t *lt, *rt;
    if (operands_kmajor) {
        // the operands arrive with the rows as their contiguous axis already: [cols, Mp]
        PT_REQUIRE(Mp % 128 == 0, "K-major operands need a padded row count that is a multiple of 128");
        lt = static_cast<const uint8_t *>(lhs);
        rt = static_cast<const uint8_t *>(rhs);
    } else {
        const size_t need = pt_grouped_gemm_fp8_variable_k_workspace_bytes(Mp, Ml, Nr);
        if (workspace == nullptr || workspace_bytes < need || !aligned_to(workspace, 16))
            return fail(PT_ERR_WORKSPACE, "pt_grouped_gemm_fp8_variable_k: workspace missing, too small or misaligned");
        // both operands become K-contiguous: [Mp, cols] -> [cols, ld] with the rows as K
        uint8_t *wl = static_cast<uint8_t *>(workspace);
        uint8_t *wr = wl + round_up(Ml * ld, 256);
        launch_transpose(static_cast<const uint8_t *>(lhs), wl, 1, Mp, Ml, ld, st);
        launch_transpose(static_cast<const uint8_t *>(rhs), wr, 1, Mp, Nr, ld, st);
        lt = wl;
        rt = wr;
    }

    // C[g] = lhs_g^T rhs_g ([Ml, Nr]); trans_c asks for its transpose: swap the operand roles
    GemmArgs g{};
    g.A          = trans_c ? rt : lt;
    g.B          = trans_c ? lt : rt;
    g.C          = c;
    g.sA         = trans_c ? rhs_scale : lhs_scale; // [Mp/128, cols]
    g.sB         = trans_c ? lhs_scale : rhs_scale;
    g.M          = trans_c ? Nr : Ml;
    g.N          = trans_c ? Ml : Nr;
    g.K          = 0; // per group
    g.lda        = ld;
    g.ldb        = ld;
    g.sa_m       = 1;
    g.sa_k       = g.M;
    g.sb_n       = 1;
    g.sb_k       = g.N;
    g.sa_shift   = 0;
    g.sb_shift   = 0;
    g.kb_valid   = 1 << 30; // every slab of a group has its scales
    g.out_dtype  = c_dtype;
    g.accumulate = accumulate;
    g.G          = static_cast<int>(G);
    g.group_offs = group_offs;
    g.b_gstride  = 0;
    g.sb_gstride = 0;
    g.c_gstride  = Ml * Nr;
    const int fl = lhs_dtype == PT_DTYPE_E5M2 ? 1 : 0, fr = rhs_dtype == PT_DTYPE_E5M2 ? 1 : 0;
    return launch_grouped<GROUP_K, true>(g, trans_c ? fr : fl, trans_c ? fl : fr, tile_cfg, st);
}

} // extern "C"
