// MX-scaled GEMMs (MXFP8 and MXFP4, NT layout): the instantiations of the GEMM kernel that let
// the matrix core apply the E8M0 block scales (v_mfma_scale_f32_16x16x128_f8f6f4), and their
// C entry point.
#include "gemm_mx8.h"

namespace pt {

template <int FA, int FB> static int launch_mx_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 = 256x256, 2 = 256x128, 3 = 128x128, 4 = 256x256 with eight wavefronts
    // (the eight-wavefront tile measured 2-4 % faster than four wavefronts on MXFP4 at 16384^3 and
    // 8192 x 28672 x 8192, and 0-9 % slower on MXFP8)
    if (tile_cfg == 0)
        tile_cfg = (a.M >= 2048 && a.N >= 2048) ? (FA == 4 ? 4 : 1) : 3;
    if (tile_cfg == 4)
        return launch_gemm_mx8<FA, FB>(a, stream);
    if (tile_cfg == 1)
        return launch_gemm_cfg<8, 8, SCALE_MX, false, FA, FB>(a, stream);
    if (tile_cfg == 2)
        return launch_gemm_cfg<8, 4, SCALE_MX, false, FA, FB>(a, stream);
    return launch_gemm_cfg<4, 4, SCALE_MX, false, FA, FB>(a, stream);
}

} // namespace pt

using namespace pt;

extern "C" {

// Bytes of one operand row as the kernel wants it: whole 128-byte slabs, at least four.
static int64_t mx_row_bytes(int64_t K, bool fp4) {
    return padded_k(fp4 ? cdiv(K, 2) : K);
}

// Word-major copy of a scale array: [rows, K / 128 words] 32-bit words transposed to [words, rows].
// Done for problems whose scale traffic matters (large K loops over many rows): a few microseconds
// on a few megabytes, against 64 separate cache lines per scale copy instruction in the GEMM.
static bool mx_wordmajor_pays(int64_t M, int64_t N, int64_t K) {
    return M >= 1024 && N >= 1024 && K >= 1024;
}
static int64_t mx_scale_words(int64_t K) {
    return cdiv(K / 32, 4);
}

size_t pt_gemm_mx_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int fp4) {
    const int64_t need = mx_row_bytes(K, fp4 != 0);
    size_t        b    = 0;
    if (mx_wordmajor_pays(M, N, K))
        b += static_cast<size_t>(round_up(M * mx_scale_words(K) * 4, 256) + round_up(N * mx_scale_words(K) * 4, 256));
    if (lda != need)
        b += static_cast<size_t>(round_up(M * need, 256));
    if (ldb != need)
        b += static_cast<size_t>(round_up(N * need, 256));
    return b;
}

int pt_gemm_mx(const void *a, const void *a_scale, const void *b, const void *b_scale, int ab_dtype, int a_e5m2,
               int b_e5m2, void *c, int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
               int64_t sa_ld, int64_t sb_ld, int accumulate, void *workspace, size_t workspace_bytes, int tile_cfg,
               void *stream) {
    const bool fp4 = ab_dtype == PT_DTYPE_E2M1X2;
    PT_REQUIRE(fp4 || ab_dtype == PT_DTYPE_E4M3 || ab_dtype == PT_DTYPE_E5M2, "operands must be fp8 or e2m1x2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(M >= 0 && N >= 0 && K > 0 && K % 32 == 0, "K must be a positive multiple of 32");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 4, "tile_cfg must be 0..4");
    const int64_t kbytes = fp4 ? K / 2 : K, kblocks = K / 32;
    PT_REQUIRE(lda >= kbytes && ldb >= kbytes && sa_ld >= kblocks && sb_ld >= kblocks, "row pitches too small");
    PT_REQUIRE(kbytes < (1LL << 24), "K too large");
    if (M == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(a && b && c && a_scale && b_scale, "NULL tensor pointer");
    PT_REQUIRE(aligned_to(a, 16) && aligned_to(b, 16) && aligned_to(c, 16) && lda % 16 == 0 && ldb % 16 == 0,
               "operands must be 16-byte aligned");
    auto st = static_cast<hipStream_t>(stream);

    // the kernel reads whole 128-byte slabs (at least four): copy rows that are shorter, or
    // that carry anything but zeros behind K, into zero-padded rows
    const int64_t  need = mx_row_bytes(K, fp4);
    const uint8_t *A = static_cast<const uint8_t *>(a), *B = static_cast<const uint8_t *>(b);
    // word-major scales need whole 32-bit words per row in the source, and room in the workspace:
    // without it (a caller that passes only what the operand copies need, or nothing) the scales
    // are read in place
    const bool     copies    = lda != need || ldb != need;
    const size_t   want_copy = static_cast<size_t>((lda != need ? round_up(M * need, 256) : 0) + (ldb != need ? round_up(N * need, 256) : 0));
    const size_t   want_all  = pt_gemm_mx_workspace_bytes(M, N, K, lda, ldb, fp4);
    const bool     have_all  = workspace != nullptr && workspace_bytes >= want_all && aligned_to(workspace, 16);
    const bool     wordmajor = have_all && mx_wordmajor_pays(M, N, K) && sa_ld % 4 == 0 && sb_ld % 4 == 0 &&
                           aligned_to(a_scale, 4) && aligned_to(b_scale, 4) && sa_ld >= mx_scale_words(K) * 4 &&
                           sb_ld >= mx_scale_words(K) * 4;
    const void *sa_use = a_scale, *sb_use = b_scale;
    if (copies || wordmajor) {
        if (workspace == nullptr || workspace_bytes < want_copy || !aligned_to(workspace, 16))
            return fail(PT_ERR_WORKSPACE, "pt_gemm_mx: workspace missing, too small or misaligned");
        uint8_t *ws = static_cast<uint8_t *>(workspace);
        if (wordmajor) {
            const int64_t W = mx_scale_words(K);
            // in: [rows, sa_ld / 4] words (the first W of every row are used) -> out: [W, rows]
            if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(a_scale), reinterpret_cast<uint32_t *>(ws), M, W, sa_ld / 4, st))
                return rc;
            sa_use = ws;
            ws += round_up(M * W * 4, 256);
            if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(b_scale), reinterpret_cast<uint32_t *>(ws), N, W, sb_ld / 4, st))
                return rc;
            sb_use = ws;
            ws += round_up(N * W * 4, 256);
        }
        if (lda != need) {
            launch_pad_rows2(A, ws, M, kbytes, lda, need, st);
            A = ws;
            ws += round_up(M * need, 256);
        }
        if (ldb != need) {
            launch_pad_rows2(B, ws, N, kbytes, ldb, need, st);
            B = ws;
        }
    }

    GemmArgs g{};
    g.A          = A;
    g.B          = B;
    g.C          = c;
    g.sA         = reinterpret_cast<const float *>(sa_use); // E8M0 bytes in this mode
    g.sB         = reinterpret_cast<const float *>(sb_use);
    g.sa_wpitch  = wordmajor ? M * 4 : 0;
    g.sb_wpitch  = wordmajor ? N * 4 : 0;
    g.M          = M;
    g.N          = N;
    g.K          = need;
    g.lda        = need;
    g.ldb        = need;
    g.sa_m       = sa_ld;
    g.sb_n       = sb_ld;
    g.kb_valid   = static_cast<int>(kblocks);
    g.out_dtype  = c_dtype;
    g.accumulate = accumulate;
    if (fp4)
        return launch_mx_tiles<4, 4>(g, tile_cfg, st);
    if (!a_e5m2 && !b_e5m2)
        return launch_mx_tiles<0, 0>(g, tile_cfg, st);
    if (!a_e5m2 && b_e5m2)
        return launch_mx_tiles<0, 1>(g, tile_cfg, st);
    if (a_e5m2 && !b_e5m2)
        return launch_mx_tiles<1, 0>(g, tile_cfg, st);
    return launch_mx_tiles<1, 1>(g, tile_cfg, st);
}

} // extern "C"
