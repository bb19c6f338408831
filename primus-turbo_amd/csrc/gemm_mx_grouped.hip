// MoE grouped MXFP8 / MXFP4 GEMM on gfx950 (E8M0 scale per 32 elements of K, applied by the
// matrix core):
//   * row groups (forward / dgrad): out[rows of g] = A[rows of g] . B[g]^T, A [rows, K] and B
//     [G, N, K] both K-contiguous; the rows of A may sit in a per-group padded layout while the
//     output is packed tight (two offset arrays);
//   * variable K (wgrad): C[g] = L[:, K range of g] . R[:, K range of g]^T with both operands
//     K-contiguous over the segment-padded token axis (the transposed column-direction output of
//     the grouped MX quantizer), K ranges on whole 128-byte slabs (multiples of 128 elements,
//     MXFP4 256).
// Semantics of Primus-Turbo's grouped MXFP8 path (primus_turbo/pytorch/ops/grouped_gemm_fp8.py:
// 604-840: forward and dgrad are one NT product per group over the padded rows with
// group_offs_out packing the result, wgrad is a variable-K NT product over the 128-padded
// column-direction operands) and of its grouped MXFP4 path (ops/grouped_gemm_fp4.py:101-309:
// the same three products over tight rows and 256-padded column-direction operands).
#include "gemm_mx8.h"

namespace pt {

template <int GMODE, int FA, int FB> static int launch_mxg_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 = 256x256, 3 = 128x128 (two workgroups per CU), 4 = 256x256 with eight
    // wavefronts (row groups only)
    if (tile_cfg == 0) {
        const bool big = GMODE == GROUP_K ? (a.M >= 1024 && a.N >= 1024)
                                          : (a.G > 0 && a.M / a.G >= 512 && a.N >= 1024);
        tile_cfg       = big ? 1 : 3;
    }
    if constexpr (GMODE == GROUP_ROWS) {
        if (tile_cfg == 4)
            return launch_gemm_mx8<FA, FB, GROUP_ROWS>(a, stream);
    }
    if (tile_cfg == 1 || tile_cfg == 2)
        return launch_gemm_cfg<8, 8, SCALE_MX, false, FA, FB, GMODE>(a, stream);
    return launch_gemm_cfg<4, 4, SCALE_MX, false, FA, FB, GMODE>(a, stream);
}

template <int GMODE> static int launch_mxg(const GemmArgs &a, int fa, int fb, int tile_cfg, hipStream_t stream) {
    if (fa == 4)
        return launch_mxg_tiles<GMODE, 4, 4>(a, tile_cfg, stream);
    if (fa == 0 && fb == 0)
        return launch_mxg_tiles<GMODE, 0, 0>(a, tile_cfg, stream);
    if (fa == 0 && fb == 1)
        return launch_mxg_tiles<GMODE, 0, 1>(a, tile_cfg, stream);
    if (fa == 1 && fb == 0)
        return launch_mxg_tiles<GMODE, 1, 0>(a, tile_cfg, stream);
    return launch_mxg_tiles<GMODE, 1, 1>(a, tile_cfg, stream);
}

// rows [first, rows) of a [rows, row_bytes] matrix := 0, first = offs[G]
__global__ __launch_bounds__(256) void zero_rows_from_kernel(uint8_t *c, const int64_t *offs, int G, int64_t rows,
                                                             int64_t row_bytes) {
    const int64_t first = offs[G];
    if (first >= rows)
        return;
    uint8_t      *p     = c + first * row_bytes;
    const int64_t bytes = (rows - first) * row_bytes;
    const int64_t tid = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x, nthr = static_cast<int64_t>(gridDim.x) * 256;
    if ((reinterpret_cast<uintptr_t>(p) & 15) == 0 && (bytes & 15) == 0) {
        u32x4 *q = reinterpret_cast<u32x4 *>(p);
        for (int64_t i = tid; i < bytes / 16; i += nthr)
            q[i] = u32x4{0u, 0u, 0u, 0u};
    } else {
        for (int64_t i = tid; i < bytes; i += nthr)
            p[i] = 0;
    }
}

} // namespace pt

using namespace pt;

extern "C" {

// Word-major copies of the scale arrays (see pt_gemm_mx): worth a pre-pass when the K loop is long.
static int64_t mxg_words(int64_t kblocks) {
    return cdiv(kblocks, 4);
}

size_t pt_grouped_gemm_mx_workspace_bytes(int64_t G, int64_t a_rows, int64_t N, int64_t K) {
    const int64_t W = mxg_words(K / 32);
    return static_cast<size_t>(round_up(a_rows * W * 4, 256) + round_up(G * N * W * 4, 256));
}

size_t pt_grouped_gemm_mx_variable_k_workspace_bytes(int64_t Ml, int64_t Nr, int64_t ld) {
    const int64_t W = mxg_words(ld / 32);
    return static_cast<size_t>(round_up(Ml * W * 4, 256) + round_up(Nr * W * 4, 256));
}

int pt_grouped_gemm_mx(const void *a, int a_dtype, const void *a_scale, int64_t lda, int64_t sa_ld, const void *b,
                       int b_dtype, const void *b_scale, int64_t ldb, int64_t sb_ld, void *c, int c_dtype,
                       const int64_t *group_offs, const int64_t *group_offs_out, int64_t G, int64_t a_rows,
                       int64_t out_rows, int64_t N, int64_t K, void *workspace, size_t workspace_bytes, int tile_cfg,
                       void *stream) {
    const bool fp4 = a_dtype == PT_DTYPE_E2M1X2;
    PT_REQUIRE(fp4 ? b_dtype == PT_DTYPE_E2M1X2 : (is_fp8_dtype(a_dtype) && is_fp8_dtype(b_dtype)),
               "operands must both be fp8 (e4m3 / e5m2) or both e2m1x2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && a_rows >= 0 && out_rows >= 0 && N >= 0, "bad dimensions");
    PT_REQUIRE(K > 0 && K % 32 == 0, "K must be a positive multiple of 32");
    const int64_t kbytes = fp4 ? K / 2 : K;
    PT_REQUIRE(lda == ldb && lda >= kbytes && lda % KSTEP == 0 && lda >= GEMM_MIN_SLABS * KSTEP,
               "row pitches must be equal multiples of 128 bytes, at least 512, that hold K");
    PT_REQUIRE(lda < (1LL << 24), "K must be below 2^24");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 4, "tile_cfg must be 0..4");
    PT_REQUIRE(sa_ld >= K / 32 && sb_ld >= K / 32 && sa_ld % 4 == 0 && sb_ld % 4 == 0,
               "scale rows must hold K / 32 bytes and be 4-byte multiples");
    auto st = static_cast<hipStream_t>(stream);
    if (out_rows == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(c && group_offs, "NULL pointer");
    PT_REQUIRE(aligned_to(c, 16), "output must be 16-byte aligned");
    if (G > 0 && a_rows > 0) {
        PT_REQUIRE(a && b && a_scale && b_scale, "NULL tensor pointer");
        PT_REQUIRE(aligned_to(a, 16) && aligned_to(b, 16), "operands must be 16-byte aligned");
        GemmArgs g{};
        g.A              = static_cast<const uint8_t *>(a);
        g.B              = static_cast<const uint8_t *>(b);
        g.C              = c;
        g.sA             = static_cast<const float *>(a_scale); // E8M0 bytes, [a_rows, sa_ld]
        g.sB             = static_cast<const float *>(b_scale); // E8M0 bytes, [G, N, sb_ld]
        g.M              = a_rows;
        g.N              = N;
        g.K              = lda; // bytes; what lies between K and the pitch is zero
        g.lda            = lda;
        g.ldb            = ldb;
        g.sa_m           = sa_ld;
        g.sb_n           = sb_ld;
        g.kb_valid       = static_cast<int>(K / 32);
        g.out_dtype      = c_dtype;
        g.G              = static_cast<int>(G);
        g.group_offs     = group_offs;
        g.group_offs_out = group_offs_out;
        g.b_gstride      = N * ldb;
        g.sb_gstride     = N * sb_ld / 4; // the kernel steps a 4-byte pointer
        // with a workspace: scale words of one K position of all rows contiguous (two cache lines
        // per scale copy of the kernel instead of sixty-four)
        const int64_t W = mxg_words(K / 32);
        if (workspace != nullptr && aligned_to(workspace, 16) && aligned_to(a_scale, 4) && aligned_to(b_scale, 4) &&
            workspace_bytes >= pt_grouped_gemm_mx_workspace_bytes(G, a_rows, N, K) && sa_ld >= 4 * W && sb_ld >= 4 * W) {
            uint32_t *wa = static_cast<uint32_t *>(workspace);
            uint32_t *wb = wa + round_up(a_rows * W * 4, 256) / 4;
            if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(a_scale), wa, a_rows, W, sa_ld / 4, st))
                return rc;
            if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(b_scale), wb, N, W, sb_ld / 4, st, G))
                return rc;
            g.sA         = reinterpret_cast<const float *>(wa);
            g.sB         = reinterpret_cast<const float *>(wb);
            g.sa_wpitch  = a_rows * 4;
            g.sb_wpitch  = N * 4;
            g.sb_gstride = W * N;
        }
        const int rc = launch_mxg<GROUP_ROWS>(g, fp4 ? 4 : a_dtype == PT_DTYPE_E5M2, b_dtype == PT_DTYPE_E5M2, tile_cfg, st);
        if (rc != PT_OK)
            return rc;
    }
    // rows past the last routed token (over-allocated outputs) read as zero
    const int64_t ES = c_dtype == PT_DTYPE_F32 ? 4 : 2;
    zero_rows_from_kernel<<<256, 256, 0, st>>>(static_cast<uint8_t *>(c), group_offs_out ? group_offs_out : group_offs,
                                               static_cast<int>(G), out_rows, N * ES);
    return check_launch("zero_rows_from_kernel");
}

int pt_grouped_gemm_mx_variable_k(const void *lhs, int lhs_dtype, const void *lhs_scale, const void *rhs, int rhs_dtype,
                                  const void *rhs_scale, void *c, int c_dtype, const int64_t *group_offs, int64_t G,
                                  int64_t Ml, int64_t Nr, int64_t ld, int accumulate, void *workspace,
                                  size_t workspace_bytes, int tile_cfg, void *stream) {
    const bool fp4 = lhs_dtype == PT_DTYPE_E2M1X2;
    PT_REQUIRE(fp4 ? rhs_dtype == PT_DTYPE_E2M1X2 : (is_fp8_dtype(lhs_dtype) && is_fp8_dtype(rhs_dtype)),
               "operands must both be fp8 (e4m3 / e5m2) or both e2m1x2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(G >= 0 && Ml >= 0 && Nr >= 0 && ld >= 0 && ld % (fp4 ? 256 : 128) == 0,
               "bad dimensions (ld must be a multiple of 128 elements, e2m1x2: 256)");
    PT_REQUIRE(ld < (1LL << 24), "at most 2^24 padded rows");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 3, "tile_cfg must be 0..3");
    if (G == 0 || Ml == 0 || Nr == 0)
        return PT_OK;
    PT_REQUIRE(lhs && rhs && lhs_scale && rhs_scale && c && group_offs, "NULL pointer");
    PT_REQUIRE(aligned_to(lhs, 16) && aligned_to(rhs, 16) && aligned_to(c, 16), "operands must be 16-byte aligned");
    GemmArgs g{};
    g.A          = static_cast<const uint8_t *>(lhs); // [Ml, ld]
    g.B          = static_cast<const uint8_t *>(rhs); // [Nr, ld]
    g.C          = c;                                  // [G, Ml, Nr]
    g.sA         = static_cast<const float *>(lhs_scale); // E8M0 bytes, [Ml, ld / 32]
    g.sB         = static_cast<const float *>(rhs_scale);
    g.M          = Ml;
    g.N          = Nr;
    g.K          = 0; // per group
    g.lda        = fp4 ? ld / 2 : ld;
    g.ldb        = g.lda;
    g.sa_m       = ld / 32;
    g.sb_n       = ld / 32;
    g.sa_k       = fp4 ? 2 : 1; // a slab's four (e2m1x2: eight) scale bytes, in steps of the kernel's 4-byte scale pointer
    g.sb_k       = g.sa_k;
    g.kb_valid   = static_cast<int>(ld / 32);
    g.out_dtype  = c_dtype;
    g.accumulate = accumulate;
    g.G          = static_cast<int>(G);
    g.group_offs = group_offs;
    g.c_gstride  = Ml * Nr;
    const int64_t W = mxg_words(ld / 32);
    if (workspace != nullptr && aligned_to(workspace, 16) && aligned_to(lhs_scale, 4) && aligned_to(rhs_scale, 4) &&
        workspace_bytes >= pt_grouped_gemm_mx_variable_k_workspace_bytes(Ml, Nr, ld) && (ld / 32) % 4 == 0) {
        auto      st = static_cast<hipStream_t>(stream);
        uint32_t *wa = static_cast<uint32_t *>(workspace);
        uint32_t *wb = wa + round_up(Ml * W * 4, 256) / 4;
        if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(lhs_scale), wa, Ml, W, ld / 32 / 4, st))
            return rc;
        if (const int rc = launch_transpose_words(static_cast<const uint32_t *>(rhs_scale), wb, Nr, W, ld / 32 / 4, st))
            return rc;
        g.sA        = reinterpret_cast<const float *>(wa);
        g.sB        = reinterpret_cast<const float *>(wb);
        g.sa_wpitch = Ml * 4;
        g.sb_wpitch = Nr * 4;
        g.sa_k      = (fp4 ? 2 : 1) * Ml; // a slab's scale words of all rows, in steps of the kernel's 4-byte scale pointer
        g.sb_k      = (fp4 ? 2 : 1) * Nr;
    }
    return launch_mxg<GROUP_K>(g, fp4 ? 4 : lhs_dtype == PT_DTYPE_E5M2, rhs_dtype == PT_DTYPE_E5M2, tile_cfg,
                               static_cast<hipStream_t>(stream));
}

} // extern "C"
