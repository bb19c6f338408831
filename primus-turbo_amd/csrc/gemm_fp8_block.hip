// hipcc-flags: -mllvm -amdgpu-mfma-vgpr-form=1
// BLOCK-scale instantiations of the FP8 GEMM kernel. Every MFMA result of this mode is an
// input of VALU FMAs (the per-128-K-block scale is applied outside the matrix core), so this
// translation unit is compiled with MFMA destinations in architectural VGPRs: results in
// accumulation registers would cost one v_accvgpr_read per element on top of each FMA.
#include "gemm_fp8_block8.h"

namespace pt {

template <bool SB_VEC, int FA, int FB>
static int launch_block_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 = 256x256, 2 = 256x128, 3 = 128x128 (two workgroups per CU),
    // 4 = 256x256 with eight wavefronts (2-D B scales only)
    if (tile_cfg == 0) {
        tile_cfg = (a.M >= 2048 && a.N >= 1024) ? 2 : 3;
        // 256x256 with eight wavefronts once both dimensions fill the machine with such tiles
        if (!SB_VEC && a.M >= 2048 && a.N >= 2048 && cdiv(a.M, 256) * cdiv(a.N, 256) >= device_cu_count())
            tile_cfg = 4;
    }
    if (tile_cfg == 4) {
        if constexpr (SB_VEC)
            tile_cfg = 2;
        else
            return launch_gemm_block8<FA, FB>(a, stream);
    }
    if (tile_cfg == 3)
        return launch_gemm_cfg<4, 4, SCALE_BLOCK, SB_VEC, FA, FB>(a, stream);
    if (tile_cfg == 1)
        return launch_gemm_cfg<8, 8, SCALE_BLOCK, SB_VEC, FA, FB>(a, stream);
    return launch_gemm_cfg<8, 4, SCALE_BLOCK, SB_VEC, FA, FB>(a, stream);
}

template <bool SB_VEC>
static int launch_block_fmt(const GemmArgs &a, int fa, int fb, int tile_cfg, hipStream_t stream) {
    if (fa == 0 && fb == 0)
        return launch_block_tiles<SB_VEC, 0, 0>(a, tile_cfg, stream);
    if (fa == 0 && fb == 1)
        return launch_block_tiles<SB_VEC, 0, 1>(a, tile_cfg, stream);
    if (fa == 1 && fb == 0)
        return launch_block_tiles<SB_VEC, 1, 0>(a, tile_cfg, stream);
    return launch_block_tiles<SB_VEC, 1, 1>(a, tile_cfg, stream);
}

int launch_gemm_block(const GemmArgs &a, int fa, int fb, bool sb_vec, int tile_cfg, hipStream_t stream) {
    return sb_vec ? launch_block_fmt<true>(a, fa, fb, tile_cfg, stream)
                  : launch_block_fmt<false>(a, fa, fb, tile_cfg, stream);
}

} // namespace pt
