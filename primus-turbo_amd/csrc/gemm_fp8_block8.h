// Block-scaled FP8 GEMM with a 256 x 256 workgroup tile and EIGHT wavefronts (two per SIMD):
//   C[M, N] = sum_kb (A_kb . B_kb^T) * sA[m, kb] * sB[n / 128, kb]      (128-wide K blocks)
// (semantics: primus_turbo/triton/gemm/gemm_fp8_kernel.py:871-1013, grouped rows:
// primus_turbo/triton/grouped_gemm/grouped_gemm_fp8_kernel.py:1405-1556).
//
// Why a second kernel next to gemm_fp8_nt_kernel<SCALE_BLOCK>: the per-block scale is applied
// by VALU FMAs on every MFMA result, so the running sums have to live in architectural VGPRs.
// With four wavefronts a 256 x 256 tile would need 256 of them per lane for the sums alone,
// which is why the four-wavefront kernel stops at 256 x 128 and is bound by the L2 -> LDS
// copies (47 B / clock / CU at full MFMA rate). Here each wavefront owns 128 x 64 (128 sums
// per lane), the tile needs 31 B / clock / CU, and the second wavefront of a SIMD issues MFMAs
// while the first waits for its fold, an LDS read or the barrier.
//
// Schedule of one 128-byte K slab (per wavefront, wm = wave / 4, wn = wave % 4):
//   * the four B fragments of the slab are in registers when it starts; A fragments stream
//     through a ring of four, read two row groups ahead of their MFMAs;
//   * row group i = 0..7: four MFMAs (i, j = 0..3) into a ring of four result tiles, each
//     folded into the sums three MFMAs later with sA[row] * sB (one value per lane and i);
//   * two LDS stages. One barrier per slab, before row group 6: everyone's copies of the next
//     slab have landed and everyone has finished reading the current stage. From there on
//     the wavefront reads the next slab's first A fragments, its scales and (after its last
//     use of each B fragment) the B fragments, and all nine copies of the slab after next (B
//     rows, scales, A rows) go into the stage just freed during row groups 6 and 7: every
//     copy a barrier waits for is then older than the stores of a result tile written in
//     between, which is what lets that wait leave the stores in flight;
//   * the slab sequence runs across tile boundaries (persistent grid), the loader changing
//     tile by swapping uniform values as in the four-wavefront kernel.
#pragma once
#include "gemm_fp8_kernel.h"

namespace pt {

constexpr int B8_THREADS = 512, B8_WAVES = 8;
constexpr int B8_TM = 8, B8_TN = 4;     // MFMA tiles per wavefront: 128 rows x 64 columns
constexpr int B8_BM = 256, B8_BN = 256; // 2 x 4 wavefronts
constexpr int B8_A_BYTES = B8_BM * KSTEP, B8_B_BYTES = B8_BN * KSTEP;
// scale words of a stage: the fp32 scale of each of the 256 tile rows (copied 64 rows per
// instruction by wavefronts 0..3), then four 256-byte areas into which wavefronts 4..7 each
// copy the B block scales of the tile's two 128-column blocks (only the first area is read;
// the others keep the code of all wavefronts identical)
constexpr int B8_SC_A   = B8_A_BYTES + B8_B_BYTES;
constexpr int B8_SC_B   = B8_SC_A + 1024;
constexpr int B8_STAGE  = B8_SC_B + 1024;
constexpr int B8_NSTAGE = 2;
constexpr int B8_LA = B8_BM / 8 / B8_WAVES, B8_LB = B8_BN / 8 / B8_WAVES; // row copies per wavefront and slab
constexpr int B8_NL = B8_LA + B8_LB + 1;                                  // + one scale copy
constexpr int B8_P1 = B8_LB + 1; // copies of a slab issued in row groups 6, 7 (B rows, scales)

template <int FA, int FB, int GMODE>
__global__ __launch_bounds__(B8_THREADS) void gemm_fp8_block8_kernel(const GemmArgs a) {
    static_assert(GMODE == GROUP_NONE || GMODE == GROUP_ROWS, "row groups or none");
    constexpr int TM = B8_TM, TN = B8_TN, BM = B8_BM, BN = B8_BN;
    constexpr int A_BYTES = B8_A_BYTES, STAGE = B8_STAGE, NSTAGE = B8_NSTAGE;
    constexpr int LA = B8_LA, LB = B8_LB, NL = B8_NL;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int lm = lane & 15, lg = lane >> 4;

    const uint32_t frag_off_lo = lm * KSTEP + ((lg ^ swz(lm)) << 4);
    const uint32_t frag_off_hi = lm * KSTEP + (((4 + lg) ^ swz(lm)) << 4);

    // ---- tile list ----
    int *prefix = reinterpret_cast<int *>(smem + NSTAGE * STAGE); // GROUP_ROWS: tiles before group g
    int  total;
    if constexpr (GMODE == GROUP_ROWS) {
        for (int g = tid; g < a.G; g += B8_THREADS) {
            const int64_t *o   = a.group_offs_out != nullptr ? a.group_offs_out : a.group_offs;
            const int64_t rows = o[g + 1] - o[g];
            prefix[g + 1]      = static_cast<int>((rows + BM - 1) / BM) * a.tiles_n;
        }
        __syncthreads();
        if (tid == 0) {
            int run   = 0;
            prefix[0] = 0;
            for (int g = 1; g <= a.G; ++g) {
                run += prefix[g];
                prefix[g] = run;
            }
        }
        __syncthreads();
        total = __builtin_amdgcn_readfirstlane(prefix[a.G]);
    } else {
        total = a.tiles_m * a.tiles_n;
    }
    const int KT_ALL = static_cast<int>(a.K / KSTEP); // >= 2 (the host pads K to four slabs at least)
    int       tile   = blockIdx.x;
    if (tile >= total || KT_ALL < 2)
        return;
    int     g_cur = 0, g_nxt = 0;
    TileCtx cur_t = make_tile<BM, BN, GMODE>(a, tile, prefix, g_cur);
    g_nxt         = g_cur;
    TileCtx nxt_t = cur_t;

    // ---- loader ----
    // lane offsets of the copies inside a slab: A rows, B rows, the wavefront's scale words
    uint32_t off[NL];
    {
        const int lrow = lane >> 3, pchk = lane & 7;
#pragma unroll
        for (int j = 0; j < LA + LB; ++j) {
            const bool isA = j < LA;
            const int  row = ((isA ? j : j - LA) * B8_WAVES + wave) * 8 + lrow;
            off[j] = static_cast<uint32_t>(row * (isA ? a.lda : a.ldb)) + ((pchk ^ swz(row)) << 4);
        }
        if (wave < 4) // scale of tile row 64 wave + lane
            off[NL - 1] = static_cast<uint32_t>((wave * 64 + lane) >> a.sa_shift) * static_cast<uint32_t>(a.sa_m) * 4u;
        else          // scale of the tile's column block `lane` (two blocks; the other lanes read nothing)
            off[NL - 1] = lane < BN / 128 ? static_cast<uint32_t>(lane) * static_cast<uint32_t>(a.sb_n) * 4u : 0x7ffffff0u;
    }
    const bool     sc_is_a = wave < 4;
    const uint8_t *ld_ga, *ld_gb; // slab the loader points at
    uint32_t       ld_na, ld_nb;  // bytes from there to the end of the tile's rows
    int            ld_kt;
    const uint8_t *ld_sc, *ld_sc_end; // this wavefront's scale source for the loader's slab
    const int64_t  sa_extent = (((a.M - 1) >> a.sa_shift) * a.sa_m + (a.kb_valid - 1) * a.sa_k + 1) * 4;
    const int64_t  sb_extent = (((a.N - 1) >> a.sb_shift) * a.sb_n + (a.kb_valid - 1) * a.sb_k + 1) * 4;
    const int64_t  sc_step   = (sc_is_a ? a.sa_k : a.sb_k) * 4;
    auto           as_bytes  = [](const float *p) { return reinterpret_cast<const uint8_t *>(p); };
    auto scale_src = [&](const TileCtx &t) {
        return sc_is_a ? as_bytes(t.sA) + ((t.m0 >> a.sa_shift) * a.sa_m) * 4
                       : as_bytes(t.sB) + ((t.n0 >> a.sb_shift) * a.sb_n) * 4;
    };
    auto scale_end = [&](const TileCtx &t) { return sc_is_a ? as_bytes(t.sA) + sa_extent : as_bytes(t.sB) + sb_extent; };
    auto loader_to = [&](const TileCtx &t) {
        ld_ga     = t.Ag;
        ld_gb     = t.Bg;
        ld_na     = t.rows_a * static_cast<uint32_t>(a.lda);
        ld_nb     = t.rows_b * static_cast<uint32_t>(a.ldb);
        ld_kt     = 0;
        ld_sc     = scale_src(t);
        ld_sc_end = scale_end(t);
    };
    auto advance_loader = [&]() {
        const bool wrap = ld_kt + 1 == KT_ALL;
        ld_kt     = wrap ? 0 : ld_kt + 1;
        ld_ga     = wrap ? nxt_t.Ag : ld_ga + KSTEP;
        ld_gb     = wrap ? nxt_t.Bg : ld_gb + KSTEP;
        ld_na     = wrap ? nxt_t.rows_a * static_cast<uint32_t>(a.lda) : ld_na - KSTEP;
        ld_nb     = wrap ? nxt_t.rows_b * static_cast<uint32_t>(a.ldb) : ld_nb - KSTEP;
        ld_sc     = wrap ? scale_src(nxt_t) : ld_sc + sc_step;
        ld_sc_end = wrap ? scale_end(nxt_t) : ld_sc_end;
    };
    // copy number L of the loader's slab into stage b: [0, LA) A rows, [LA, LA + LB) B rows, then scales
    auto issue_copy = [&](auto lc, int b) {
        constexpr int L   = lc;
        uint8_t      *dst = smem + b * STAGE;
#if defined(__HIP_DEVICE_COMPILE__) // the buffer resource type only exists in the device pass
        constexpr uint32_t RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format
        if constexpr (L == NL - 1) {
            // nothing is read for a slab of zero padding beyond the K blocks the arrays hold
            const int64_t  n     = ld_sc_end - ld_sc;
            const uint32_t bytes = (n <= 0 || ld_kt >= a.kb_valid) ? 0u : (n > 0x7fffffff ? 0x7fffffffu : static_cast<uint32_t>(n));
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_sc), 0, bytes, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + B8_SC_A + wave * 256), 4, off[L], 0, 0, 0);
        } else if constexpr (L < LA) {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_ga), 0, ld_na, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + (L * B8_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        } else {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_gb), 0, ld_nb, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + A_BYTES + ((L - LA) * B8_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        }
#endif
    };
    // the copies of a slab in issue order: B rows, scales (first part), then A rows (second part)
    auto issue_nth = [&](auto cc, int b) {
        constexpr int C = cc;
        issue_copy(std::integral_constant<int, (C < LB ? LA + C : (C == LB ? NL - 1 : C - B8_P1))>{}, b);
    };

    // ---- registers of the K loop ----
    f32x4 acc[TM][TN];
    i32x8 fb[TN], fa[4];
    float sn[TM], sbn; // scales of the next slab as read from its stage
    float sc[TM];      // sA[row] * sB of the slab being multiplied
    int   buf = 0;

    auto ldfrag = [&](const uint8_t *part, int f) {
        const uint8_t *p  = part + f * 16 * KSTEP;
        const u32x4    lo = *reinterpret_cast<const u32x4 *>(p + frag_off_lo);
        const u32x4    hh = *reinterpret_cast<const u32x4 *>(p + frag_off_hi);
        i32x8          r;
        r[0] = lo.x; r[1] = lo.y; r[2] = lo.z; r[3] = lo.w;
        r[4] = hh.x; r[5] = hh.y; r[6] = hh.z; r[7] = hh.w;
        return r;
    };
    auto read_scales = [&](const uint8_t *stage) {
        const float *sa = reinterpret_cast<const float *>(stage + B8_SC_A) + wm * (TM * 16) + lm;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            sn[i] = sa[i * 16];
        sbn = reinterpret_cast<const float *>(stage + B8_SC_B)[wn >> 1];
    };
    const uint32_t a_part = wm * (TM * 16) * KSTEP;
    const uint32_t b_part = A_BYTES + wn * (TN * 16) * KSTEP;

    // ---- pipeline start: slabs 0 and 1 ----
    // (the loader steps past slab 1 here: with two slabs per tile that is the next tile already)
    if (tile + static_cast<int>(gridDim.x) < total)
        nxt_t = make_tile<BM, BN, GMODE>(a, tile + gridDim.x, prefix, g_nxt);
    loader_to(cur_t);
    static_for<0, NL>([&](auto c) { issue_nth(c, 0); });
    advance_loader();
    static_for<0, NL>([&](auto c) { issue_nth(c, 1); });
    advance_loader();
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
    __builtin_amdgcn_s_barrier();
    // Stores of the result tile this wavefront has just written that may still be in flight (0, or
    // the count of the epilogue's straight-line path). All copies of a slab are issued a slab
    // ahead, so behind an epilogue those stores are the only memory operations younger than the
    // copies the next barrier waits for: memory operations retire in order, and leaving that many
    // outstanding waits for the copies without waiting for the stores to be acknowledged.
    int pending = 0;
    read_scales(smem);
#pragma unroll
    for (int j = 0; j < TN; ++j)
        fb[j] = ldfrag(smem + b_part, j);
    fa[0] = ldfrag(smem + a_part, 0);
    fa[1] = ldfrag(smem + a_part, 1);

    while (true) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int next_tile = tile + gridDim.x;
        nxt_t               = cur_t;
        if (next_tile < total)
            nxt_t = make_tile<BM, BN, GMODE>(a, next_tile, prefix, g_nxt);

        // one K slab per iteration; the body stays a single basic block
        for (int kt = 0; kt < KT_ALL; ++kt) {
            const uint8_t *cur = smem + buf * STAGE;
            const uint8_t *nxt = smem + (buf ^ 1) * STAGE;
#pragma unroll
            for (int i = 0; i < TM; ++i)
                sc[i] = sn[i] * sbn;

            constexpr int DEPTH = 3, RING = DEPTH + 1, TILES = TM * TN;
            f32x4         ring[RING];
            auto          fold = [&](int t) {
                const int    i = t / TN, j = t % TN;
                const f32x4 &p = ring[t % RING];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    acc[i][j][e] = fmaf(p[e], sc[i], acc[i][j][e]);
            };

            static_for<0, TM>([&](auto ic) {
                constexpr int i = ic;
                if constexpr (i == 6) {
                    // ---- the slab's barrier: my copies of the next slab have landed (nothing
                    // younger is in flight) and my reads of the current stage are complete ----
                    // (the case distinction lives inside the asm statement so that the slab stays
                    // one basic block for the compiler)
                    asm volatile("s_cmp_eq_u32 %0, 16\n\t"
                                 "s_cbranch_scc1 .Lb16_%=\n\t"
                                 "s_cmp_eq_u32 %0, 32\n\t"
                                 "s_cbranch_scc1 .Lb32_%=\n\t"
                                 "s_waitcnt vmcnt(0) lgkmcnt(0)\n\t"
                                 "s_branch .Lbend_%=\n"
                                 ".Lb16_%=:\n\t"
                                 "s_waitcnt vmcnt(16) lgkmcnt(0)\n\t"
                                 "s_branch .Lbend_%=\n"
                                 ".Lb32_%=:\n\t"
                                 "s_waitcnt vmcnt(32) lgkmcnt(0)\n"
                                 ".Lbend_%=:"
                                 :
                                 : "s"(pending)
                                 : "memory", "scc");
                    pending = 0;
                    __builtin_amdgcn_s_barrier();
                    read_scales(nxt);
                }
                // A fragment two row groups ahead
                if constexpr (i + 2 < TM)
                    fa[(i + 2) % 4] = ldfrag(cur + a_part, i + 2);
                else
                    fa[(i + 2) % 4] = ldfrag(nxt + a_part, i + 2 - TM);
                __builtin_amdgcn_sched_barrier(0);
                static_for<0, TN>([&](auto jc) {
                    constexpr int j = jc, t = i * TN + j;
                    ring[t % RING] = mfma_fp8<FA, FB>(fb[j], fa[i % 4], f32x4{0.f, 0.f, 0.f, 0.f});
                    if constexpr (t >= DEPTH)
                        fold(t - DEPTH);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (i == TM - 1)
                        fb[j] = ldfrag(nxt + b_part, j); // dead from here on: refill from the next slab
                    // all copies of the slab after next: row groups 6 and 7, into the stage the
                    // barrier has just freed (nine copies in eight MFMA slots)
                    if constexpr (i >= 6) {
                        constexpr int s = (i - 6) * TN + j; // 0..7
                        issue_nth(std::integral_constant<int, s>{}, buf);
                        if constexpr (s == 7) {
                            issue_nth(std::integral_constant<int, 8>{}, buf);
                            advance_loader();
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
#pragma unroll
            for (int t = TILES - DEPTH; t < TILES; ++t)
                fold(t);
            buf ^= 1;
        }

        const int64_t wm_base = cur_t.m0 + wm * (TM * 16), wn_base = cur_t.n0 + wn * (TN * 16);
        // stores of the epilogue's straight-line path (0, 16 or 32: the cases of the barrier's wait)
        pending = __builtin_amdgcn_readfirstlane(
            epilogue<TM, TN, SCALE_BLOCK, false>(a, acc, cur_t.C, cur_t.sA, cur_t.sB, cur_t.m_end, wm_base, wn_base, lane));
        static_assert(TM * TN == 32, "the barrier's wait distinguishes 16 and 32 stores in flight");

        if (next_tile >= total)
            break;
        tile  = next_tile;
        cur_t = nxt_t;
    }
    // no copy into this workgroup's LDS may still be in flight when the LDS is handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int FA, int FB, int GMODE = GROUP_NONE>
static int launch_gemm_block8(const GemmArgs &args_in, hipStream_t stream) {
    constexpr int STAGES  = B8_NSTAGE * B8_STAGE;
    constexpr int MAX_G   = 2048;
    constexpr int LDS_MAX = STAGES + (GMODE == GROUP_ROWS ? (MAX_G + 2) * 4 : 0);
    static_assert(LDS_MAX <= 160 * 1024, "tile configuration does not fit the LDS");
    GemmArgs a = args_in;
    a.gmode    = GMODE;
    a.tiles_m  = static_cast<int>(cdiv(a.M, B8_BM));
    a.tiles_n  = static_cast<int>(cdiv(a.N, B8_BN));
    if (GMODE != GROUP_NONE && a.G > MAX_G)
        return fail(PT_ERR_INVALID_ARGUMENT, "grouped gemm: too many groups for this tile configuration");
    if (a.sb_shift != 7 || (GMODE == GROUP_ROWS && a.sa_shift != 0))
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_fp8: unsupported block-scale layout for the 256x256 tile");
    if (a.K / KSTEP < 2)
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_fp8: K too short for the 256x256 tile");
    auto kern = gemm_fp8_block8_kernel<FA, FB, GMODE>;
    static std::atomic<unsigned long long> attr_set{0};
    int                                    dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return fail(PT_ERR_LAUNCH, "gemm_fp8: no current device (or a device index beyond 63)");
    const unsigned long long dev_bit = 1ULL << dev;
    if (!(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_MAX) !=
            hipSuccess)
            return fail(PT_ERR_LAUNCH, "gemm_fp8: cannot raise the dynamic LDS limit");
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    const int lds = STAGES + (GMODE == GROUP_ROWS ? (a.G + 2) * 4 : 0);
    int64_t   total = GMODE == GROUP_ROWS ? (static_cast<int64_t>(a.tiles_m) + a.G) * a.tiles_n
                                          : static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    int64_t   grid  = device_cu_count(); // one workgroup per CU (LDS-limited), persistent
    if (grid > total)
        grid = total;
    if (grid <= 0)
        return PT_OK;
    kern<<<static_cast<unsigned>(grid), B8_THREADS, lds, stream>>>(a);
    return check_launch("gemm_fp8_block8_kernel");
}

} // namespace pt
