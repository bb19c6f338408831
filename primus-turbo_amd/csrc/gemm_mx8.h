// MX-scaled GEMM (MXFP8 / MXFP4, NT) with a 256 x 256 workgroup tile and EIGHT wavefronts (two per
// SIMD): C[M, N] = sum over 32-wide K blocks of (A_kb . B_kb^T) * 2^(ea[m, kb] + eb[n, kb]), the E8M0
// exponents applied by the matrix core (v_mfma_scale_f32_16x16x128_f8f6f4). Semantics as
// gemm_fp8_nt_kernel<SCALE_MX> (primus_turbo/pytorch/kernels/gemm/gemm_fp8_impl.py, MX_BLOCKWISE;
// kernels/gemm/gemm_fp4_impl.py).
//
// Why next to the four-wavefront kernel: an MXFP4 slab holds 256 codes per row, i.e. 128 MFMAs of
// 16 clocks per SIMD; with one wavefront per SIMD every LDS read, copy request and wait of that
// wavefront sits between two MFMAs of the same instruction stream, and the matrix pipes were 53 %
// busy. Here two wavefronts share a SIMD (each owns 128 x 64 of the tile, 128 sums in AGPRs), and
// one issues MFMAs while the other is busy with anything else. The slab schedule is that of
// gemm_fp8_block8.h without its fold: B fragments resident, A fragments through a ring of four,
// two LDS stages, one barrier per slab before row group 6, the copies of the slab after next split
// into B rows + scale words (row groups 6, 7) and A rows (row groups 0..3 of the next slab).
// Scale words: wavefronts 0..3 copy the words of the tile's 256 rows (64 each), wavefronts 4..7
// those of its 256 columns, one word per slab (two for MXFP4); every wavefront reads the bytes of
// its 8 + 4 fragments from the current stage at the start of the slab. GROUP_ROWS enumerates
// (group, tile) pairs from the device-side offsets as gemm_fp8_block8.h does (MoE forward / dgrad).
#pragma once
#include "gemm_fp8_block8.h"

namespace pt {

template <int FA, int FB, int GMODE = GROUP_NONE>
__global__ __launch_bounds__(B8_THREADS) void gemm_mx8_kernel(const GemmArgs a) {
    static_assert(GMODE == GROUP_NONE || GMODE == GROUP_ROWS, "row groups or none");
    constexpr int  TM = B8_TM, TN = B8_TN, BM = B8_BM, BN = B8_BN;
    constexpr bool F4 = FA == 4;
    static_assert((FA == 4) == (FB == 4), "FP4 operands come in pairs");
    constexpr int NH = F4 ? 2 : 1;                  // MFMAs per fragment pair = scale words per row and slab
    constexpr int A_BYTES = B8_A_BYTES, SC = B8_A_BYTES + B8_B_BYTES;
    constexpr int STAGE = SC + NH * 2048;           // per half: 256 row words, 256 column words
    constexpr int LA = B8_LA, LB = B8_LB, NL = LA + LB + NH;
    constexpr int P1 = LB + NH;                     // copies of a slab issued in row groups 6, 7
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 2, wn = wave & 3;
    const int lm = lane & 15, lg = lane >> 4;

    const uint32_t frag_off_lo = lm * KSTEP + ((lg ^ swz(lm)) << 4);
    const uint32_t frag_off_hi = lm * KSTEP + (((4 + lg) ^ swz(lm)) << 4);

    // ---- tile list (row groups: tiles before group g, from the device-side offsets) ----
    int *prefix = reinterpret_cast<int *>(smem + B8_NSTAGE * STAGE);
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
    const int KT_ALL = static_cast<int>(a.K / KSTEP); // >= 2
    int       tile   = blockIdx.x;
    if (tile >= total || KT_ALL < 2)
        return;
    int     g_cur = 0, g_nxt = 0;
    TileCtx cur_t = make_tile<BM, BN, GMODE, F4>(a, tile, prefix, g_cur);
    g_nxt         = g_cur;
    TileCtx nxt_t = cur_t;

    // ---- loader ----
    // scale addressing in bytes: from one row (column) to the next, and from one 32-bit word of a
    // row to its next (row-major arrays, or the word-major copy)
    const bool     wordmajor = a.sa_wpitch != 0;
    const bool     sc_is_a   = wave < 4;
    const uint32_t sc_rowp   = wordmajor ? 4u : static_cast<uint32_t>(sc_is_a ? a.sa_m : a.sb_n);
    const uint32_t sc_wordp  = wordmajor ? static_cast<uint32_t>(sc_is_a ? a.sa_wpitch : a.sb_wpitch) : 4u;
    uint32_t       off[NL];
    {
        const int lrow = lane >> 3, pchk = lane & 7;
#pragma unroll
        for (int j = 0; j < LA + LB; ++j) {
            const bool isA = j < LA;
            const int  row = ((isA ? j : j - LA) * B8_WAVES + wave) * 8 + lrow;
            off[j] = static_cast<uint32_t>(row * (isA ? a.lda : a.ldb)) + ((pchk ^ swz(row)) << 4);
        }
#pragma unroll
        for (int h = 0; h < NH; ++h) // word h of tile row (column) 64 (wave % 4) + lane
            off[LA + LB + h] = static_cast<uint32_t>((wave & 3) * 64 + lane) * sc_rowp + h * sc_wordp;
    }
    const uint8_t *ld_ga, *ld_gb;     // slab the loader points at
    uint32_t       ld_na, ld_nb;      // bytes from there to the end of the tile's rows
    int            ld_kt;
    const uint8_t *ld_sc, *ld_sc_end; // this wavefront's scale source for the loader's slab
    auto           as_bytes = [](const float *p) { return reinterpret_cast<const uint8_t *>(p); };
    const int64_t  words    = (a.kb_valid + 3) / 4;
    const int64_t  sc_extent = sc_is_a ? (wordmajor ? words * a.sa_wpitch : (a.M - 1) * a.sa_m + a.kb_valid)
                                       : (wordmajor ? words * a.sb_wpitch : (a.N - 1) * a.sb_n + a.kb_valid);
    const int64_t  sc_step   = static_cast<int64_t>(NH) * sc_wordp; // bytes per slab
    auto scale_src = [&](const TileCtx &t) {
        return sc_is_a ? as_bytes(t.sA) + t.m0 * sc_rowp : as_bytes(t.sB) + t.n0 * sc_rowp;
    };
    auto scale_end = [&](const TileCtx &t) { return as_bytes(sc_is_a ? t.sA : t.sB) + sc_extent; };
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
    // copy number L of the loader's slab into stage b: [0, LA) A rows, [LA, LA + LB) B rows, then scale words
    auto issue_copy = [&](auto lc, int b) {
        constexpr int L   = lc;
        uint8_t      *dst = smem + b * STAGE;
#if defined(__HIP_DEVICE_COMPILE__) // the buffer resource type only exists in the device pass
        constexpr uint32_t RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format
        if constexpr (L >= LA + LB) {
            constexpr int H = L - LA - LB;
            // nothing is read for a slab of zero padding beyond the K blocks the arrays hold
            // (whatever lies there must not meet the matrix core: an E8M0 NaN would stick)
            const int64_t  n     = ld_sc_end - ld_sc;
            const bool     valid = (ld_kt * NH + H) * 4 < a.kb_valid;
            const uint32_t bytes = (n <= 0 || !valid) ? 0u : (n > 0x7fffffff ? 0x7fffffffu : static_cast<uint32_t>(n));
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_sc), 0, bytes, RSRC_FLAGS);
            // stage area: [half H][row words 1 KB | column words 1 KB], 256 B per wavefront
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + SC + H * 2048 + wave * 256), 4, off[L], 0, 0, 0);
        } else if constexpr (L < LA) {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_ga), 0, ld_na, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + (L * B8_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        } else {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_gb), 0, ld_nb, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + A_BYTES + ((L - LA) * B8_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        }
#endif
    };
    // the copies of a slab in issue order: B rows, scale words (first part), then A rows (second part)
    auto issue_nth = [&](auto cc, int b) {
        constexpr int C = cc;
        issue_copy(std::integral_constant<int, (C < LB ? LA + C : (C < P1 ? LA + LB + (C - LB) : C - P1))>{}, b);
    };

    // ---- registers of the K loop ----
    f32x4    acc[TM][TN];
    i32x8    fb[TN], fa[4];
    uint32_t mxa[TM][NH], mxb[TN][NH]; // lane (r, g): the E8M0 byte of fragment row r and K block g
    int      buf = 0;

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
        const uint8_t *ra = stage + SC + (wm * (TM * 16) + lm) * 4 + lg;
        const uint8_t *rb = stage + SC + 1024 + (wn * (TN * 16) + lm) * 4 + lg;
#pragma unroll
        for (int h = 0; h < NH; ++h) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                mxa[i][h] = ra[h * 2048 + i * 64];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                mxb[j][h] = rb[h * 2048 + j * 64];
        }
    };
    const uint32_t a_part = wm * (TM * 16) * KSTEP;
    const uint32_t b_part = A_BYTES + wn * (TN * 16) * KSTEP;

    // ---- pipeline start: slab 0 whole, first part of slab 1 ----
    loader_to(cur_t);
    static_for<0, NL>([&](auto c) { issue_nth(c, 0); });
    advance_loader();
    static_for<0, P1>([&](auto c) { issue_nth(c, 1); });
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(P1) : "memory");
    __builtin_amdgcn_s_barrier();
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
            nxt_t = make_tile<BM, BN, GMODE, F4>(a, next_tile, prefix, g_nxt);

        // one K slab per iteration; the body stays a single basic block
        for (int kt = 0; kt < KT_ALL; ++kt) {
            const uint8_t *cur = smem + buf * STAGE;
            const uint8_t *nxt = smem + (buf ^ 1) * STAGE;
            read_scales(cur);

            static_for<0, TM>([&](auto ic) {
                constexpr int i = ic;
                if constexpr (i == 6) {
                    // ---- the slab's barrier: my copies of the next slab have landed (nothing
                    // younger is in flight) and my reads of the current stage are complete ----
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                }
                // A fragment two row groups ahead
                if constexpr (i + 2 < TM)
                    fa[(i + 2) % 4] = ldfrag(cur + a_part, i + 2);
                else
                    fa[(i + 2) % 4] = ldfrag(nxt + a_part, i + 2 - TM);
                __builtin_amdgcn_sched_barrier(0);
                // the MFMAs of the row group: (h, j) with j fastest, so that the two halves of an
                // MXFP4 fragment pair, which add into the same sums, are four instructions apart
                static_for<0, NH * TN>([&](auto sc) {
                    constexpr int h = sc / TN, j = sc % TN;
                    if constexpr (F4) {
                        const i32x8 &bf = fb[j], &af = fa[i % 4];
                        const i32x4  bq = h ? __builtin_shufflevector(bf, bf, 4, 5, 6, 7) : __builtin_shufflevector(bf, bf, 0, 1, 2, 3);
                        const i32x4  aq = h ? __builtin_shufflevector(af, af, 4, 5, 6, 7) : __builtin_shufflevector(af, af, 0, 1, 2, 3);
                        mfma_inplace_f4(acc[i][j], bq, aq, mxb[j][h], mxa[i][h]);
                    } else {
                        mfma_inplace<FA, FB>(acc[i][j], fb[j], fa[i % 4], mxb[j][0], mxa[i][0]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (i == TM - 1 && h == NH - 1)
                        fb[j] = ldfrag(nxt + b_part, j); // dead from here on: refill from the next slab
                    // second part (A rows) of the next slab's copies: row groups 0..3, into the next stage
                    if constexpr (i < LA && sc == 1)
                        issue_nth(std::integral_constant<int, P1 + i>{}, buf ^ 1);
                    // first part (B rows, scale words) of the slab after next: row groups 6 and 7, into
                    // the stage the barrier has just freed
                    if constexpr (i >= 6) {
                        constexpr int s = (i - 6) * NH * TN + sc; // 0 .. 2 NH TN - 1
                        if constexpr (s >= 1 && s <= P1)
                            issue_nth(std::integral_constant<int, s - 1>{}, buf);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
                if constexpr (i == LA)
                    advance_loader(); // the next slab is requested in full: on to the one after
            });
            buf ^= 1;
        }

        // the epilogue reads the accumulators with hand-written instructions the compiler's hazard
        // tracking does not see: let the last MFMA's write-back finish first
        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
        const int64_t wm_base = cur_t.m0 + wm * (TM * 16), wn_base = cur_t.n0 + wn * (TN * 16);
        epilogue<TM, TN, SCALE_MX, true>(a, acc, cur_t.C, cur_t.sA, cur_t.sB, cur_t.m_end, wm_base, wn_base, lane);

        if (next_tile >= total)
            break;
        tile  = next_tile;
        cur_t = nxt_t;
    }
    // no copy into this workgroup's LDS may still be in flight when the LDS is handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int FA, int FB, int GMODE = GROUP_NONE> static int launch_gemm_mx8(const GemmArgs &args_in, hipStream_t stream) {
    constexpr int STAGES  = B8_NSTAGE * (B8_A_BYTES + B8_B_BYTES + (FA == 4 ? 2 : 1) * 2048);
    constexpr int MAX_G   = 2048;
    constexpr int LDS_MAX = STAGES + (GMODE == GROUP_ROWS ? (MAX_G + 2) * 4 : 0);
    static_assert(LDS_MAX <= 160 * 1024, "tile configuration does not fit the LDS");
    GemmArgs a = args_in;
    a.gmode    = GMODE;
    a.tiles_m  = static_cast<int>(cdiv(a.M, B8_BM));
    a.tiles_n  = static_cast<int>(cdiv(a.N, B8_BN));
    if (GMODE != GROUP_NONE && a.G > MAX_G)
        return fail(PT_ERR_INVALID_ARGUMENT, "grouped gemm_mx: too many groups for this tile configuration");
    if (a.sa_shift != 0 || a.sb_shift != 0 || (a.sa_wpitch == 0 && (a.sa_m % 4 != 0 || a.sb_n % 4 != 0)) ||
        (a.sa_wpitch != 0) != (a.sb_wpitch != 0) || a.sa_wpitch % 4 != 0 || a.sb_wpitch % 4 != 0 ||
        reinterpret_cast<uintptr_t>(a.sA) % 4 != 0 || reinterpret_cast<uintptr_t>(a.sB) % 4 != 0)
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_mx: scale rows must be 4-byte aligned");
    if (a.K / KSTEP < 2)
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_mx: K too short for the 256x256 tile");
    auto kern = gemm_mx8_kernel<FA, FB, GMODE>;
    static std::atomic<unsigned long long> attr_set{0};
    int                                    dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return fail(PT_ERR_LAUNCH, "gemm_mx: no current device (or a device index beyond 63)");
    const unsigned long long dev_bit = 1ULL << dev;
    if (!(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_MAX) != hipSuccess)
            return fail(PT_ERR_LAUNCH, "gemm_mx: cannot raise the dynamic LDS limit");
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    const int     LDS   = STAGES + (GMODE == GROUP_ROWS ? (a.G + 2) * 4 : 0);
    const int64_t total = GMODE == GROUP_ROWS ? (static_cast<int64_t>(a.tiles_m) + a.G) * a.tiles_n
                                              : static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    int64_t       grid  = device_cu_count(); // one workgroup per CU (LDS-limited), persistent
    if (grid > total)
        grid = total;
    if (grid <= 0)
        return PT_OK;
    kern<<<static_cast<unsigned>(grid), B8_THREADS, LDS, stream>>>(a);
    return check_launch("gemm_mx8_kernel");
}

} // namespace pt
