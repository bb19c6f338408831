// Variable-K grouped FP8 GEMM (the wgrad of a grouped linear layer) with the 256 x 256 tile and
// eight wavefronts of gemm_fp8_block8.h:
//   C[g][m, n] (+)= sum over the 128-row blocks kb of group g:
//                    (A[m, kb] . B[n, kb]^T) * sA[kb, m] * sB[kb, n]
// A [M, ld] and B [N, ld] hold the K-contiguous (transposed) operands of all groups side by side,
// group g occupying K positions [offs[g], offs[g + 1]) (multiples of 128); both carry one scale per
// row and 128-wide K block (semantics: primus_turbo/triton/grouped_gemm/grouped_gemm_fp8_kernel.py:
// 1559-1720, the variable-K kernel of the blockwise recipe).
//
// Because the groups lie side by side along K, an output position (tm, tn) can stream through the
// K ranges of consecutive groups without ever restarting its pipeline: the slab sequence simply
// continues, and at a group boundary the running sums are written to C[g] and cleared while the
// next group's first slabs are already in registers and in flight. A unit of work is therefore
// one output position times a run of consecutive groups ("chunk"); the groups are cut into
// `chunks` runs of about equal K length so that the number of units suits the grid, all
// workgroups walk the chunks in the same order (the operand panels of a chunk are shared through
// the caches while they are hot), and an empty group costs one store of zeros.
//
// Differences from the dense kernel's slab: both operands have per-row scales, so wavefronts 4..7
// copy the 256 column scales of the slab (as wavefronts 0..3 copy the row scales), a wavefront
// reads its 8 + 16 scale values from the current stage at the start of the slab, and the fold
// costs a multiply and an FMA per value. All nine copies of the slab after next are issued right
// behind the slab's barrier (row groups 6 and 7), none in the following slab: the copies a
// barrier waits for are then always older than the stores of a result tile written in between,
// and the wait can leave exactly those stores in flight (memory operations retire in order)
// instead of stalling every workgroup until its 128 KB of output have drained.
#pragma once
#include "gemm_fp8_block8.h"

namespace pt {

constexpr int B8V_MAX_CHUNKS = VK_MAX_CHUNKS;

template <int FA, int FB>
__global__ __launch_bounds__(B8_THREADS) void gemm_fp8_block8_vk_kernel(const GemmArgs a, const int chunks) {
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

    // ---- chunk c = groups [chunk_start[c], chunk_start[c + 1]): the first group of chunk c is the
    // first one that starts at or behind c / chunks of the total K length ----
    int          *chunk_start = reinterpret_cast<int *>(smem + NSTAGE * STAGE);
    const int64_t k_first = a.group_offs[0], k_total = a.group_offs[a.G] - k_first;
    if (tid <= chunks)
        chunk_start[tid] = a.G;
    __syncthreads();
    for (int g = tid; g < a.G; g += B8_THREADS) {
        const int64_t cum = a.group_offs[g] - k_first, prev = g > 0 ? a.group_offs[g - 1] - k_first : -1;
        for (int c = 0; c < chunks; ++c) {
            const int64_t thr = k_total * c / chunks;
            if (cum >= thr && prev < thr)
                chunk_start[c] = g;
        }
    }
    __syncthreads();

    const int positions = a.tiles_m * a.tiles_n;
    const int total     = positions * chunks;
    PT_GEMM_TRACE_DECL;

    // ---- loader ----
    uint32_t off[NL];
    {
        const int lrow = lane >> 3, pchk = lane & 7;
#pragma unroll
        for (int j = 0; j < LA + LB; ++j) {
            const bool isA = j < LA;
            const int  row = ((isA ? j : j - LA) * B8_WAVES + wave) * 8 + lrow;
            off[j] = static_cast<uint32_t>(row * (isA ? a.lda : a.ldb)) + ((pchk ^ swz(row)) << 4);
        }
        // scale of tile row (wavefronts 0..3) or tile column (4..7) 64 (wave % 4) + lane
        off[NL - 1] = static_cast<uint32_t>((wave & 3) * 64 + lane) * static_cast<uint32_t>(wave < 4 ? a.sa_m : a.sb_n) * 4u;
    }
    const bool     sc_is_a = wave < 4;
    const uint8_t *ld_ga, *ld_gb;     // slab the loader points at
    uint32_t       ld_na, ld_nb;      // bytes from there to the end of the tile's rows
    int            ld_s, ld_S;        // its index within the unit, slabs of the unit
    const uint8_t *ld_sc, *ld_sc_end; // this wavefront's scale source for the loader's slab
    const int64_t  slabs_all = a.group_offs[a.G] / KSTEP;
    const int64_t  sc_step   = (sc_is_a ? a.sa_k : a.sb_k) * 4;
    auto           as_bytes  = [](const float *p) { return reinterpret_cast<const uint8_t *>(p); };
    // the scale arrays end behind the last row's value of the last slab
    const uint8_t *sc_end_all = sc_is_a ? as_bytes(a.sA) + ((a.M - 1) * a.sa_m + (slabs_all - 1) * a.sa_k + 1) * 4
                                        : as_bytes(a.sB) + ((a.N - 1) * a.sb_n + (slabs_all - 1) * a.sb_k + 1) * 4;
    auto advance_loader = [&]() {
        // behind the unit's last slab the loader stays where it is (re-reads that nobody uses)
        const int adv = ld_s + 1 < ld_S ? KSTEP : 0;
        ld_s += adv / KSTEP;
        ld_ga += adv;
        ld_gb += adv;
        ld_na -= adv;
        ld_nb -= adv;
        ld_sc += adv ? sc_step : 0;
    };
    auto issue_copy = [&](auto lc, int b) {
        constexpr int L   = lc;
        uint8_t      *dst = smem + b * STAGE;
#if defined(__HIP_DEVICE_COMPILE__) // the buffer resource type only exists in the device pass
        constexpr uint32_t RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format
        if constexpr (L == NL - 1) {
            const int64_t  n     = ld_sc_end - ld_sc;
            const uint32_t bytes = n <= 0 ? 0u : (n > 0x7fffffff ? 0x7fffffffu : static_cast<uint32_t>(n));
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
    float sa_cur[TM];
    f32x4 sb_cur[TN];
    int   buf = 0;
    int   pending = 0; // memory operations of the latest result-tile store that may still be in flight

    auto ldfrag = [&](const uint8_t *part, int f) {
        const uint8_t *p  = part + f * 16 * KSTEP;
        const u32x4    lo = *reinterpret_cast<const u32x4 *>(p + frag_off_lo);
        const u32x4    hh = *reinterpret_cast<const u32x4 *>(p + frag_off_hi);
        i32x8          r;
        r[0] = lo.x; r[1] = lo.y; r[2] = lo.z; r[3] = lo.w;
        r[4] = hh.x; r[5] = hh.y; r[6] = hh.z; r[7] = hh.w;
        return r;
    };
    const uint32_t a_part = wm * (TM * 16) * KSTEP;
    const uint32_t b_part = A_BYTES + wn * (TN * 16) * KSTEP;
    const int      ES     = a.out_dtype == PT_DTYPE_F32 ? 4 : 2;

    for (int unit = blockIdx.x; unit < total; unit += gridDim.x) {
        const int chunk = unit / positions, upos = unit - chunk * positions;
        const int gs = __builtin_amdgcn_readfirstlane(chunk_start[chunk]);
        const int ge = __builtin_amdgcn_readfirstlane(chunk_start[chunk + 1]);
        if (gs >= ge)
            continue;
        int tm, tn;
        tile_coords_local(xcd_contiguous_id(upos, positions), a.tiles_m, a.tiles_n, tm, tn);
        const int64_t m0 = static_cast<int64_t>(tm) * BM, n0 = static_cast<int64_t>(tn) * BN;
        const int     rows_a = (a.M - m0) < BM ? static_cast<int>(a.M - m0) : BM;
        const int     rows_b = (a.N - n0) < BN ? static_cast<int>(a.N - n0) : BN;
        const int64_t k_lo = uniform_load(a.group_offs + gs), k_hi = uniform_load(a.group_offs + ge);

        // ---- pipeline start: slabs 0 and 1 ----
        ld_S = static_cast<int>((k_hi - k_lo) / KSTEP);
        if (ld_S > 0) {
            ld_ga     = a.A + m0 * a.lda + k_lo;
            ld_gb     = a.B + n0 * a.ldb + k_lo;
            ld_na     = rows_a * static_cast<uint32_t>(a.lda);
            ld_nb     = rows_b * static_cast<uint32_t>(a.ldb);
            ld_s      = 0;
            ld_sc     = sc_is_a ? as_bytes(a.sA) + ((k_lo / KSTEP) * a.sa_k + m0 * a.sa_m) * 4
                                : as_bytes(a.sB) + ((k_lo / KSTEP) * a.sb_k + n0 * a.sb_n) * 4;
            ld_sc_end = sc_end_all;
            static_for<0, NL>([&](auto c) { issue_nth(c, 0); });
            advance_loader();
            static_for<0, NL>([&](auto c) { issue_nth(c, 1); });
            advance_loader();
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
            __builtin_amdgcn_s_barrier();
            buf = 0;
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j] = ldfrag(smem + b_part, j);
            fa[0] = ldfrag(smem + a_part, 0);
            fa[1] = ldfrag(smem + a_part, 1);
        }

        PT_GEMM_TRACE_POINT(7);
        int64_t pos = k_lo, g_hi = uniform_load(a.group_offs + gs + 1);
        for (int g = gs; g < ge; ++g) {
            const int KT = static_cast<int>((g_hi - pos) / KSTEP);
            // the end of the group after this one, fetched while this one is multiplied
            const int64_t nxt_hi = g + 2 <= ge ? uniform_load(a.group_offs + g + 2) : g_hi;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

            // one K slab per iteration; the body stays a single basic block
            for (int kt = 0; kt < KT; ++kt) {
                const uint8_t *cur = smem + buf * STAGE;
                const uint8_t *nxt = smem + (buf ^ 1) * STAGE;
                {
                    const float *sa = reinterpret_cast<const float *>(cur + B8_SC_A) + wm * (TM * 16) + lm;
                    const float *sb = reinterpret_cast<const float *>(cur + B8_SC_B) + wn * (TN * 16) + lg * 4;
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        sa_cur[i] = sa[i * 16];
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        sb_cur[j] = *reinterpret_cast<const f32x4 *>(sb + j * 16);
                }

                constexpr int DEPTH = 3, RING = DEPTH + 1, TILES = TM * TN;
                f32x4         ring[RING];
                auto          fold = [&](int t) {
                    const int    i = t / TN, j = t % TN;
                    const f32x4 &p = ring[t % RING];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][j][e] = fmaf(p[e], sa_cur[i] * sb_cur[j][e], acc[i][j][e]);
                };

                static_for<0, TM>([&](auto ic) {
                    constexpr int i = ic;
                    if constexpr (i == 6) {
                        // ---- the slab's barrier: my copies of the next slab have landed (nothing
                        // younger is in flight) and my reads of the current stage are complete ----
                        // The copies of the next slab were issued a slab ago; the only younger memory
                        // operations a wavefront can have in flight are the stores of a result tile it
                        // has just written (`pending` of them at least): memory operations retire in
                        // order, so leaving that many outstanding waits for the copies and not for the
                        // stores. (The case distinction lives inside the asm statement so that the slab
                        // stays one basic block for the compiler.)
                        asm volatile("s_cmp_eq_u32 %0, 16\n\t"
                                     "s_cbranch_scc1 .Lvk16_%=\n\t"
                                     "s_cmp_eq_u32 %0, 32\n\t"
                                     "s_cbranch_scc1 .Lvk32_%=\n\t"
                                     "s_waitcnt vmcnt(0) lgkmcnt(0)\n\t"
                                     "s_branch .Lvkend_%=\n"
                                     ".Lvk16_%=:\n\t"
                                     "s_waitcnt vmcnt(16) lgkmcnt(0)\n\t"
                                     "s_branch .Lvkend_%=\n"
                                     ".Lvk32_%=:\n\t"
                                     "s_waitcnt vmcnt(32) lgkmcnt(0)\n"
                                     ".Lvkend_%=:"
                                     :
                                     : "s"(pending)
                                     : "memory", "scc");
                        pending = 0;
                        __builtin_amdgcn_s_barrier();
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

            PT_GEMM_TRACE_POINT(5);
            uint8_t *Cg = static_cast<uint8_t *>(a.C) + static_cast<int64_t>(g) * a.c_gstride * ES;
            const int64_t wm_base = m0 + wm * (TM * 16), wn_base = n0 + wn * (TN * 16);
            // stores of the epilogue's straight-line path (0, 16 or 32: the cases of the barrier's wait)
            pending = __builtin_amdgcn_readfirstlane(
                epilogue<TM, TN, SCALE_BLOCK, false, false>(a, acc, Cg, a.sA, a.sB, a.M, wm_base, wn_base, lane));
            static_assert(TM * TN == 32, "the barrier's wait distinguishes 16 and 32 stores in flight");
            PT_GEMM_TRACE_POINT(6);
            pos  = g_hi;
            g_hi = nxt_hi;
        }
        // the re-read copies behind the unit's last slab must have landed everywhere, and everyone
        // must be done with the stages, before the next unit's first copies go into them
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        pending = 0; // nothing is in flight any more: the next unit's first wait is for its own copies
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    PT_GEMM_TRACE_FLUSH;
}

template <int FA, int FB> static int launch_gemm_block8_vk(const GemmArgs &args_in, hipStream_t stream) {
    constexpr int LDS = B8_NSTAGE * B8_STAGE + (B8V_MAX_CHUNKS + 2) * 4 + PT_GEMM_TRACE_LDS_BYTES;
    static_assert(LDS <= 160 * 1024, "tile configuration does not fit the LDS");
    GemmArgs a = args_in;
    a.gmode    = GROUP_K;
    a.tiles_m  = static_cast<int>(cdiv(a.M, B8_BM));
    a.tiles_n  = static_cast<int>(cdiv(a.N, B8_BN));
    if (a.sa_shift != 0 || a.sb_shift != 0)
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_fp8: the variable-K 256x256 tile wants one scale per row on both sides");
    if (a.G <= 0)
        return PT_OK;
    auto kern = gemm_fp8_block8_vk_kernel<FA, FB>;
    static std::atomic<unsigned long long> attr_set{0};
    int                                    dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return fail(PT_ERR_LAUNCH, "gemm_fp8: no current device (or a device index beyond 63)");
    const unsigned long long dev_bit = 1ULL << dev;
    if (!(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
            return fail(PT_ERR_LAUNCH, "gemm_fp8: cannot raise the dynamic LDS limit");
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    const int64_t positions = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    const int64_t cus       = device_cu_count();
    const int     chunks    = vk_pick_chunks(positions, cus, a.G);
    int64_t       grid      = positions * chunks < cus ? positions * chunks : cus;
    if (grid <= 0)
        return PT_OK;
    kern<<<static_cast<unsigned>(grid), B8_THREADS, LDS, stream>>>(a, chunks);
    return check_launch("gemm_fp8_block8_vk_kernel");
}

} // namespace pt
