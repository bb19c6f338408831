// Scaled FP8 GEMM kernel template for gfx950:  C[M, N] = scale( A[M, K] . B[N, K]^T ),  fp32 accumulate.
//
// Scaling modes (semantics of Primus-Turbo's FP8 GEMMs,
// primus_turbo/triton/gemm/gemm_fp8_kernel.py:123-243,446-565,871-1013):
//   VECTOR  C = (A.B^T) * sA[m] * sB[n]            tensorwise (stride 0) and rowwise
//   BLOCK   C = sum_kb (A_kb.B_kb^T) * sA[m / bm, kb] * sB[n / bn, kb]   128-wide K blocks,
//           bm, bn = 128 (2-D weight blocks) or 1 (1-D activation blocks)
//
// Kernel structure (this library's own):
//   * one workgroup = 4 wavefronts in a 2 x 2 grid; each wavefront owns a
//     (16 TM) x (16 TN) sub-tile built from v_mfma_f32_16x16x128_f8f6f4;
//   * K advances 128 bytes per step; A and B tiles go HBM/L2 -> LDS directly
//     (global_load_lds_dwordx4, no VGPR staging) into a double buffer, so the loads of
//     step k+1 fly during the MFMAs of step k and one barrier per step suffices;
//   * LDS rows are 128 B; the 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 7),
//     which makes the 16 lanes of an MFMA operand read hit 16 different bank groups;
//   * the MFMA is issued with B as the "row" operand, so a lane ends up holding four
//     consecutive n for one m; the epilogue regroups them through LDS into whole output
//     rows and stores 16 bytes per lane;
//   * workgroup ids are remapped so that the 8 XCDs (one L2 each) work on compact
//     neighbourhoods of the tile grid.
#pragma once
#include "pt_common.h"

#include <type_traits>

// Timing probes for kernel development: a test translation unit may define this macro to
// record timestamps; in the library it expands to nothing.
#ifndef PT_GEMM_TRACE_POINT
#define PT_GEMM_TRACE_DECL
#define PT_GEMM_TRACE_POINT(id)
#endif
// Development switch (timing experiments only, results are wrong when non-zero):
// bit 0 = no tile prefetch inside the K loop, bit 1 = no MFMA, bit 2 = no fragment reads.
#ifndef PT_GEMM_EXP
#define PT_GEMM_EXP 0
#endif

namespace pt {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int   i32x8 __attribute__((ext_vector_type(8)));

enum : int { SCALE_VECTOR = 0, SCALE_BLOCK = 1 };

struct GemmArgs {
    const uint8_t *A; // [M, K] fp8, K contiguous
    const uint8_t *B; // [N, K] fp8, K contiguous
    void          *C; // [M, N] out_dtype
    const float   *sA;
    const float   *sB;
    int64_t        M, N, K;     // K is a multiple of 128 here (the host pads)
    int64_t        lda, ldb;    // row pitch of A and B in bytes (>= K)
    // VECTOR: sA[m * sa_m], sB[n * sb_n]                      (stride 0 = one scalar)
    // BLOCK : sA[(m >> sa_shift) * sa_m + kb * sa_k], sB[(n >> sb_shift) * sb_n + kb * sb_k]
    int64_t sa_m, sa_k, sb_n, sb_k;
    int     sa_shift, sb_shift; // 0 (one scale per row) or 7 (one per 128 rows)
    int     out_dtype;
    int     accumulate; // C += result (beta = 1) instead of C = result
    int     tiles_m, tiles_n;
};

constexpr int KSTEP      = 128; // bytes of K per pipeline step (= one MFMA K)
constexpr int GEMM_WAVES = 4;

__device__ __forceinline__ int swz(int row) {
    return (row >> 1) & 7;
}

typedef __attribute__((address_space(3))) void       *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *glb_ptr_t;

// Copy `ROWS` rows x 128 bytes from global (row stride ld bytes) into LDS, swizzled.
// Each wave instruction moves 8 rows (1 KB); rows at or beyond `rows_valid` re-read the
// last valid row (their products are never stored).
template <int ROWS>
__device__ __forceinline__ void tile_to_lds(const uint8_t *__restrict__ g, int64_t ld,
                                            int rows_valid, uint8_t *lds, int wave, int lane) {
    constexpr int INSTR = ROWS / 8 / GEMM_WAVES;
    const int     lrow  = lane >> 3; // row within the 8-row group
    const int     pchk  = lane & 7;  // physical chunk this lane fills
#pragma unroll
    for (int j = 0; j < INSTR; ++j) {
        const int r8  = j * GEMM_WAVES + wave;
        int       row = r8 * 8 + lrow;
        const int lch = pchk ^ swz(row);
        int       src = row < rows_valid ? row : rows_valid - 1;
        const uint8_t *p = g + static_cast<int64_t>(src) * ld + lch * 16;
        __builtin_amdgcn_global_load_lds((glb_ptr_t)p, (lds_ptr_t)(lds + r8 * 1024), 16, 0, 0);
    }
}

// MFMA operand fragment of 16 tile rows: lane (r = lane % 16, g = lane / 16) takes K bytes
// [16g, 16g+16) and [64+16g, 64+16g+16) of row r, i.e. two 16-byte LDS reads. The swizzle
// term of a row depends only on r (16 rows = 2 swizzle periods), so every fragment of a
// wavefront's sub-tile uses the same two lane addresses plus an immediate offset.
//
// The reads are inline assembly on purpose: the compiler's wait-count pass has to assume
// that an outstanding direct-to-LDS load may alias any LDS read it can see and would drain
// the prefetch (vmcnt(0)) before every one of them. Completion is awaited explicitly with
// frag_wait<N>() -- LDS returns data in order, so "at most N operations outstanding" means
// everything but the N youngest reads has landed -- and a fragment must pass through
// frag_ready() before its first use so that no consumer can be scheduled above the wait.
struct Frag {
    u32x4 lo, hi;
};

__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)p));
}

template <int OFF> __device__ __forceinline__ void frag_issue(Frag &f, uint32_t addr_lo, uint32_t addr_hi) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.lo) : "v"(addr_lo), "n"(OFF));
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.hi) : "v"(addr_hi), "n"(OFF));
}

template <int N> __device__ __forceinline__ void frag_wait() {
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ i32x8 frag_ready(Frag &f) {
    asm volatile("" : "+v"(f.lo), "+v"(f.hi));
    i32x8 r;
    r[0] = f.lo.x; r[1] = f.lo.y; r[2] = f.lo.z; r[3] = f.lo.w;
    r[4] = f.hi.x; r[5] = f.hi.y; r[6] = f.hi.z; r[7] = f.hi.w;
    return r;
}

template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int FA, int FB>
__device__ __forceinline__ f32x4 mfma_fp8(const i32x8 &rowop, const i32x8 &colop, f32x4 c) {
    // rowop carries B-matrix rows (format FB), colop carries A-matrix rows (format FA)
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(rowop, colop, c, FB, FA, 0, 0x7f7f7f7f,
                                                            0, 0x7f7f7f7f);
}

template <typename T> __device__ __forceinline__ void store4(T *p, f32x4 v, bool vec4, int nvalid, bool accumulate) {
    if (accumulate) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nvalid)
                v[e] += HP<T>::to_f32(p[e]);
    }
    if (vec4) {
        if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<f32x4 *>(p) = v;
        } else {
            u32x2 o;
            o.x = pack2<T>(v[0], v[1]);
            o.y = pack2<T>(v[2], v[3]);
            *reinterpret_cast<u32x2 *>(p) = o;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (e < nvalid)
                p[e] = HP<T>::from_f32(v[e]);
    }
}

// Tile coordinates of a workgroup: XCD-contiguous ids, then groups of GROUP_M tile rows
// walked column-major so that concurrently running tiles share A and B panels in L2.
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
    constexpr int NXCD    = 8;
    constexpr int GROUP_M = 8;
    const int     total   = tiles_m * tiles_n;
    int           lid     = pid;
    if (total >= NXCD * 4) {
        // workgroup i runs on XCD i % 8: give each XCD one contiguous id range
        const int per  = total / NXCD, rem = total % NXCD;
        const int xcd  = pid % NXCD, slot = pid / NXCD;
        // XCDs [0, rem) own per + 1 ids
        lid = xcd * per + (xcd < rem ? xcd : rem) + slot;
    }
    const int in_group = GROUP_M * tiles_n;
    const int gid      = lid / in_group;
    const int first_m  = gid * GROUP_M;
    const int gsz      = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int r        = lid % in_group;
    tm                 = first_m + r % gsz;
    tn                 = r / gsz;
}

// Epilogue. A lane holds, for tile (i, j), C[wm_base + 16 i + lm][wn_base + 16 j + 4 lg + e],
// e = 0..3: written directly that is 32-byte pieces scattered over 16 rows per instruction.
// Instead every wavefront passes its sub-tile, 16 rows x 64 (or 32) columns (fp32) at a time,
// through a private LDS strip and writes it back out row-wise: a lane scales, converts
// and stores 16 bytes of one row, so HBM sees full 128-byte lines.
// Strip width: 64 columns where one workgroup per CU leaves room for it, 32 columns for the
// 128 x 128 tile so that two workgroups still fit into the 160 KB of LDS.
template <int TM, int TN> struct EpiGeom {
    static constexpr int COLS  = (TM * TN >= 32) ? 64 : 32;
    static constexpr int ROWB  = COLS * 4 + 16; // padded LDS row pitch in bytes
    static constexpr int BYTES = 16 * ROWB;     // per wavefront
};

template <typename T, int TM, int TN, int MODE>
__device__ __forceinline__ void epilogue(const GemmArgs &a, const f32x4 (&acc)[TM][TN],
                                         int64_t wm_base, int64_t wn_base, int lane,
                                         uint8_t *strip) {
    constexpr int EPI_COLS = EpiGeom<TM, TN>::COLS, EPI_ROWB = EpiGeom<TM, TN>::ROWB;
    constexpr int ES  = sizeof(T);
    constexpr int EPC = 16 / ES;        // output elements per 16-byte chunk
    constexpr int CPR = EPI_COLS / EPC; // chunks per strip row
    constexpr int RPI = 64 / CPR;       // rows written per store instruction
    constexpr int JH  = EPI_COLS / 16;  // MFMA tiles per strip width
    static_assert(TN % JH == 0, "sub-tile width must be a multiple of the strip width");
    const int  lm = lane & 15, lg = lane >> 4;
    T         *C    = static_cast<T *>(a.C);
    const bool accu = a.accumulate != 0;
    // 16-byte global accesses need every row start on a 16-byte boundary
    const bool vec  = (a.N * ES) % 16 == 0;
    const int  crow = lane / CPR, cchk = lane % CPR; // this lane's (row, chunk) in the write-out
    // VECTOR mode: fetch every scale this lane will need before the first store is issued
    // (a load issued behind stores cannot complete before they are acknowledged)
    constexpr int NR = 16 / RPI, NH = TN / JH;
    [[maybe_unused]] float sa_e[TM][NR], sb_e[NH][EPC];
    if constexpr (MODE == SCALE_VECTOR) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int q = 0; q < NR; ++q) {
                const int64_t m = wm_base + i * 16 + q * RPI + crow;
                sa_e[i][q]      = a.sA[(m < a.M ? m : a.M - 1) * a.sa_m];
            }
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int e = 0; e < EPC; ++e) {
                const int64_t ne = wn_base + h * EPI_COLS + cchk * EPC + e;
                sb_e[h][e]       = a.sB[(ne < a.N ? ne : a.N - 1) * a.sb_n];
            }
    }
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        const int64_t n = wn_base + h * EPI_COLS + cchk * EPC;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            // 1. accumulators -> LDS strip [16][64] fp32
#pragma unroll
            for (int jj = 0; jj < JH; ++jj)
                *reinterpret_cast<f32x4 *>(strip + lm * EPI_ROWB + (jj * 16 + lg * 4) * 4) = acc[i][h * JH + jj];
            // 2. LDS strip -> global, row-wise (the same wavefront wrote and reads; LDS keeps
            //    its accesses in program order)
#pragma unroll
            for (int r0 = 0; r0 < 16; r0 += RPI) {
                const int     r = r0 + crow;
                const int64_t m = wm_base + i * 16 + r;
                float         f[EPC];
#pragma unroll
                for (int q = 0; q < EPC / 4; ++q) {
                    const f32x4 t = *reinterpret_cast<const f32x4 *>(strip + r * EPI_ROWB + (cchk * EPC + q * 4) * 4);
                    f[4 * q] = t[0]; f[4 * q + 1] = t[1]; f[4 * q + 2] = t[2]; f[4 * q + 3] = t[3];
                }
                if (m < a.M && n < a.N) {
                    if constexpr (MODE == SCALE_VECTOR) {
                        const float sa = sa_e[i][r0 / RPI];
#pragma unroll
                        for (int e = 0; e < EPC; ++e)
                            f[e] = f[e] * sa * sb_e[h][e];
                    }
                    T *gp = C + m * a.N + n;
                    if (vec && n + EPC <= a.N) {
                        if (accu) {
                            const u32x4 old = ld128(gp);
                            if constexpr (ES == 4) {
                                f[0] += __uint_as_float(old.x); f[1] += __uint_as_float(old.y);
                                f[2] += __uint_as_float(old.z); f[3] += __uint_as_float(old.w);
                            } else {
                                const uint32_t ow[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
                                for (int q = 0; q < 4; ++q) {
                                    float o0, o1;
                                    unpack2<T>(ow[q], o0, o1);
                                    f[2 * q] += o0;
                                    f[2 * q + 1] += o1;
                                }
                            }
                        }
                        u32x4 w;
                        if constexpr (ES == 4) {
                            w = u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
                        } else {
                            w = u32x4{pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])};
                        }
                        st128(gp, w);
                    } else {
#pragma unroll
                        for (int e = 0; e < EPC; ++e)
                            if (n + e < a.N) {
                                float v = f[e];
                                if (accu)
                                    v += HP<T>::to_f32(gp[e]);
                                gp[e] = HP<T>::from_f32(v);
                            }
                    }
                }
            }
        }
    }
}

// Where a workgroup's current tile lives.
struct TileCtx {
    const uint8_t *Ag, *Bg; // first row of the tile in A / B
    int            rows_a, rows_b;
    int64_t        m0, n0;
};

template <int BM, int BN>
__device__ __forceinline__ TileCtx make_tile(const GemmArgs &a, int tile) {
    int tm, tn;
    tile_coords(tile, a.tiles_m, a.tiles_n, tm, tn);
    TileCtx t;
    t.m0     = static_cast<int64_t>(tm) * BM;
    t.n0     = static_cast<int64_t>(tn) * BN;
    t.rows_a = (a.M - t.m0) < BM ? static_cast<int>(a.M - t.m0) : BM;
    t.rows_b = (a.N - t.n0) < BN ? static_cast<int>(a.N - t.n0) : BN;
    t.Ag     = a.A + t.m0 * a.lda;
    t.Bg     = a.B + t.n0 * a.ldb;
    return t;
}

// Persistent kernel: the grid is sized to the machine and every workgroup walks tiles
// blockIdx.x, blockIdx.x + gridDim.x, ... . The K pipeline runs across tile boundaries: the
// first K slab of the next tile is already being loaded while the current tile's last
// slab is multiplied and its result written out, so the matrix cores only pause for the
// epilogue's own instructions.
template <int TM, int TN, int MODE, bool SB_VEC, int FA, int FB>
__global__ __launch_bounds__(256) void gemm_fp8_nt_kernel(const GemmArgs a) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    constexpr int A_BYTES = BM * KSTEP, B_BYTES = BN * KSTEP, STAGE = A_BYTES + B_BYTES;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    uint8_t *strips = smem + 2 * STAGE; // epilogue staging, outside the pipeline buffers

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1; // wavefront position in the 2 x 2 grid
    const int lm = lane & 15, lg = lane >> 4;

    // byte offsets of this lane's two 16-byte fragment reads within a 16-row group
    const uint32_t frag_off_lo = lm * KSTEP + ((lg ^ swz(lm)) << 4);
    const uint32_t frag_off_hi = lm * KSTEP + (((4 + lg) ^ swz(lm)) << 4);

    const int total = a.tiles_m * a.tiles_n;
    const int KT    = static_cast<int>(a.K / KSTEP);
    int       tile  = blockIdx.x;
    if (tile >= total)
        return;
    TileCtx cur_t = make_tile<BM, BN>(a, tile);

    f32x4 acc[TM][TN];

    // BLOCK mode: the fp32 scales of the next K block are fetched one step ahead (before
    // the tile prefetch is issued, so that the tile loads stay the youngest entries of the
    // vector-memory counter) and are in registers when their step starts.
    [[maybe_unused]] float sa_cur[TM], sa_nxt[TM];
    [[maybe_unused]] float sb_cur[TN][SB_VEC ? 4 : 1], sb_nxt[TN][SB_VEC ? 4 : 1];
    auto fetch_scales = [&](const TileCtx &t, int kt, float (&sa)[TM], float (&sb)[TN][SB_VEC ? 4 : 1]) {
        if constexpr (MODE == SCALE_BLOCK) {
            const int64_t wm_base = t.m0 + wm * (TM * 16), wn_base = t.n0 + wn * (TN * 16);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                int64_t m = wm_base + i * 16 + lm;
                m         = m < a.M ? m : a.M - 1;
                sa[i]     = a.sA[(m >> a.sa_shift) * a.sa_m + kt * a.sa_k];
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (SB_VEC) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        int64_t n = wn_base + j * 16 + lg * 4 + e;
                        n         = n < a.N ? n : a.N - 1;
                        sb[j][e]  = a.sB[n * a.sb_n + kt * a.sb_k];
                    }
                } else {
                    int64_t       nb    = (wn_base + j * 16) >> a.sb_shift;
                    const int64_t nbmax = (a.N - 1) >> a.sb_shift;
                    nb                  = nb < nbmax ? nb : nbmax;
                    sb[j][0]            = a.sB[nb * a.sb_n + kt * a.sb_k];
                }
            }
        }
    };
    auto load_stage = [&](const TileCtx &t, int kt, uint8_t *buf) {
        tile_to_lds<BM>(t.Ag + static_cast<int64_t>(kt) * KSTEP, a.lda, t.rows_a, buf, wave, lane);
        tile_to_lds<BN>(t.Bg + static_cast<int64_t>(kt) * KSTEP, a.ldb, t.rows_b, buf + A_BYTES, wave, lane);
    };

    int buf = 0;
    PT_GEMM_TRACE_DECL;
    PT_GEMM_TRACE_POINT(0);
    if (KT > 0) {
        fetch_scales(cur_t, 0, sa_nxt, sb_nxt);
        load_stage(cur_t, 0, smem);
    }

    while (true) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int next_tile = tile + gridDim.x;
        TileCtx   nxt_t     = cur_t;
        if (next_tile < total)
            nxt_t = make_tile<BM, BN>(a, next_tile);

        for (int kt = 0; kt < KT; ++kt) {
            uint8_t *cur = smem + buf * STAGE;
            PT_GEMM_TRACE_POINT(1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            PT_GEMM_TRACE_POINT(2);
            __builtin_amdgcn_s_barrier();
            PT_GEMM_TRACE_POINT(3);
            if constexpr (MODE == SCALE_BLOCK) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    sa_cur[i] = sa_nxt[i];
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < (SB_VEC ? 4 : 1); ++e)
                        sb_cur[j][e] = sb_nxt[j][e];
            }
            // prefetch the next step of the pipeline: same tile, or the next tile's first slab
            if ((PT_GEMM_EXP & 1) && kt > 0) {
            } else if (kt + 1 < KT) {
                fetch_scales(cur_t, kt + 1, sa_nxt, sb_nxt);
                load_stage(cur_t, kt + 1, smem + (buf ^ 1) * STAGE);
            } else if (next_tile < total) {
                fetch_scales(nxt_t, 0, sa_nxt, sb_nxt);
                load_stage(nxt_t, 0, smem + (buf ^ 1) * STAGE);
            }
            // lane addresses of the A / B fragments of this wavefront in the current stage
            const uint32_t la = lds_addr(cur) + wm * (TM * 16) * KSTEP + frag_off_lo;
            const uint32_t lb = lds_addr(cur) + A_BYTES + wn * (TN * 16) * KSTEP + frag_off_lo;
            const uint32_t hi = frag_off_hi - frag_off_lo; // same for A and B

            Frag fa[TM], fb[2];
            if ((PT_GEMM_EXP & 4) && kt > 0) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    fa[i].lo = fa[i].hi = u32x4{la, lb, hi, (uint32_t)kt};
                fb[0].lo = fb[0].hi = fb[1].lo = fb[1].hi = u32x4{la, lb, hi, (uint32_t)kt};
            } else {
            static_for<0, TM>([&](auto i) { frag_issue<i * 16 * KSTEP>(fa[i], la, la + hi); });
            frag_issue<0>(fb[0], lb, lb + hi);
            if constexpr (TN > 1)
                frag_issue<16 * KSTEP>(fb[1], lb, lb + hi);
            }
            i32x8 af[TM];

            [[maybe_unused]] constexpr int DEPTH = 2, RING = DEPTH + 1, TILES = TM * TN;
            [[maybe_unused]] f32x4 ring[RING];
            [[maybe_unused]] auto  fold = [&](int t) {
                // BLOCK mode: fold the finished product of one 128-wide K block into the
                // running sum with its block scale (VALU work in the shadow of later MFMAs)
                const int    i = t % TM, j = t / TM;
                const f32x4 &p = ring[t % RING];
                if constexpr (SB_VEC) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][j][e] = fmaf(p[e], sa_cur[i] * sb_cur[j][SB_VEC ? e : 0], acc[i][j][e]);
                } else {
                    const float sc = sa_cur[i] * sb_cur[j][0];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][j][e] = fmaf(p[e], sc, acc[i][j][e]);
                }
            };

            static_for<0, TN>([&](auto jc) {
                constexpr int j = jc;
                // B fragment j (and, for j == 0, every A fragment) must have landed; the two
                // reads of fragment j + 1 may still be in flight
                if constexpr (j + 1 < TN)
                    frag_wait<2>();
                else
                    frag_wait<0>();
                if constexpr (j == 0) {
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        af[i] = frag_ready(fa[i]);
                }
                const i32x8 bf = frag_ready(fb[j & 1]);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    if constexpr (MODE == SCALE_BLOCK) {
                        const int t    = j * TM + i;
                        ring[t % RING] = mfma_fp8<FA, FB>(bf, af[i], f32x4{0.f, 0.f, 0.f, 0.f});
                        if (t >= DEPTH)
                            fold(t - DEPTH);
                    } else if (PT_GEMM_EXP & 2) {
                        acc[i][j][0] += __builtin_bit_cast(float, bf[i & 7] ^ af[i][j & 7]);
                    } else {
                        acc[i][j] = mfma_fp8<FA, FB>(bf, af[i], acc[i][j]);
                    }
                }
                if constexpr (j + 2 < TN) {
                    if (!((PT_GEMM_EXP & 4) && kt > 0))
                        frag_issue<(j + 2) * 16 * KSTEP>(fb[j & 1], lb, lb + hi);
                }
            });
            if constexpr (MODE == SCALE_BLOCK) {
#pragma unroll
                for (int t = TILES - DEPTH; t < TILES; ++t)
                    fold(t);
            }
            buf ^= 1;
            PT_GEMM_TRACE_POINT(4);
        }

        PT_GEMM_TRACE_POINT(5);
        // epilogue through this wavefront's private strip (no workgroup barrier needed)
        const int64_t wm_base = cur_t.m0 + wm * (TM * 16), wn_base = cur_t.n0 + wn * (TN * 16);
        uint8_t      *strip   = strips + wave * EpiGeom<TM, TN>::BYTES;
        if (a.out_dtype == PT_DTYPE_BF16)
            epilogue<bf16_t, TM, TN, MODE>(a, acc, wm_base, wn_base, lane, strip);
        else if (a.out_dtype == PT_DTYPE_F16)
            epilogue<f16_t, TM, TN, MODE>(a, acc, wm_base, wn_base, lane, strip);
        else
            epilogue<float, TM, TN, MODE>(a, acc, wm_base, wn_base, lane, strip);

        PT_GEMM_TRACE_POINT(6);
        if (next_tile >= total)
            break;
        tile  = next_tile;
        cur_t = nxt_t;
    }
}

template <int TM, int TN, int MODE, bool SB_VEC, int FA, int FB>
static int launch_gemm_cfg(const GemmArgs &args_in, hipStream_t stream) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    constexpr int LDS = 2 * (BM + BN) * KSTEP + GEMM_WAVES * EpiGeom<TM, TN>::BYTES;
    GemmArgs      a   = args_in;
    a.tiles_m         = static_cast<int>(cdiv(a.M, BM));
    a.tiles_n         = static_cast<int>(cdiv(a.N, BN));
    auto kern         = gemm_fp8_nt_kernel<TM, TN, MODE, SB_VEC, FA, FB>;
    static bool attr_set = false;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
            return fail(PT_ERR_LAUNCH, "gemm_fp8: cannot raise the dynamic LDS limit");
        attr_set = true;
    }
    // persistent grid: as many workgroups as fit on the machine at once (LDS-limited)
    const int     per_cu = (160 * 1024) / LDS;
    const int64_t total  = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    int64_t       grid   = static_cast<int64_t>(device_cu_count()) * (per_cu < 1 ? 1 : per_cu);
    if (grid > total)
        grid = total;
    kern<<<static_cast<unsigned>(grid), 256, LDS, stream>>>(a);
    return check_launch("gemm_fp8_nt_kernel");
}

} // namespace pt
