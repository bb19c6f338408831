// Scaled FP8 GEMM kernel template for gfx950:  C[M, N] = scale( A[M, K] . B[N, K]^T ),  fp32 accumulate.
//
// Scaling modes (semantics of Primus-Turbo's FP8 GEMMs,
// primus_turbo/triton/gemm/gemm_fp8_kernel.py:123-243,446-565,871-1013):
//   VECTOR  C = (A.B^T) * sA[m] * sB[n]            tensorwise (stride 0) and rowwise
//   BLOCK   C = sum_kb (A_kb.B_kb^T) * sA[m / bm, kb] * sB[n / bn, kb]   128-wide K blocks,
//           bm, bn = 128 (2-D weight blocks) or 1 (1-D activation blocks)
//   MX      C = sum_kb (A_kb.B_kb^T) * 2^(sA[m, kb] - 127) * 2^(sB[n, kb] - 127), 32-wide K
//           blocks with E8M0 scale bytes applied by the matrix core itself (MXFP8, and MXFP4
//           with two E2M1 codes per byte: gemm_fp8_impl.py:341-496, gemm_fp4_impl.py:53-319)
//
// Kernel structure (this library's own):
//   * one workgroup = 4 wavefronts in a 2 x 2 grid; each wavefront owns a
//     (16 TM) x (16 TN) sub-tile built from v_mfma_scale_f32_16x16x128_f8f6f4;
//   * K advances 128 bytes per step ("slab"); A and B tiles go HBM/L2 -> LDS directly
//     (buffer_load_dwordx4 ... lds, no VGPR staging) into two or three LDS stages; the MFMA
//     operand fragments of a slab all live in registers and are refilled from the next slab's
//     stage one by one as they die, so the copies of the slab after that can be spread over the
//     whole slab; two barriers per slab (see the kernel);
//   * LDS rows are 128 B; the 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 7),
//     which makes the 16 lanes of an MFMA operand read hit 16 different bank groups;
//   * BLOCK and MX scales travel through the LDS stages with the slab they belong to;
//   * the MFMA is issued with B as the "row" operand, so a lane ends up holding four
//     consecutive n for one m; 16-bit outputs exchange 16-lane rows between neighbouring tiles
//     so that a lane stores eight consecutive n;
//   * workgroup ids are remapped so that the 8 XCDs (one L2 each) work on compact
//     neighbourhoods of the tile grid.
#pragma once
#include "pt_common.h"

#include <atomic>
#include <type_traits>

// Timing probes for kernel development: a test translation unit may define this macro to
// record timestamps; in the library it expands to nothing.
#ifndef PT_GEMM_TRACE_POINT
#define PT_GEMM_TRACE_DECL
#define PT_GEMM_TRACE_POINT(id)
#define PT_GEMM_TRACE_FLUSH
#define PT_GEMM_TRACE_LDS_BYTES 0
#endif
namespace pt {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int   i32x8 __attribute__((ext_vector_type(8)));

enum : int { SCALE_VECTOR = 0, SCALE_BLOCK = 1, SCALE_MX = 2 };

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
    // MX    : sA / sB point at E8M0 bytes, byte[m * sa_m + kb] and byte[n * sb_n + kb];
    //         or, "word-major" (sa_wpitch, sb_wpitch != 0): the 32-bit word w of row m (its K blocks
    //         4 w .. 4 w + 3) at byte m * 4 + w * sa_wpitch, i.e. the words of one K position of all
    //         rows are contiguous and a scale copy fetches two cache lines instead of sixty-four
    int64_t sa_m, sa_k, sb_n, sb_k;
    int64_t sa_wpitch, sb_wpitch;
    // GROUP_K: the groups are cut into this many runs of about equal K length; a unit of work is one
    // output position times one run (set by the launcher)
    int vk_chunks;
    int     sa_shift, sb_shift; // 0 (one scale per row) or 7 (one per 128 rows)
    int     kb_valid;           // BLOCK / MX: K blocks the scale arrays hold (slabs beyond are zero padding)
    int     out_dtype;
    int     accumulate; // C += result (beta = 1) instead of C = result
    int     tiles_m, tiles_n;
    // Grouped problems (MoE experts); group_offs is a device array of G + 1 int64 prefix sums.
    //   GROUP_ROWS: rows [offs[g], offs[g+1]) of A and C belong to group g, which multiplies
    //               with B + g * b_gstride (scales sB + g * sb_gstride); M is the row count of A.
    //   GROUP_K   : group g reduces over K elements [offs[g], offs[g+1]) of A and B (whole
    //               128-byte slabs: multiples of 128, MXFP4 256) into C + g * c_gstride; scales
    //               start at the slab offs[g] / 128 (MXFP4: / 256).
    int            gmode;
    int            G;
    const int64_t *group_offs;
    // GROUP_ROWS only, optional: row offsets of the groups in C when they differ from those in A
    // (A in a per-group padded layout, C packed tight); NULL = the same offsets
    const int64_t *group_offs_out;
    int64_t        b_gstride;  // bytes
    int64_t        sb_gstride; // floats
    int64_t        c_gstride;  // elements
};

enum : int { GROUP_NONE = 0, GROUP_ROWS = 1, GROUP_K = 2 };

constexpr int KSTEP      = 128; // bytes of K per pipeline step (= one MFMA K)
constexpr int GEMM_WAVES = 4;
// pipeline depth of a tile configuration (see the kernel); K must span at least depth + 1 slabs
constexpr int gemm_stages(int TM, int TN, bool F4 = false) {
    return (TM == 8 && TN == 4 && !F4) ? 3 : 2;
}
constexpr int GEMM_MIN_SLABS = 4;
// BLOCK and MX modes: the scales of a slab travel with it through the LDS stages; every
// wavefront keeps a private copy of the scale words (one per slab, two for MXFP4) of its
// 16 * TM rows and 16 * TN columns.
constexpr int gemm_scale_bytes(int TM, int TN, int MODE, bool F4) {
    return MODE == 0 ? 0 : GEMM_WAVES * (TM * 16 + TN * 16) * 4 * (F4 ? 2 : 1);
}
constexpr int gemm_stage_bytes(int TM, int TN, int MODE, bool F4) {
    return (2 * TM * 16 + 2 * TN * 16) * KSTEP + gemm_scale_bytes(TM, TN, MODE, F4);
}

__device__ __forceinline__ int swz(int row) {
    return (row >> 1) & 7;
}

typedef __attribute__((address_space(3))) void       *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *glb_ptr_t;

// Direct-to-LDS copies: each wave instruction moves 8 tile rows x 128 B = 1 KB to
// contiguous LDS; lane l fills physical chunk l % 8 of row l / 8, reading the logical chunk
// that the swizzle maps there. Rows at or beyond the end of the tile's share of the matrix
// read as zero (buffer descriptor bounds); their products are never stored.
//
// MFMA operand fragment of 16 tile rows: lane (r = lane % 16, g = lane / 16) takes K bytes
// [16g, 16g+16) and [64+16g, 64+16g+16) of row r, i.e. two 16-byte LDS reads. The swizzle
// term of a row depends only on r (16 rows = 2 swizzle periods), so every fragment of a
// wavefront's sub-tile uses the same two lane addresses plus an immediate offset. The reads
// are ordinary loads: with buffer-load copies the compiler's wait-count pass does not treat an
// outstanding direct-to-LDS copy as aliasing them.

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

// E8M0 block scales of the instruction: lane (r, g) supplies, in the low byte of its scale
// operand, the scale of matrix row r and 32-wide K block g of the 128 K values consumed.

// The instruction written out by hand, accumulating in place in an AGPR tuple. The compiler's
// own selection turns the tied accumulate form into "copy the accumulator tile, then write the
// original registers" (four v_accvgpr_mov and a dozen wait states in front of every MFMA)
// whenever it has registers to spare, which halves the matrix-core rate. Used by the modes
// that accumulate inside the matrix core (VECTOR, MX). The compiler does not know this is an
// MFMA, so the hazards are the caller's: the accumulators are only read (v_accvgpr_read in the
// epilogue) after a padding of wait states, and two MFMAs on one accumulator are never issued
// back to back.
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int FA, int FB>
__device__ __forceinline__ void mfma_inplace(f32x4 &c, const i32x8 &rowop, const i32x8 &colop, uint32_t row_scale,
                                             uint32_t col_scale) {
#if defined(__HIP_DEVICE_COMPILE__) // the host pass cannot parse the AGPR constraint
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:%5 blgp:%6"
                 : "+a"(c)
                 : "v"(rowop), "v"(colop), "v"(row_scale), "v"(col_scale), "n"(FB), "n"(FA));
#endif
}
// FP4 operands are 128 bits per lane
__device__ __forceinline__ void mfma_inplace_f4(f32x4 &c, const i32x4 &rowop, const i32x4 &colop, uint32_t row_scale,
                                                uint32_t col_scale) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                 : "+a"(c)
                 : "v"(rowop), "v"(colop), "v"(row_scale), "v"(col_scale));
#endif
}

// Tile coordinates of a workgroup: XCD-contiguous ids, then groups of GROUP_M tile rows
// walked column-major so that concurrently running tiles share A and B panels in L2.
__device__ __forceinline__ void tile_coords_local(int lid, int tiles_m, int tiles_n, int &tm, int &tn);
__device__ __forceinline__ int xcd_contiguous_id(int pid, int total) {
    constexpr int NXCD = 8;
    if (total < NXCD * 4)
        return pid;
    // workgroup i runs on XCD i % 8: give each XCD one contiguous id range
    const int per = total / NXCD, rem = total % NXCD;
    const int xcd = pid % NXCD, slot = pid / NXCD;
    // XCDs [0, rem) own per + 1 ids
    return xcd * per + (xcd < rem ? xcd : rem) + slot;
}
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
    tile_coords_local(xcd_contiguous_id(pid, tiles_m * tiles_n), tiles_m, tiles_n, tm, tn);
}
__device__ __forceinline__ void tile_coords_local(int lid, int tiles_m, int tiles_n, int &tm, int &tn) {
    constexpr int GROUP_M  = 8;
    const int     in_group = GROUP_M * tiles_n;
    const int gid      = lid / in_group;
    const int first_m  = gid * GROUP_M;
    const int gsz      = (tiles_m - first_m) < GROUP_M ? (tiles_m - first_m) : GROUP_M;
    const int r        = lid % in_group;
    tm                 = first_m + r % gsz;
    tn                 = r / gsz;
}

// Tile coordinates inside one group of a row-grouped problem (gtm tile rows x tiles_n tile
// columns, local = 0 .. gtm * tiles_n - 1). Workgroup ids, hence consecutive tiles, go to the
// eight XCDs round-robin, and the tiles that run at the same time are a window of consecutive
// ids: what matters for the traffic between the L2s and the fabric is which tiles share an XCD,
// i.e. the tiles whose ids are congruent modulo 8. The group's tile rows are cut into panels of
// 8, 4, 2 and 1 rows (binary decomposition of gtm), walked one after the other; inside a panel
// of R x C tiles the eight residue classes each own a compact block of the panel (R = 8: 4 rows
// x C / 4 columns; R = 4: 2 rows x C / 4 columns; R = 2: 2 rows x C / 8 columns), walked row-fastest, so that the tiles an
// XCD works on at a time share A panels AND B panels in its L2. (With the plain row-fastest
// numbering an XCD owns one tile row of the panel and every tile of it fetches a B panel of its
// own: the forward launch of 32 Zipf-sized groups moved 4.2 times its operand bytes.)
__device__ __forceinline__ void group_tile_coords(int local, int gtm, int tiles_n, int &tm, int &tn) {
    const int C  = tiles_n;
    const int n8 = gtm >> 3;
    int       first_m, R, r;
    if (local < n8 * 8 * C) {
        first_m = (local / (8 * C)) * 8;
        r       = local % (8 * C);
        R       = 8;
    } else {
        r       = local - n8 * 8 * C;
        first_m = n8 * 8;
        R       = 1;
        const int left = gtm - first_m; // 0 .. 7
        if (left & 4) {
            if (r < 4 * C) {
                R = 4;
            } else {
                r -= 4 * C;
                first_m += 4;
            }
        }
        if (R == 1 && (left & 2)) {
            if (r < 2 * C) {
                R = 2;
            } else {
                r -= 2 * C;
                first_m += 2;
            }
        }
    }
    const int k = r & 7, sl = r >> 3;
    if (R == 8 && (C & 3) == 0) {
        const int cw = C >> 2;
        tm           = first_m + (k & 1) * 4 + (sl & 3);
        tn           = (k >> 1) * cw + (sl >> 2);
    } else if (R == 4 && (C & 3) == 0) {
        const int cw = C >> 2;
        tm           = first_m + (k & 1) * 2 + (sl & 1);
        tn           = (k >> 1) * cw + (sl >> 1);
    } else if (R == 2 && (C & 7) == 0) {
        const int cw = C >> 3;
        tm           = first_m + (sl & 1);
        tn           = k * cw + (sl >> 1);
    } else {
        tm = first_m + r % R;
        tn = r / R;
    }
}

// Epilogue. A lane holds, for MFMA tile (i, j), C[wm_base + 16 i + lm][wn_base + 16 j + 4 lg + e],
// e = 0..3. It scales, converts and stores those four values itself (8 bytes of bf16/fp16,
// 16 bytes of fp32): per instruction the wavefront writes 16 rows x 32 (64) contiguous bytes,
// the neighbouring j tiles complete the 128-byte lines in the write-back L2, and the
// accumulators need no exchange between lanes, which keeps the instruction count per
// output near its minimum (two multiplies and half a convert).
//
// One straight-line loop nest per output type serves sub-tiles that lie wholly inside the
// matrix with aligned rows; a generic nest (per-element bounds checks, run-time type)
// serves the rest. The accumulators are read with hand-written v_accvgpr_read where they
// are needed: left to itself the compiler copies all of them out of the AGPRs ahead of the
// case distinction and spills everything else.
template <bool ACC_IN_AGPR> __device__ __forceinline__ f32x4 read_acc(const f32x4 &c) {
    f32x4 v;
    if constexpr (ACC_IN_AGPR) {
#if defined(__HIP_DEVICE_COMPILE__) // the host pass cannot parse the AGPR constraint
#pragma unroll
        for (int e = 0; e < 4; ++e)
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(c[e]));
#endif
    } else {
        v = c;
    }
    return v;
}

// 16-bit outputs are written by pairs of MFMA tiles (i, j), (i, j + 1): the odd 16-lane rows of
// tile j are swapped with the even rows of tile j + 1 (v_permlane16_swap), after which a lane
// holds eight consecutive n of one m -- one 16-byte store, and 64 contiguous bytes per matrix
// row and store instruction, so that no partially written 64-byte unit ever leaves the L2.
// `row` points at C[m][wn_base + 16 (lg & 1) + 8 (lg >> 1)] for 16-bit outputs and at
// C[m][wn_base + 4 lg] for fp32.
// Returns the number of store instructions it has issued (every one of them younger than any
// memory operation issued before the call): what a caller may leave in flight when it next waits
// for older operations by count.
// `rows_left`: rows of the matrix from this lane's first row on (its row of MFMA tile i is
// 16 i): a lane skips the loads and stores of the row groups at or beyond it, so a sub-tile that
// hangs over the end of its matrix (the last rows of a group) still leaves in 16-byte stores.
// (ROWCHECK = false: every row group is stored; for callers whose sub-tile is known to lie inside.)
template <typename T, int TM, int TN, int MODE, bool ACC_IN_AGPR, bool ROWCHECK>
__device__ __forceinline__ int epilogue_inner(T *row, int64_t step, bool accu, const f32x4 (&acc)[TM][TN],
                                              const float (&sa)[TM], const f32x4 (&sb)[TN], const int64_t rows_left) {
    int stores = 0;
    static_for<0, TM>([&](auto ic) {
        constexpr int i = ic;
        const bool    live = !ROWCHECK || 16 * i < rows_left;
        if constexpr (sizeof(T) == 4) {
            // accumulating: the old values of four tiles are requested together, then used (one
            // load at a time would pay the memory latency TN times per row)
            constexpr int JB = TN < 4 ? TN : 4;
            static_for<0, TN / JB>([&](auto jbc) {
                constexpr int j0 = JB * jbc;
                // one branch holds the loads AND their uses: a load whose use sat behind a second
                // test of the same condition would look outstanding, to the compiler's wait-count
                // bookkeeping, on the path that skips that use, and the K loop of a persistent
                // kernel would then open every slab with a full vmcnt(0) wait that drains its
                // direct-to-LDS copies
                auto tile_value = [&](auto jc2) {
                    constexpr int j = jc2;
                    f32x4         v = read_acc<ACC_IN_AGPR>(acc[i][j]);
                    if constexpr (MODE == SCALE_VECTOR) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] = v[e] * sa[i] * sb[j][e];
                    }
                    return v;
                };
                if (accu && live) {
                    f32x4 old[JB];
#pragma unroll
                    for (int jj = 0; jj < JB; ++jj)
                        old[jj] = *reinterpret_cast<const f32x4 *>(row + (j0 + jj) * 16);
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, JB>([&](auto jjc) {
                        constexpr int j = j0 + jjc;
                        *reinterpret_cast<f32x4 *>(row + j * 16) = tile_value(std::integral_constant<int, j>{}) + old[j - j0];
                        // keep each accumulator's read next to its store (register pressure)
                        __builtin_amdgcn_sched_barrier(0);
                    });
                } else if (live) {
                    static_for<0, JB>([&](auto jjc) {
                        constexpr int j = j0 + jjc;
                        *reinterpret_cast<f32x4 *>(row + j * 16) = tile_value(std::integral_constant<int, j>{});
                        __builtin_amdgcn_sched_barrier(0);
                    });
                }
                stores += JB;
            });
        } else {
            // Two tiles (j, j + 1) give a lane eight consecutive columns after an exchange between
            // lane groups (v_permlane16_swap, written out by hand: the compiler's builtin for this
            // instruction loses track of vector elements; the wait states cover the VALU writes
            // just before). One test of `live` per row group. The plain form packs first, so the
            // exchange moves two registers per tile pair; the accumulating form exchanges the fp32
            // values, requests the old values of the row group together and adds in fp32.
            auto swap16 = [](auto &p, auto &q) { asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(p), "+v"(q)); };
            auto scaled = [&](auto jc2) {
                constexpr int j = jc2;
                f32x4         v = read_acc<ACC_IN_AGPR>(acc[i][j]);
                if constexpr (MODE == SCALE_VECTOR) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        v[e] = v[e] * sa[i] * sb[j][e];
                }
                return v;
            };
            if (live) {
                if (accu) {
                    u32x4 old[TN / 2];
#pragma unroll
                    for (int jj = 0; jj < TN / 2; ++jj)
                        old[jj] = *reinterpret_cast<const u32x4 *>(row + jj * 32);
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, TN / 2>([&](auto jc) {
                        constexpr int j = 2 * jc;
                        f32x4         x = scaled(std::integral_constant<int, j>{}), y = scaled(std::integral_constant<int, j + 1>{});
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            float xe = x[e], ye = y[e];
                            swap16(xe, ye);
                            x[e] = xe;
                            y[e] = ye;
                        }
                        asm volatile("s_nop 1" ::: "memory");
                        const u32x4 &o = old[jc];
                        float        o0, o1;
                        unpack2<T>(o.x, o0, o1); x[0] += o0; x[1] += o1;
                        unpack2<T>(o.y, o0, o1); x[2] += o0; x[3] += o1;
                        unpack2<T>(o.z, o0, o1); y[0] += o0; y[1] += o1;
                        unpack2<T>(o.w, o0, o1); y[2] += o0; y[3] += o1;
                        *reinterpret_cast<u32x4 *>(row + j * 16) =
                            u32x4{pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3]), pack2<T>(y[0], y[1]), pack2<T>(y[2], y[3])};
                        __builtin_amdgcn_sched_barrier(0);
                    });
                } else {
                    static_for<0, TN / 2>([&](auto jc) {
                        constexpr int j = 2 * jc;
                        const f32x4   x = scaled(std::integral_constant<int, j>{}), y = scaled(std::integral_constant<int, j + 1>{});
                        uint32_t      w0 = pack2<T>(x[0], x[1]), w1 = pack2<T>(x[2], x[3]);
                        uint32_t      w2 = pack2<T>(y[0], y[1]), w3 = pack2<T>(y[2], y[3]);
                        swap16(w0, w2);
                        swap16(w1, w3);
                        asm volatile("s_nop 1" ::: "memory");
                        *reinterpret_cast<u32x4 *>(row + j * 16) = u32x4{w0, w1, w2, w3}; // (streaming stores measured no faster here)
                        __builtin_amdgcn_sched_barrier(0);
                    });
                }
            }
            stores += TN / 2;
        }
        row += step;
    });
    return stores; // (a compile-time constant after unrolling: TM * TN, or TM * TN / 2 for 16-bit outputs)
}

__device__ __forceinline__ void store_elem(float f, uint8_t *q, int out_dtype, bool accu) {
    if (out_dtype == PT_DTYPE_F32) {
        float *p = reinterpret_cast<float *>(q);
        *p       = accu ? f + *p : f;
    } else if (out_dtype == PT_DTYPE_BF16) {
        bf16_t *p = reinterpret_cast<bf16_t *>(q);
        *p        = HP<bf16_t>::from_f32(accu ? f + HP<bf16_t>::to_f32(*p) : f);
    } else {
        f16_t *p = reinterpret_cast<f16_t *>(q);
        *p       = HP<f16_t>::from_f32(accu ? f + HP<f16_t>::to_f32(*p) : f);
    }
}

// `Cm` / `sAm` / `sBm` / `m_end` describe the matrix the tile belongs to (the whole problem,
// or one group's share of it).
// Returns (uniform over the wavefront) how many of the vector-memory operations it issued are
// guaranteed to be younger than everything issued before the call and may still be in flight on
// return: the store count of the straight-line path, 0 for the generic path. Kernels that wait
// for older direct-to-LDS copies by count (memory operations retire in order) leave exactly
// that many operations outstanding instead of waiting for the stores to be acknowledged.
// ROWCHECK = false keeps the 16-byte stores for sub-tiles that lie wholly inside the matrix only
// (a hanging one takes the generic path): for kernels that cannot afford the registers of the
// row test around their epilogue.
template <int TM, int TN, int MODE, bool ACC_IN_AGPR, bool ROWCHECK = true>
__device__ __forceinline__ int epilogue(const GemmArgs &a, const f32x4 (&acc)[TM][TN], uint8_t *Cm,
                                         const float *sAm, const float *sBm, int64_t m_end,
                                         int64_t wm_base, int64_t wn_base, int lane) {
    const int     ES = a.out_dtype == PT_DTYPE_F32 ? 4 : 2;
    const int     lm = lane & 15, lg = lane >> 4;
    uint8_t      *C    = Cm;
    const bool    accu = a.accumulate != 0;
    const int64_t m0 = wm_base + lm, n0 = wn_base + lg * 4;

    [[maybe_unused]] float sa[TM];
    [[maybe_unused]] f32x4 sb[TN];
    if constexpr (MODE == SCALE_VECTOR) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int64_t m = m0 + i * 16;
            sa[i]           = sAm[(m < a.M ? m : a.M - 1) * a.sa_m];
        }
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t n = n0 + j * 16 + e;
                sb[j][e]        = sBm[(n < a.N ? n : a.N - 1) * a.sb_n];
            }
        // The scales are used inside the row tests below. On a path that skipped every one of those
        // blocks the loads would still count as outstanding in the compiler's wait-count bookkeeping
        // when the K loop of the next tile begins, and it would open every slab with a full
        // vmcnt(0) wait: an (empty) use of each value here makes the loads complete on every path.
#pragma unroll
        for (int i = 0; i < TM; ++i)
            asm volatile("" ::"v"(sa[i]));
#pragma unroll
        for (int j = 0; j < TN; ++j)
            asm volatile("" ::"v"(sb[j]));
    }
    // all columns of the sub-tile inside the matrix and every 16-byte group aligned: 16-byte stores,
    // with the row groups beyond the end of the matrix (the end of a group's rows) left out
    // (only a sub-tile that lies wholly inside is certain to have issued every store it counts)
    const bool whole = wm_base + TM * 16 <= m_end;
    const bool fast  = (ROWCHECK || whole) && wn_base + TN * 16 <= a.N && (a.N & 7) == 0 &&
                      (reinterpret_cast<uintptr_t>(C) & 15) == 0;
    uint8_t      *row  = C + (m0 * a.N + n0) * ES;
    const int64_t step = 16 * a.N;
    const int64_t rows_left = m_end - m0;
    if (fast) {
        // 16-bit outputs: the lane's eight columns after the exchange between tile pairs
        uint8_t *rowp = C + (m0 * a.N + wn_base + 16 * (lg & 1) + 8 * (lg >> 1)) * 2;
        int stores;
        if (a.out_dtype == PT_DTYPE_BF16)
            stores = epilogue_inner<bf16_t, TM, TN, MODE, ACC_IN_AGPR, ROWCHECK>(reinterpret_cast<bf16_t *>(rowp), step, accu, acc, sa, sb, rows_left);
        else if (a.out_dtype == PT_DTYPE_F16)
            stores = epilogue_inner<f16_t, TM, TN, MODE, ACC_IN_AGPR, ROWCHECK>(reinterpret_cast<f16_t *>(rowp), step, accu, acc, sa, sb, rows_left);
        else
            stores = epilogue_inner<float, TM, TN, MODE, ACC_IN_AGPR, ROWCHECK>(reinterpret_cast<float *>(row), step, accu, acc, sa, sb, rows_left);
        return whole ? stores : 0;
    } else {
        static_for<0, TM>([&](auto ic) {
            constexpr int i = ic;
            static_for<0, TN>([&](auto jc) {
                constexpr int j = jc;
                f32x4         v = read_acc<ACC_IN_AGPR>(acc[i][j]);
                if constexpr (MODE == SCALE_VECTOR) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        v[e] = v[e] * sa[i] * sb[j][e];
                }
                if (m0 + i * 16 < m_end) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n0 + j * 16 + e < a.N)
                            store_elem(v[e], row + (j * 16 + e) * ES, a.out_dtype, accu);
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            row += step * ES;
        });
    }
    return 0;
}

// Wavefront-uniform 64-bit loads of values written before the launch (group offsets), through the
// scalar cache. Left to the compiler these are vector loads -- the kernel also stores to global
// memory, so it cannot prove the location unclobbered -- and the wait for a vector load is also a
// wait for every result-tile store issued before it (memory operations retire in order): each
// tile of a grouped problem would begin by draining the previous tile's stores.
__device__ __forceinline__ void uniform_load_pair(const int64_t *p, int64_t &v0, int64_t &v1) {
#if defined(__HIP_DEVICE_COMPILE__) // the host pass cannot parse the scalar-register constraint
    asm volatile("s_load_dwordx2 %0, %2, 0x0\n\t"
                 "s_load_dwordx2 %1, %2, 0x8\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&s"(v0), "=&s"(v1)
                 : "s"(p)
                 : "memory");
#else
    v0 = p[0];
    v1 = p[1];
#endif
}
__device__ __forceinline__ int64_t uniform_load(const int64_t *p) {
    int64_t v;
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_load_dwordx2 %0, %1, 0x0\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=s"(v)
                 : "s"(p)
                 : "memory");
#else
    v = p[0];
#endif
    return v;
}

// Where a workgroup's tile lives. The second half only varies between tiles of grouped
// problems; in the dense case it repeats the kernel arguments.
struct TileCtx {
    const uint8_t *Ag, *Bg; // first row of the tile in A / B (at the tile's first K column)
    int            rows_a, rows_b;
    int64_t        m0, n0;  // first output row / column (row index in the tile's C matrix)
    int64_t        m_end;   // rows of C at or beyond this belong to someone else
    const float   *sA, *sB; // scale arrays of the tile's matrix (BLOCK: at its first K block)
    uint8_t       *C;       // the tile's output matrix
    int            KT;      // K slabs of this tile
    int            g0, g1;  // GROUP_K: the unit's groups [g0, g1) (KT = slabs of all of them)
};

// GROUP_ROWS: prefix[g] = number of tiles of the groups before g (in LDS), `g` is a search
// hint that only moves forward as a workgroup walks its tiles.
template <int BM, int BN, int GMODE, bool F4 = false>
__device__ __forceinline__ TileCtx make_tile(const GemmArgs &a, int tile, const int *prefix, int &g) {
    TileCtx t;
    t.g0 = t.g1 = 0;
    int tm, tn;
    if constexpr (GMODE == GROUP_NONE) {
        tile_coords(tile, a.tiles_m, a.tiles_n, tm, tn);
        t.m0    = static_cast<int64_t>(tm) * BM;
        t.m_end = a.M;
        t.Ag    = a.A + t.m0 * a.lda;
        t.Bg    = a.B;
        t.sA    = a.sA;
        t.sB    = a.sB;
        t.C     = static_cast<uint8_t *>(a.C);
        t.KT    = static_cast<int>(a.K / KSTEP);
    } else if constexpr (GMODE == GROUP_ROWS) {
        // (tile ids stay round-robin over the XCDs here: the XCD-contiguous renumbering of the
        // dense case measured 3-15% slower on Zipf-distributed groups)
        while (g + 1 < a.G && tile >= __builtin_amdgcn_readfirstlane(prefix[g + 1]))
            ++g;
        const int     local = tile - __builtin_amdgcn_readfirstlane(prefix[g]);
        int64_t lo, hi, out_lo = 0, out_hi = 0;
        uniform_load_pair(a.group_offs + g, lo, hi);
        // with separate output offsets the group's row count is theirs (A may be padded per group)
        if (a.group_offs_out != nullptr) {
            uniform_load_pair(a.group_offs_out + g, out_lo, out_hi);
            hi = lo + (out_hi - out_lo);
        }
        const int     gtm = static_cast<int>((hi - lo + BM - 1) / BM);
        group_tile_coords(local, gtm, a.tiles_n, tm, tn);
        t.m0    = lo + static_cast<int64_t>(tm) * BM;
        t.m_end = hi;
        t.Ag    = a.A + t.m0 * a.lda;
        t.Bg    = a.B + g * a.b_gstride;
        t.sA    = a.sA;
        t.sB    = a.sB + g * a.sb_gstride;
        t.C     = static_cast<uint8_t *>(a.C);
        if (a.group_offs_out != nullptr) // the tile's rows keep their A numbering; C moves instead
            t.C += (out_lo - lo) * a.N * (a.out_dtype == PT_DTYPE_F32 ? 4 : 2);
        t.KT    = static_cast<int>(a.K / KSTEP);
    } else {
        // unit = (chunk of consecutive groups, output position); the positions in XCD-contiguous
        // order (workgroup i runs on XCD i % 8 and walks units i, i + grid, ...): every XCD works on a
        // compact block of the output, so the chunk's operand panels are fetched into few L2s, and
        // all workgroups are in the same chunk at the same time
        const int per   = a.tiles_m * a.tiles_n;
        const int chunk = tile / per;
        tile_coords_local(xcd_contiguous_id(tile - chunk * per, per), a.tiles_m, a.tiles_n, tm, tn);
        t.g0 = __builtin_amdgcn_readfirstlane(prefix[chunk]);
        t.g1 = __builtin_amdgcn_readfirstlane(prefix[chunk + 1]);
        g    = t.g0;
        // K ranges are given in elements; two E2M1 codes share a byte
        const int64_t lo = uniform_load(a.group_offs + t.g0) >> (F4 ? 1 : 0), hi = uniform_load(a.group_offs + t.g1) >> (F4 ? 1 : 0);
        t.m0    = static_cast<int64_t>(tm) * BM;
        t.m_end = a.M;
        t.Ag    = a.A + t.m0 * a.lda + lo;
        t.Bg    = a.B + lo;
        t.sA    = a.sA + (lo / KSTEP) * a.sa_k;
        t.sB    = a.sB + (lo / KSTEP) * a.sb_k;
        t.C     = static_cast<uint8_t *>(a.C);
        t.KT    = static_cast<int>((hi - lo) / KSTEP);
    }
    t.n0     = static_cast<int64_t>(tn) * BN;
    t.rows_a = (t.m_end - t.m0) < BM ? static_cast<int>(t.m_end - t.m0) : BM;
    t.rows_b = (a.N - t.n0) < BN ? static_cast<int>(a.N - t.n0) : BN;
    t.Bg += t.n0 * a.ldb;
    return t;
}

// Persistent kernel: the grid is sized to the machine and every workgroup walks tiles
// blockIdx.x, blockIdx.x + gridDim.x, ... as one uninterrupted sequence of K steps
// ("slabs" of 128 bytes of K, rotating through the LDS stages). With one wavefront per SIMD
// nothing hides a stall, and the path from L2 into the LDS moves about 64 bytes per clock and
// CU -- more than half of what the MFMAs of a 256 x 256 tile consume per clock -- so a slab
// is scheduled such that no MFMA waits for an LDS round trip and the copies are spread over
// the whole slab instead of arriving at the copy unit in bursts:
//   * all MFMA operand fragments of the slab being multiplied live in registers; the MFMA
//     tiles (i, j) are walked column by column, and a fragment is refilled from the next
//     slab's stage as soon as it is dead: B fragment j after column j, A fragment i after
//     tile (i, TN - 1). Every LDS read is thus issued at least TM MFMAs before its first use;
//   * the stage of the slab being multiplied is therefore only read during the slab before,
//     and receives the slab two steps ahead during the current one: the B part (and the block
//     scales) while columns 1 .. TN/2 - 1 are multiplied, the A part during the rest. Where
//     three stages fit, that slab goes into the stage freed one slab ago instead, and its
//     copies are spread over all of the current slab's MFMAs;
//   * two barriers per slab: "X" after column 0 (everyone has finished reading the current
//     stage; everyone's copies of the next slab's B part have landed) and "Y" after column
//     TN/2 - 1 (the next slab's A part has landed). Both wait for copies requested at least
//     half a slab earlier;
//   * tile boundaries do not drain the pipeline: while a tile's result is written out, the
//     fragments of the next tile's first slab are already in registers and its second slab is
//     in flight.
template <int TM, int TN, int MODE, bool SB_VEC, int FA, int FB, int GMODE>
__global__ __launch_bounds__(256) void gemm_fp8_nt_kernel(const GemmArgs a) {
    static_assert(TN % 4 == 0 && TM % 4 == 0, "sub-tiles are multiples of 64 x 64");
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    constexpr int A_BYTES = BM * KSTEP, B_BYTES = BN * KSTEP, STAGE = gemm_stage_bytes(TM, TN, MODE, FA == 4);
    constexpr int NSTAGE = gemm_stages(TM, TN, FA == 4);
    constexpr int LA = BM / 8 / GEMM_WAVES, LB = BN / 8 / GEMM_WAVES; // data copies per wave and slab
    constexpr int NLD = LA + LB;
    // MXFP4: a 128-byte slab row holds 256 E2M1 codes, i.e. two MFMAs' worth of K; a lane's two
    // 16-byte fragment reads (chunks g and 4 + g) then feed one MFMA each instead of one together
    constexpr bool F4 = FA == 4;
    static_assert((FA == 4) == (FB == 4), "FP4 operands come in pairs");
    constexpr int NH = F4 ? 2 : 1; // MFMAs per fragment pair
    // BLOCK and MX modes: the scales of a slab travel with it through the stages. Per row
    // (column) of the wavefront's sub-tile and slab that is one 32-bit word -- an fp32 block
    // scale, or the E8M0 bytes of four 32-wide K blocks (two words for MXFP4) -- fetched 64 rows
    // per copy instruction into an area of the stage that is private to the wavefront.
    constexpr bool LDS_SC  = MODE != SCALE_VECTOR;
    constexpr int  SC_A    = TM * 16, SC_B = TN * 16, SC_ROWS = SC_A + SC_B;
    constexpr int  NW      = MODE == SCALE_MX ? NH : 1;       // scale words per row and slab
    constexpr int  NSC     = LDS_SC ? NW * SC_ROWS / 64 : 0;  // scale copies per wave and slab
    constexpr int  SC_WAVE = NW * SC_ROWS * 4;                // bytes of a wavefront's scale area
    constexpr int  SC_ELT  = MODE == SCALE_MX ? 1 : 4;        // bytes per scale array element
    constexpr int  NB      = LB + NSC;                        // copies of the "B part" of a slab
    constexpr int  NL      = NLD + NSC;                       // copies per wave and slab
    constexpr int  JY      = TN / 2;                          // barrier Y follows column JY - 1
    constexpr int  NSB     = SB_VEC ? 4 : 1;
    static_assert(MODE != SCALE_BLOCK || SB_VEC || TN * 16 <= 128, "one B scale per wavefront and slab");
    [[maybe_unused]] uint32_t unit_scale = 0x7f7f7f7fu; // E8M0 1.0 for all four K blocks
    // GROUP_K: a "tile" is a unit of work, one output position streaming through the K ranges of a
    // chunk of consecutive groups (they lie side by side along K): the slab sequence continues
    // across group boundaries, where the sums are written to the group's C and cleared. Units have
    // their own K extent (possibly none at all), so the pipeline is restarted per unit instead of
    // running across unit boundaries; only the request for a unit's first two slabs is moved
    // ahead of the previous unit's last epilogue.
    constexpr bool XPIPE = GMODE != GROUP_K;
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1; // wavefront position in the 2 x 2 grid
    const int lm = lane & 15, lg = lane >> 4;

    // byte offsets of this lane's two 16-byte fragment reads within a 16-row group
    const uint32_t frag_off_lo = lm * KSTEP + ((lg ^ swz(lm)) << 4);
    const uint32_t frag_off_hi = lm * KSTEP + (((4 + lg) ^ swz(lm)) << 4);

    // ---- tile list ----
    // GROUP_ROWS: tiles before group g; GROUP_K: first group of chunk c
    int *prefix = reinterpret_cast<int *>(smem + NSTAGE * STAGE);
    int  total;
    if constexpr (GMODE == GROUP_ROWS) {
        for (int g = tid; g < a.G; g += 256) {
            const int64_t *o   = a.group_offs_out != nullptr ? a.group_offs_out : a.group_offs;
            const int64_t rows = o[g + 1] - o[g];
            prefix[g + 1]      = static_cast<int>((rows + BM - 1) / BM) * a.tiles_n;
        }
        __syncthreads();
        if (tid == 0) {
            int run = 0;
            prefix[0] = 0;
            for (int g = 1; g <= a.G; ++g) {
                run += prefix[g];
                prefix[g] = run;
            }
        }
        __syncthreads();
        total = __builtin_amdgcn_readfirstlane(prefix[a.G]);
    } else if constexpr (GMODE == GROUP_K) {
        // chunk c = groups [prefix[c], prefix[c + 1]): its first group is the first one that starts at
        // or behind c / chunks of the total K length
        const int     chunks  = a.vk_chunks;
        const int64_t k_first = a.group_offs[0], k_total = a.group_offs[a.G] - k_first;
        if (tid <= chunks)
            prefix[tid] = a.G;
        __syncthreads();
        for (int g = tid; g < a.G; g += 256) {
            const int64_t cum = a.group_offs[g] - k_first, prev = g > 0 ? a.group_offs[g - 1] - k_first : -1;
            for (int c = 0; c < chunks; ++c) {
                const int64_t thr = k_total * c / chunks;
                if (cum >= thr && prev < thr)
                    prefix[c] = g;
            }
        }
        __syncthreads();
        total = chunks * a.tiles_m * a.tiles_n;
    } else {
        total = a.tiles_m * a.tiles_n;
    }
    const int KT_ALL = static_cast<int>(a.K / KSTEP); // XPIPE: every tile has this many slabs (> 2)
    int       tile   = blockIdx.x;
    if (tile >= total || (XPIPE && KT_ALL <= 2))
        return;
    int     g_cur = 0, g_nxt = 0;
    TileCtx cur_t = make_tile<BM, BN, GMODE, FA == 4>(a, tile, prefix, g_cur);
    g_nxt         = g_cur;

    // ---- loader: two slabs ahead of the MFMAs ----
    // Copies are buffer loads: a lane's offset inside a slab (row * pitch + swizzled chunk)
    // is the same for every tile; the tile and the K position live in the (uniform) buffer
    // descriptor, whose size makes rows beyond the tile's share of the matrix read as zero.
    // The loader therefore changes tile by swapping scalars -- no branch in the K loop, which
    // the compiler would use to sink MFMAs -- and it does so after requesting the tile's last
    // slab, two steps before the MFMAs get there (the host guarantees KT > 2). Without
    // cross-tile pipelining it stops at the tile's last slab and keeps re-reading that one.
    // scale addressing in bytes: from one row (column) to the next, and (MX) from one 32-bit word
    // of a row to its next
    [[maybe_unused]] const bool     mx_wordmajor = MODE == SCALE_MX && a.sa_wpitch != 0;
    [[maybe_unused]] const uint32_t sa_rowp  = mx_wordmajor ? 4u : static_cast<uint32_t>(a.sa_m) * (MODE == SCALE_MX ? 1 : 4);
    [[maybe_unused]] const uint32_t sb_rowp  = mx_wordmajor ? 4u : static_cast<uint32_t>(a.sb_n) * (MODE == SCALE_MX ? 1 : 4);
    [[maybe_unused]] const uint32_t sa_wordp = mx_wordmajor ? static_cast<uint32_t>(a.sa_wpitch) : 4u;
    [[maybe_unused]] const uint32_t sb_wordp = mx_wordmajor ? static_cast<uint32_t>(a.sb_wpitch) : 4u;
    uint32_t off[NL];
    {
        const int lrow = lane >> 3, pchk = lane & 7;
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const bool isA = j < LA;
            const int  row = ((isA ? j : j - LA) * GEMM_WAVES + wave) * 8 + lrow;
            off[j] = static_cast<uint32_t>(row * (isA ? a.lda : a.ldb)) + ((pchk ^ swz(row)) << 4);
        }
        // scale copies: lane l of copy q fetches the word of the wavefront's row (or column)
        // 64 q + l, at an offset relative to the scale of the tile's first row / column (exact,
        // because tiles start on multiples of 128 wherever a scale spans 128 rows)
#pragma unroll
        for (int q = 0; q < NSC; ++q) {
            const int e = (q % (SC_ROWS / 64)) * 64 + lane;
            if (e < SC_A)
                off[NLD + q] = static_cast<uint32_t>((wm * SC_A + e) >> a.sa_shift) * sa_rowp +
                               (q / (SC_ROWS / 64)) * sa_wordp; // (+ the second scale word of an MXFP4 slab)
            else
                off[NLD + q] = static_cast<uint32_t>((wn * SC_B + e - SC_A) >> a.sb_shift) * sb_rowp +
                               (q / (SC_ROWS / 64)) * sb_wordp;
        }
    }
    const uint8_t *ld_ga, *ld_gb; // slab the loader points at
    uint32_t       ld_na, ld_nb;  // bytes from there to the end of the tile's rows
    int            ld_kt;
    int            ld_KT = 0;     // slabs of the loader's tile (tiles with their own K extent)
    // scales of the loader's slab for the tile's first row / column, and the end of the scale
    // arrays (reads beyond return zero; they only ever meet rows that are never stored)
    [[maybe_unused]] const uint8_t *ld_sa = nullptr, *ld_sb = nullptr, *ld_sa_end = nullptr, *ld_sb_end = nullptr;
    [[maybe_unused]] const int64_t  sa_extent =
        MODE == SCALE_MX ? (mx_wordmajor ? static_cast<int64_t>((a.kb_valid + 3) / 4) * a.sa_wpitch : (a.M - 1) * a.sa_m + a.kb_valid)
                         : (((a.M - 1) >> a.sa_shift) * a.sa_m + (a.kb_valid - 1) * a.sa_k + 1) * 4;
    [[maybe_unused]] const int64_t sb_extent =
        MODE == SCALE_MX ? (mx_wordmajor ? static_cast<int64_t>((a.kb_valid + 3) / 4) * a.sb_wpitch : (a.N - 1) * a.sb_n + a.kb_valid)
                         : (((a.N - 1) >> a.sb_shift) * a.sb_n + (a.kb_valid - 1) * a.sb_k + 1) * 4;
    [[maybe_unused]] const int64_t sa_step = MODE == SCALE_MX ? static_cast<int64_t>(NW) * sa_wordp : a.sa_k * 4; // bytes per slab
    [[maybe_unused]] const int64_t sb_step = MODE == SCALE_MX ? static_cast<int64_t>(NW) * sb_wordp : a.sb_k * 4;
    auto as_bytes = [](const float *p) { return reinterpret_cast<const uint8_t *>(p); };
    auto scales_to = [&](const TileCtx &t) {
        if constexpr (LDS_SC) {
            ld_sa     = as_bytes(t.sA) + (t.m0 >> a.sa_shift) * sa_rowp;
            ld_sb     = as_bytes(t.sB) + (t.n0 >> a.sb_shift) * sb_rowp;
            ld_sa_end = as_bytes(GMODE == GROUP_K ? a.sA : t.sA) + sa_extent;
            ld_sb_end = as_bytes(GMODE == GROUP_K ? a.sB : t.sB) + sb_extent;
        }
    };
    TileCtx nxt_t     = cur_t; // tile after the MFMAs' tile (the same tile after the last one)
    auto    loader_to = [&](const TileCtx &t) {
        ld_ga = t.Ag;
        ld_gb = t.Bg;
        ld_na = t.rows_a * static_cast<uint32_t>(a.lda);
        ld_nb = t.rows_b * static_cast<uint32_t>(a.ldb);
        ld_kt = 0;
        ld_KT = t.KT;
        scales_to(t);
    };
    // bytes a scale copy may read: none for a slab of zero padding beyond the K blocks the
    // arrays hold (whatever lies there must not meet the matrix core: an E8M0 NaN would stick)
    [[maybe_unused]] auto bytes_left = [&](const uint8_t *p, const uint8_t *end, int h) {
        const int64_t n     = end - p;
        const bool    valid = GMODE == GROUP_K || (MODE == SCALE_MX ? (ld_kt * NW + h) * 4 : ld_kt) < a.kb_valid;
        return (n <= 0 || !valid) ? 0u : (n > 0x7fffffff ? 0x7fffffffu : static_cast<uint32_t>(n));
    };
    // copy number L of the loader's slab into stage `b`: [0, LA) A rows, [LA, NLD) B rows,
    // [NLD, NL) scale words
    auto issue_copy = [&](auto lc, int b) {
        constexpr int L   = lc;
        uint8_t      *dst = smem + b * STAGE;
#if defined(__HIP_DEVICE_COMPILE__) // the buffer resource type only exists in the device pass
        constexpr uint32_t RSRC_FLAGS = 0x00020000; // raw buffer, 32-bit data format
        if constexpr (L >= NLD) {
            constexpr int  Q = L - NLD, H = Q / (SC_ROWS / 64), QQ = Q % (SC_ROWS / 64);
            constexpr bool isA = QQ * 64 < SC_A;
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint8_t *>(isA ? ld_sa : ld_sb), 0,
                isA ? bytes_left(ld_sa, ld_sa_end, H) : bytes_left(ld_sb, ld_sb_end, H), RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + A_BYTES + B_BYTES + wave * SC_WAVE + Q * 256), 4,
                                                     off[L], 0, 0, 0);
        } else if constexpr (L < LA) {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_ga), 0, ld_na, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + (L * GEMM_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        } else {
            __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(ld_gb), 0, ld_nb, RSRC_FLAGS);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr_t)(dst + A_BYTES + ((L - LA) * GEMM_WAVES + wave) * 1024), 16, off[L], 0, 0, 0);
        }
#endif
    };
    // the copies of a slab in issue order: B part (B rows, then scales), then A part
    auto issue_part_b = [&](auto cc, int b) {
        constexpr int C = cc;
        issue_copy(std::integral_constant<int, (C < LB ? LA + C : NLD + (C - LB))>{}, b);
    };
    auto advance_loader = [&]() {
        if constexpr (XPIPE) {
            const bool wrap = ld_kt + 1 == KT_ALL;
            ld_kt = wrap ? 0 : ld_kt + 1;
            ld_ga = wrap ? nxt_t.Ag : ld_ga + KSTEP;
            ld_gb = wrap ? nxt_t.Bg : ld_gb + KSTEP;
            ld_na = wrap ? nxt_t.rows_a * static_cast<uint32_t>(a.lda) : ld_na - KSTEP;
            ld_nb = wrap ? nxt_t.rows_b * static_cast<uint32_t>(a.ldb) : ld_nb - KSTEP;
            if constexpr (LDS_SC) {
                const uint8_t *na = as_bytes(nxt_t.sA) + (nxt_t.m0 >> a.sa_shift) * sa_rowp;
                const uint8_t *nb = as_bytes(nxt_t.sB) + (nxt_t.n0 >> a.sb_shift) * sb_rowp;
                ld_sa             = wrap ? na : ld_sa + sa_step;
                ld_sb             = wrap ? nb : ld_sb + sb_step;
                ld_sa_end         = wrap ? as_bytes(nxt_t.sA) + sa_extent : ld_sa_end;
                ld_sb_end         = wrap ? as_bytes(nxt_t.sB) + sb_extent : ld_sb_end;
            }
        } else {
            const int adv = ld_kt + 1 < ld_KT ? KSTEP : 0;
            ld_kt += adv / KSTEP;
            ld_ga += adv;
            ld_gb += adv;
            ld_na -= adv;
            ld_nb -= adv;
            if constexpr (LDS_SC) {
                ld_sa += adv ? sa_step : 0;
                ld_sb += adv ? sb_step : 0;
            }
        }
    };

    // BLOCK mode: the fp32 scales of a slab are read from its stage one slab ahead (after
    // barrier X). Without per-column scales one B value serves the whole wavefront and is
    // multiplied into the row scales once per slab.
    constexpr int NSBJ = SB_VEC ? TN : 1;
    [[maybe_unused]] float sa_nxt[TM], sb_nxt[NSBJ][NSB], sc_cur[TM], sb_cur[NSBJ][NSB];
    // MX mode: lane (r, g) takes the E8M0 byte of fragment row r and K block g
    [[maybe_unused]] uint32_t mxa_cur[TM][NH], mxa_nxt[TM][NH], mxb_cur[TN][NH], mxb_nxt[TN][NH];
    auto read_scales = [&](const uint8_t *stage) {
        if constexpr (MODE == SCALE_BLOCK) {
            const float *reg = reinterpret_cast<const float *>(stage + A_BYTES + B_BYTES + wave * SC_WAVE);
#pragma unroll
            for (int i = 0; i < TM; ++i)
                sa_nxt[i] = reg[i * 16 + lm];
            if constexpr (SB_VEC) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(reg + SC_A + j * 16 + lg * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        sb_nxt[j][e] = v[e];
                }
            } else {
                sb_nxt[0][0] = reg[SC_A];
            }
        }
        if constexpr (MODE == SCALE_MX) {
            const uint8_t *reg = stage + A_BYTES + B_BYTES + wave * SC_WAVE + lm * 4 + lg;
#pragma unroll
            for (int h = 0; h < NH; ++h) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    mxa_nxt[i][h] = reg[(h * SC_ROWS + i * 16) * 4];
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    mxb_nxt[j][h] = reg[(h * SC_ROWS + SC_A + j * 16) * 4];
            }
        }
    };

    f32x4 acc[TM][TN];
    // MFMA operand fragments (8 VGPRs each) of the slab being multiplied
    i32x8 fa[TM], fb[TN];
    int   buf = 0;

    // fragment f (16 rows) of the A or B part of a stage: two 16-byte LDS reads per lane
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

    // pipeline start at tile t, in two steps: the first two slabs are requested (stages 0 and 1,
    // which nobody may still be reading) ...
    auto request_first_slabs = [&](const TileCtx &t) {
        loader_to(t);
        static_for<0, 2>([&](auto st) {
            static_for<0, NB>([&](auto c) { issue_part_b(c, st); });
            static_for<0, LA>([&](auto c) { issue_copy(c, st); });
            advance_loader();
        });
    };
    // ... and, once slab 0 has landed, its fragments go into registers. The wait leaves NL
    // operations in flight: whatever else was issued after the two slabs (output stores of the
    // previous tile), the copies of slab 0 are older than the NL copies of slab 1 and copies
    // complete in order, so none of them can be among the NL youngest.
    auto take_first_slab = [&]() {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NL) : "memory");
        __builtin_amdgcn_s_barrier();
        buf = 0;
        read_scales(smem);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[j] = ldfrag(smem + b_part, j);
#pragma unroll
        for (int i = 0; i < TM; ++i)
            fa[i] = ldfrag(smem + a_part, i);
    };
    // Stores of the result tile a wavefront has just written that may still be in flight (0, or the
    // count of the straight-line epilogue for 16-bit / fp32 outputs). They are younger than the
    // copies the first slab of the next tile waits for and older than that slab's own copies;
    // memory operations retire in order, so the first slab's waits leave that many more
    // operations outstanding instead of waiting for the stores to be acknowledged.
    constexpr int ST16 = TM * TN / 2, ST32 = TM * TN;
    int           pending = 0;
    PT_GEMM_TRACE_DECL;
    PT_GEMM_TRACE_POINT(0);
    if constexpr (XPIPE) {
        request_first_slabs(cur_t);
        take_first_slab();
    } else {
        if (cur_t.KT > 0)
            request_first_slabs(cur_t);
    }

    while (true) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int next_tile = tile + gridDim.x;
        nxt_t               = cur_t;
        if (next_tile < total)
            nxt_t = make_tile<BM, BN, GMODE, FA == 4>(a, next_tile, prefix, g_nxt);
        const int KT = XPIPE ? KT_ALL : cur_t.KT;
        if constexpr (!XPIPE) {
            if (KT > 0)
                take_first_slab(); // requested before the loop or before the previous tile's epilogue
            PT_GEMM_TRACE_POINT(1);
        }

        // one K slab per iteration; the body must stay a single basic block (no branches), or
        // the compiler sinks the MFMAs behind them
        auto run_slabs = [&](const int n_slabs) {
        for (int kt = 0; kt < n_slabs; ++kt) {
            const int      buf_n = buf + 1 == NSTAGE ? 0 : buf + 1;
            const uint8_t *nxt   = smem + buf_n * STAGE;
            // where the slab two steps ahead goes: the current stage (after barrier X), or with
            // three stages the one that was current a slab ago
            const int      buf_w = NSTAGE == 2 ? buf : (buf == 0 ? NSTAGE - 1 : buf - 1);
            if constexpr (MODE == SCALE_BLOCK) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    sc_cur[i] = SB_VEC ? sa_nxt[i] : sa_nxt[i] * sb_nxt[0][0];
#pragma unroll
                for (int j = 0; j < NSBJ; ++j)
#pragma unroll
                    for (int e = 0; e < NSB; ++e)
                        sb_cur[j][e] = sb_nxt[j][e];
            }
            if constexpr (MODE == SCALE_MX) {
#pragma unroll
                for (int h = 0; h < NH; ++h) {
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        mxa_cur[i][h] = mxa_nxt[i][h];
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        mxb_cur[j][h] = mxb_nxt[j][h];
                }
            }

            // BLOCK mode: MFMA t (in issue order, t = j TM + i) writes ring[t % RING]; DEPTH
            // MFMAs later its product is folded into the running sum with the block scales
            // (VALU work in the shadow of later MFMAs).
            [[maybe_unused]] constexpr int DEPTH = 3, RING = DEPTH + 1, TILES = TM * TN; // depth 2 costs a dozen wait states per fold
            [[maybe_unused]] f32x4 ring[RING];
            [[maybe_unused]] auto  fold = [&](int t) {
                const int    i = t % TM, j = t / TM;
                const f32x4 &p = ring[t % RING];
                if constexpr (SB_VEC) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][j][e] = fmaf(p[e], sc_cur[i] * sb_cur[SB_VEC ? j : 0][SB_VEC ? e : 0], acc[i][j][e]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[i][j][e] = fmaf(p[e], sc_cur[i], acc[i][j][e]);
                }
            };
            // h selects the half of an MXFP4 slab (always 0 otherwise)
            auto mma = [&](int i, int j, int h) {
                const i32x8 &af = fa[i], &bf = fb[j];
                if constexpr (MODE == SCALE_BLOCK) {
                    const int t    = j * TM + i;
                    ring[t % RING] = mfma_fp8<FA, FB>(bf, af, f32x4{0.f, 0.f, 0.f, 0.f});
                    if (t >= DEPTH)
                        fold(t - DEPTH);
                } else if constexpr (F4) {
                    const i32x4 bq = h ? __builtin_shufflevector(bf, bf, 4, 5, 6, 7) : __builtin_shufflevector(bf, bf, 0, 1, 2, 3);
                    const i32x4 aq = h ? __builtin_shufflevector(af, af, 4, 5, 6, 7) : __builtin_shufflevector(af, af, 0, 1, 2, 3);
                    mfma_inplace_f4(acc[i][j], bq, aq, mxb_cur[j][h ? NH - 1 : 0], mxa_cur[i][h ? NH - 1 : 0]);
                } else if constexpr (MODE == SCALE_MX) {
                    mfma_inplace<FA, FB>(acc[i][j], bf, af, mxb_cur[j][0], mxa_cur[i][0]);
                } else {
                    mfma_inplace<FA, FB>(acc[i][j], bf, af, unit_scale, unit_scale);
                }
            };

            // MFMA slots of a slab: s = (j NH + h) TM + i. B-part copies are spread over the
            // slots of columns [1, JY), A-part copies over those of columns [JY, TN).
            // (Three stages: both parts spread over all slots in proportion to their copy counts.)
            constexpr int COL = NH * TM, SLOTS = TN * COL;
            constexpr int S_B0 = NSTAGE == 2 ? COL : 0, S_B1 = NSTAGE == 2 ? JY * COL : SLOTS * NB / NL;
            constexpr int S_A0 = S_B1, S_A1 = SLOTS;
            // copies of this slab's schedule issued before slot s
            constexpr auto issued_before = [](int s) {
                const int b = s <= S_B0 ? 0 : (s >= S_B1 ? NB : (s - S_B0) * NB / (S_B1 - S_B0));
                const int a = s <= S_A0 ? 0 : (s >= S_A1 ? LA : (s - S_A0) * LA / (S_A1 - S_A0));
                return b + a;
            };
            static_for<0, TN>([&](auto jc) {
                constexpr int j = jc;
                static_for<0, COL>([&](auto sc) {
                    constexpr int h = sc / TM, i = sc % TM, s = j * COL + sc;
                    mma(i, j, h);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (j == TN - 1 && h == NH - 1)
                        fa[i] = ldfrag(nxt + a_part, i); // dead from here on: refill from the next slab
                    if constexpr (s >= S_B0 && s < S_B1)
                        static_for<(s - S_B0) * NB / (S_B1 - S_B0), (s + 1 - S_B0) * NB / (S_B1 - S_B0)>(
                            [&](auto c) { issue_part_b(c, buf_w); });
                    if constexpr (s >= S_A0 && s < S_A1)
                        static_for<(s - S_A0) * LA / (S_A1 - S_A0), (s + 1 - S_A0) * LA / (S_A1 - S_A0)>(
                            [&](auto c) { issue_copy(c, buf_w); });
                    __builtin_amdgcn_sched_barrier(0);
                });
                if constexpr (j == 0) {
                    // ---- barrier X ----
                    // my reads of the current stage are done (they were issued a column ago) and my
                    // copies of the next slab's B part have landed; younger copies may be in flight
                    PT_GEMM_TRACE_POINT(2);
                    // (the case distinction on `pending` lives inside the asm statement so that the
                    // slab stays one basic block for the compiler; the counter field holds 63 at most)
                    if constexpr (GMODE == GROUP_NONE) {
                        // (dense problems: few tiles per workgroup, and the case distinction costs
                        // about 1 % of a long K loop: the plain wait)
                        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LA + issued_before(COL)) : "memory");
                    } else {
                        constexpr int W = LA + issued_before(COL);
                        asm volatile("s_cmp_eq_u32 %0, 0\n\t"
                                     "s_cbranch_scc1 .Lx0_%=\n\t"
                                     "s_cmp_eq_u32 %0, %4\n\t"
                                     "s_cbranch_scc1 .Lx16_%=\n\t"
                                     "s_waitcnt vmcnt(%3) lgkmcnt(0)\n\t"
                                     "s_branch .Lxe_%=\n"
                                     ".Lx16_%=:\n\t"
                                     "s_waitcnt vmcnt(%2) lgkmcnt(0)\n\t"
                                     "s_branch .Lxe_%=\n"
                                     ".Lx0_%=:\n\t"
                                     "s_waitcnt vmcnt(%1) lgkmcnt(0)\n"
                                     ".Lxe_%=:"
                                     :
                                     : "s"(pending), "n"(W), "n"(W + ST16 > 63 ? 63 : W + ST16),
                                       "n"(W + ST32 > 63 ? 63 : W + ST32), "n"(ST16)
                                     : "memory", "scc");
                    }
                    __builtin_amdgcn_s_barrier();
                    PT_GEMM_TRACE_POINT(3);
                    read_scales(nxt);
                }
                if constexpr (j == JY - 1) {
                    // ---- barrier Y: the next slab's A part has landed ----
                    if constexpr (GMODE == GROUP_NONE) {
                        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(issued_before(JY * COL)) : "memory");
                    } else {
                        constexpr int W = issued_before(JY * COL);
                        asm volatile("s_cmp_eq_u32 %0, 0\n\t"
                                     "s_cbranch_scc1 .Ly0_%=\n\t"
                                     "s_cmp_eq_u32 %0, %4\n\t"
                                     "s_cbranch_scc1 .Ly16_%=\n\t"
                                     "s_waitcnt vmcnt(%3)\n\t"
                                     "s_branch .Lye_%=\n"
                                     ".Ly16_%=:\n\t"
                                     "s_waitcnt vmcnt(%2)\n\t"
                                     "s_branch .Lye_%=\n"
                                     ".Ly0_%=:\n\t"
                                     "s_waitcnt vmcnt(%1)\n"
                                     ".Lye_%=:"
                                     :
                                     : "s"(pending), "n"(W), "n"(W + ST16 > 63 ? 63 : W + ST16),
                                       "n"(W + ST32 > 63 ? 63 : W + ST32), "n"(ST16)
                                     : "memory", "scc");
                    }
                    pending = 0; // from the next slab on every wait is for copies younger than the stores
                    __builtin_amdgcn_s_barrier();
                }
                fb[j] = ldfrag(nxt + b_part, j); // column j is done: refill from the next slab
                __builtin_amdgcn_sched_barrier(0);
            });
            if constexpr (MODE == SCALE_BLOCK) {
#pragma unroll
                for (int t = TILES - DEPTH; t < TILES; ++t)
                    fold(t);
            }
            advance_loader();
            buf = buf_n;
        }
        };
        const int64_t wm_base = cur_t.m0 + wm * (TM * 16), wn_base = cur_t.n0 + wn * (TN * 16);
        if constexpr (XPIPE) {
            run_slabs(KT);
            PT_GEMM_TRACE_POINT(4);
            // the epilogue reads the accumulators with hand-written instructions the compiler's
            // hazard tracking does not see: let the last MFMA's write-back finish first
            if constexpr (MODE != SCALE_BLOCK)
                asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
            PT_GEMM_TRACE_POINT(5);
            // (0, ST16 or ST32: the stores of the epilogue's straight-line path)
            pending = __builtin_amdgcn_readfirstlane(epilogue<TM, TN, MODE, MODE != SCALE_BLOCK>(
                a, acc, cur_t.C, cur_t.sA, cur_t.sB, cur_t.m_end, wm_base, wn_base, lane));
        } else {
            const int ES     = a.out_dtype == PT_DTYPE_F32 ? 4 : 2;
            int64_t   g_lo   = uniform_load(a.group_offs + cur_t.g0) >> (F4 ? 1 : 0);
            for (int g = cur_t.g0; g < cur_t.g1; ++g) {
                const int64_t g_hi = uniform_load(a.group_offs + g + 1) >> (F4 ? 1 : 0);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
                run_slabs(static_cast<int>((g_hi - g_lo) / KSTEP));
                g_lo = g_hi;
                PT_GEMM_TRACE_POINT(4);
                if (g + 1 == cur_t.g1) {
                    // the re-read copies of the unit's last slab must have landed everywhere, and
                    // everyone must be done reading the stages, before the next unit's first copies go
                    // into them
                    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    // the next unit's first slabs travel while this unit's last result is written out
                    if (next_tile < total && nxt_t.KT > 0)
                        request_first_slabs(nxt_t);
                }
                if constexpr (MODE != SCALE_BLOCK)
                    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
                PT_GEMM_TRACE_POINT(5);
                uint8_t *Cg = cur_t.C + static_cast<int64_t>(g) * a.c_gstride * ES;
                // (the stores of a group's result are waited for at the next barrier here: leaving them in
                // flight, as the row-group mode does, measured no faster in this mode)
                epilogue<TM, TN, MODE, MODE != SCALE_BLOCK>(a, acc, Cg, cur_t.sA, cur_t.sB, cur_t.m_end, wm_base, wn_base, lane);
            }
            if (cur_t.g0 >= cur_t.g1 && next_tile < total && nxt_t.KT > 0)
                request_first_slabs(nxt_t); // (an empty chunk: nothing was in flight)
        }

        PT_GEMM_TRACE_POINT(6);
        if (next_tile >= total)
            break;
        tile  = next_tile;
        cur_t = nxt_t;
    }
    // no copy into this workgroup's LDS may still be in flight when the LDS is handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// GROUP_K: chunks of consecutive groups per output position: the smallest count (up to the group
// count) with which the units fill whole rounds of the grid to within 5 %, else the best found
constexpr int VK_MAX_CHUNKS = 16;
static inline int vk_pick_chunks(int64_t positions, int64_t grid, int64_t groups) {
    int           best     = 1;
    double        best_eff = 0.0;
    const int64_t cmax     = groups < VK_MAX_CHUNKS ? groups : VK_MAX_CHUNKS;
    for (int c = 1; c <= cmax; ++c) {
        const int64_t u   = positions * c;
        const double  eff = static_cast<double>(u) / static_cast<double>((u + grid - 1) / grid * grid);
        if (eff > best_eff + 1e-9) {
            best     = c;
            best_eff = eff;
        }
        if (eff >= 0.95)
            break;
    }
    return best;
}

// Upper bound on the number of tiles (exact for the ungrouped case): GROUP_ROWS cannot know
// the per-group row counts on the host, but every group adds at most one partial tile row.
template <int TM, int TN, int MODE, bool SB_VEC, int FA, int FB, int GMODE = GROUP_NONE>
static int launch_gemm_cfg(const GemmArgs &args_in, hipStream_t stream) {
    constexpr int BM = 2 * TM * 16, BN = 2 * TN * 16;
    constexpr int STAGES  = gemm_stages(TM, TN, FA == 4) * gemm_stage_bytes(TM, TN, MODE, FA == 4);
    // groups whose tile prefix sums fit into the LDS next to the stages
    constexpr int MAX_G   = (160 * 1024 - STAGES) / 4 - 2 < 2048 ? 1024 : 2048;
    constexpr int LDS_MAX = STAGES + (GMODE == GROUP_ROWS ? (MAX_G + 2) * 4 : GMODE == GROUP_K ? (VK_MAX_CHUNKS + 2) * 4 : 0);
    static_assert(LDS_MAX <= 160 * 1024, "tile configuration does not fit the LDS");
    GemmArgs a = args_in;
    a.gmode    = GMODE;
    a.tiles_m  = static_cast<int>(cdiv(a.M, BM));
    a.tiles_n  = static_cast<int>(cdiv(a.N, BN));
    if (GMODE != GROUP_NONE && a.G > MAX_G)
        return fail(PT_ERR_INVALID_ARGUMENT, "grouped gemm: too many groups for this tile configuration");
    if (MODE == SCALE_BLOCK && ((!SB_VEC && a.sb_shift != 7) || (GMODE == GROUP_ROWS && a.sa_shift != 0)))
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_fp8: unsupported block-scale layout");
    // MX scale words are fetched as aligned 32-bit units
    if (MODE == SCALE_MX && (a.sa_shift != 0 || a.sb_shift != 0 || (a.sa_wpitch == 0 && (a.sa_m % 4 != 0 || a.sb_n % 4 != 0)) ||
                             (a.sa_wpitch != 0) != (a.sb_wpitch != 0) || a.sa_wpitch % 4 != 0 || a.sb_wpitch % 4 != 0 ||
                             reinterpret_cast<uintptr_t>(a.sA) % 4 != 0 || reinterpret_cast<uintptr_t>(a.sB) % 4 != 0))
        return fail(PT_ERR_INVALID_ARGUMENT, "gemm_mx: scale rows must be 4-byte aligned");
    auto kern            = gemm_fp8_nt_kernel<TM, TN, MODE, SB_VEC, FA, FB, GMODE>;
    // the attribute belongs to the (kernel, device) pair: one bit per device, set once
    static std::atomic<unsigned long long> attr_set{0};
    int                                    dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return fail(PT_ERR_LAUNCH, "gemm_fp8: no current device (or a device index beyond 63)");
    const unsigned long long dev_bit = 1ULL << dev;
    if (!(attr_set.load(std::memory_order_acquire) & dev_bit)) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, LDS_MAX) != hipSuccess)
            return fail(PT_ERR_LAUNCH, "gemm_fp8: cannot raise the dynamic LDS limit");
        attr_set.fetch_or(dev_bit, std::memory_order_release);
    }
    const int lds = STAGES + (GMODE == GROUP_ROWS ? (a.G + 2) * 4 : GMODE == GROUP_K ? (VK_MAX_CHUNKS + 2) * 4 : 0);
    // persistent grid: as many workgroups as fit on the machine at once (LDS-limited)
    const int per_cu = (160 * 1024) / lds;
    int64_t   grid   = static_cast<int64_t>(device_cu_count()) * (per_cu < 1 ? 1 : per_cu);
    int64_t   total;
    if (GMODE == GROUP_ROWS) {
        total = (static_cast<int64_t>(a.tiles_m) + a.G) * a.tiles_n;
    } else if (GMODE == GROUP_K) {
        const int64_t positions = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
        a.vk_chunks             = vk_pick_chunks(positions, grid, a.G);
        total                   = positions * a.vk_chunks;
    } else {
        total = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
    }
    if (grid > total)
        grid = total;
    if (grid <= 0)
        return PT_OK;
    kern<<<static_cast<unsigned>(grid), 256, lds, stream>>>(a);
    return check_launch("gemm_fp8_nt_kernel");
}

// ---- host helpers shared by the translation units that instantiate the kernel ----
static inline int64_t round_up(int64_t x, int64_t m) {
    return (x + m - 1) / m * m;
}
// The kernel wants K as a multiple of 128 and at least GEMM_MIN_SLABS 128-byte slabs.
static inline int64_t padded_k(int64_t K) {
    const int64_t kp = round_up(K, KSTEP);
    return kp < GEMM_MIN_SLABS * KSTEP ? GEMM_MIN_SLABS * KSTEP : kp;
}
// in[batch][R, C] -> out[batch][C, ldo] (columns [R, ldo) zero-filled), fp8 bytes
void launch_transpose(const uint8_t *in, uint8_t *out, int64_t batch, int64_t R, int64_t C, int64_t ldo,
                      hipStream_t st);
// in[R, C] -> out[R, ldo] (columns [C, ldo) zero-filled)
void launch_pad_rows(const uint8_t *in, uint8_t *out, int64_t R, int64_t C, int64_t ldo, hipStream_t st);
// in[R, C] with row pitch ldi -> out[R, ldo] (columns [C, ldo) zero-filled)
void launch_pad_rows2(const uint8_t *in, uint8_t *out, int64_t R, int64_t C, int64_t ldi, int64_t ldo, hipStream_t st);
// out[b][w * R + r] = in[b][r * pitch + w] for w < W (32-bit words): scale arrays made contiguous along their rows
int launch_transpose_words(const uint32_t *in, uint32_t *out, int64_t R, int64_t W, int64_t pitch, hipStream_t st,
                            int64_t batch = 1);
int  launch_gemm_block(const GemmArgs &a, int fa, int fb, bool sb_vec, int tile_cfg, hipStream_t stream);

} // namespace pt
