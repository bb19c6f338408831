// FP8 128-blockwise quantizers (fp32 scales) for gfx950:
//   1 x 128 row blocks, 128 x 1 column blocks, both at once ("dual"),
//   128 x 128 weight tiles, and the fused grouped row + segment-padded column
//   quantizer that feeds the MoE grouped GEMM, plus their de-quantizers and the
//   group-offset prefix sums.
//
// Numerics (identical for every variant): per block
//   scale = qmax / max(amax, 1e-4), stored value = 1.0f / scale,
//   q = fp8_rne(clamp(float(x) * scale, -qmax, qmax)),
// following primus_turbo/triton/quantization/quant_blockwise.py:11-327 and
// csrc/kernels/quantization/quantization_blockwise.cu:18-346 of Primus-Turbo.
//
// One workgroup (256 threads, 4 wavefronts) owns one 128 x 128 tile and reads it
// from HBM once; all requested outputs come from the register copy. A tile row is
// spread over the 16 lanes of one DPP row, so the 1 x 128 amax is four DPP steps;
// column maxima meet through 8 KB of LDS.
#include "pt_activation.h"

namespace pt {

constexpr int BQ        = 128; // block edge
constexpr int BQ_PACK   = 8;   // elements per thread per row visit
constexpr int BQ_ROUNDS = 8;   // 16 rows per round x 8 rounds = 128 rows
constexpr float BQ_EPS  = 1e-4f;

enum : int { MODE_ROW = 1, MODE_COL = 2, MODE_TILE = 4 };

struct BlockQuantArgs {
    const void *x;
    uint8_t    *q_row;     // MODE_ROW / MODE_TILE output codes
    float      *s_row;     // MODE_ROW: 1/scale per (row, n-block); MODE_TILE: per tile
    uint8_t    *q_col;     // MODE_COL output codes
    float      *s_col;     // MODE_COL: 1/scale per (m-block, col)
    int64_t     M, N;      // rows / cols of one batch slice of x
    int64_t     rs_m, rs_n; // s_row index = m * rs_m + nblock * rs_n
    // grouped (segment-padded) mode
    const int64_t *group_offs;  // [G+1] row offsets of the groups in x
    const int64_t *padded_offs; // [G+1] offsets with every group rounded up to 128 rows
    int            num_groups;
    float          qmax;
    // optional transposed copy of the tile codes (MODE_TILE: [B, N, ldt]) or of the column
    // codes (MODE_COL: [N, ldt]): the operand a GEMM reads when it reduces over the rows of x
    uint8_t *q_t;
    int64_t  ldt;
    // gated-activation input (grouped row + column mode): x is [M, 2 N], gate columns first, and
    // the tile quantized is T(act(gate) * up * probs[row]), zero where row_mask[row] == 0
    const float   *probs;
    const int64_t *row_mask;
};

// Eight consecutive elements of a tile row as they come from memory (16-bit inputs stay packed:
// four registers instead of eight between the phases of the kernel).
template <typename T> struct Held8 {
    static constexpr int WORDS = sizeof(T) == 4 ? 8 : 4;
    uint32_t             w[WORDS];
    template <bool STREAM = false> __device__ __forceinline__ void load(const T *p) {
        const u32x4 a = STREAM ? ld128_nt(p) : ld128(p);
        w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w;
        if constexpr (sizeof(T) == 4) {
            const u32x4 b = STREAM ? ld128_nt(p + 4) : ld128(p + 4);
            w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
        }
    }
    // element by element, zeros where `ok` says so (tile edges, rows of other groups)
    template <typename OK> __device__ __forceinline__ void load_checked(const T *p, OK ok) {
        uint32_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            e[i] = 0;
            if (ok(i)) {
                if constexpr (sizeof(T) == 4) {
                    e[i] = __float_as_uint(p[i]);
                } else {
                    uint16_t b;
                    __builtin_memcpy(&b, p + i, 2);
                    e[i] = b;
                }
            }
        }
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                w[i] = e[i];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = e[2 * i] | (e[2 * i + 1] << 16);
        }
    }
    __device__ __forceinline__ void get(float (&f)[8]) const {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                f[i] = __uint_as_float(w[i]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                unpack2<T>(w[i], f[2 * i], f[2 * i + 1]);
        }
    }
};

template <bool E5M2>
__device__ __forceinline__ u32x2 quant8(const float (&f)[8], const float (&s)[8], float qmax) {
    u32x2 o;
    o.x = cvt4_fp8<E5M2>(scale_clamp(f[0], s[0], qmax), scale_clamp(f[1], s[1], qmax),
                         scale_clamp(f[2], s[2], qmax), scale_clamp(f[3], s[3], qmax));
    o.y = cvt4_fp8<E5M2>(scale_clamp(f[4], s[4], qmax), scale_clamp(f[5], s[5], qmax),
                         scale_clamp(f[6], s[6], qmax), scale_clamp(f[7], s[7], qmax));
    return o;
}

// STREAM: a whole piece leaves as a non-temporal store
template <bool STREAM> __device__ __forceinline__ void store8(uint8_t *p, u32x2 v, bool vec, int64_t gn, int64_t N) {
    if (vec) {
        if constexpr (STREAM)
            st64_nt(p, v);
        else
            *reinterpret_cast<u32x2 *>(p) = v;
    } else {
        const uint32_t w[2] = {v.x, v.y};
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (gn + i < N)
                p[i] = static_cast<uint8_t>((w[i >> 2] >> (8 * (i & 3))) & 0xffu);
    }
}

// Row of the tile that round r of thread row slot `rslot` handles: a thread owns two runs of four
// consecutive rows, so that it can transpose its 4 x 4 byte blocks in registers.
__device__ __forceinline__ int tile_row_of(int rslot, int r) {
    return 4 * rslot + (r & 3) + 64 * (r >> 2);
}

constexpr int BQ_TP = 33; // words per row of the transposed LDS tile

// Codes of four consecutive tile rows x eight columns (one u32x2 per row) -> eight words "four
// rows of one column" in the transposed tile t[column][BQ_TP], word index = row / 4.
__device__ __forceinline__ void stage_transposed(uint32_t *t, const u32x2 (&c)[4], int cseg, int rowgroup) {
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        const uint32_t a0 = w ? c[0].y : c[0].x, a1 = w ? c[1].y : c[1].x, a2 = w ? c[2].y : c[2].x,
                       a3 = w ? c[3].y : c[3].x;
        const uint32_t t0 = __builtin_amdgcn_perm(a1, a0, 0x05010400u);
        const uint32_t t1 = __builtin_amdgcn_perm(a1, a0, 0x07030602u);
        const uint32_t t2 = __builtin_amdgcn_perm(a3, a2, 0x05010400u);
        const uint32_t t3 = __builtin_amdgcn_perm(a3, a2, 0x07030602u);
        const int      col = cseg * 8 + w * 4;
        t[(col + 0) * BQ_TP + rowgroup] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
        t[(col + 1) * BQ_TP + rowgroup] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
        t[(col + 2) * BQ_TP + rowgroup] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
        t[(col + 3) * BQ_TP + rowgroup] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
    }
}

// The staged tile leaves as rows of the transposed output: out[(c0 + c) * ldt + m0 + 0..127] for
// the columns c0 + c < cols; 16-byte chunks beyond `rows` (a multiple of 16) are not written.
__device__ __forceinline__ void flush_transposed(const uint32_t *t, uint8_t *out, int64_t ldt, int64_t c0, int64_t cols,
                                                 int64_t m0, int64_t rows, int tid) {
    const int j = tid & 7;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     c  = (tid >> 3) + 32 * p;
        const int64_t gm = m0 + j * 16;
        if (c0 + c < cols && gm < rows) {
            u32x4 v;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                v[k] = t[c * BQ_TP + j * 4 + k];
            *reinterpret_cast<u32x4 *>(out + (c0 + c) * ldt + gm) = v;
        }
    }
}

// MODE: bitmask of MODE_ROW / MODE_COL / MODE_TILE.  GROUPED: tiles live in the
// segment-padded row space and map back to input rows through the group offsets.
// VEC8: N % 8 == 0 and all pointers 16-byte aligned (128-bit loads, 64-bit stores).
// TRANS: also emit the transposed copy described at BlockQuantArgs::q_t.
// GLU: 0 = x is the tile source itself; 1 + ACT_SILU / 1 + ACT_GELU = x holds gate and up halves
// and the gated activation (rounded to T, as the stand-alone activation kernel stores it) is what
// gets quantized, so that the activation never travels through HBM.
template <typename T, bool E5M2, int MODE, bool GROUPED, bool VEC8, bool TRANS = false, int GLU = 0>
__device__ __forceinline__ void quant_block128_tile(const BlockQuantArgs &a) {
    static_assert(!TRANS || ((MODE & MODE_TILE) != 0) != ((MODE & MODE_COL) != 0), "one transposed output");
    static_assert(GLU == 0 || (GROUPED && sizeof(T) == 2), "the gated input belongs to the grouped 16-bit quantizer");
    __shared__ uint32_t s_tr[TRANS ? BQ * BQ_TP : 1];
    // The input is read once and nobody reads the row output soon: non-temporal loads and row
    // stores (weight quantizer, 32 x 4096 x 7168: 0.506 -> 0.459 ms, with the transposed copy
    // 0.707 -> 0.656 ms; row + column outputs of 16384 x 7168: 98 -> 90 us). The transposed and
    // column outputs keep plain stores: with the hint they are slower (92 us).
    const int     tid   = threadIdx.x;
    const int     cseg  = tid & 15; // which 8-column segment of the tile row
    const int     rslot = tid >> 4; // row within a round
    uint32_t tile_x, tile_y; // (tile order: blocks of 8 x 8 tiles per XCD, see xcd_block_tile)
    xcd_block_tile(tile_x, tile_y);
    const int64_t tn = tile_x, tm = tile_y, batch = blockIdx.z;
    const int64_t M = a.M, N = a.N;
    const float   qmax = a.qmax;

    const T *x     = static_cast<const T *>(a.x) + batch * M * N;
    int64_t  in_m0 = tm * BQ; // input row of tile row 0
    int64_t  in_end = M;      // first invalid input row
    int64_t  M_out  = M;      // rows of the (padded) column output that exist
    if constexpr (GROUPED) {
        M_out = a.padded_offs[a.num_groups];
        const int64_t pad_start_tile = tm * BQ;
        if (pad_start_tile >= M_out)
            return;
        const int g = find_group(a.padded_offs, a.num_groups, pad_start_tile);
        const int64_t o0 = a.group_offs[g], o1 = a.group_offs[g + 1];
        in_m0  = o0 + (pad_start_tile - a.padded_offs[g]);
        in_end = o1 < M ? o1 : M;
    }

    const int64_t gn   = tn * BQ + cseg * BQ_PACK;
    const bool    full = VEC8 && (gn + BQ_PACK <= N);

    // phase 1: the whole tile share of this thread is requested before anything is used. With
    // whole 16-byte pieces no branch may separate the loads (the compiler would wait for each one
    // in turn): a piece outside the matrix reads the matrix's first bytes and is zeroed afterwards.
    Held8<T> held[BQ_ROUNDS];
    if constexpr (GLU == 0) {
        if constexpr (VEC8) {
            bool ok[BQ_ROUNDS];
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r) {
                const int64_t in_m = in_m0 + tile_row_of(rslot, r);
                ok[r]              = in_m < in_end && gn < N;
                held[r].template load<true>(x + (ok[r] ? in_m * N + gn : 0));
            }
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r)
#pragma unroll
                for (int i = 0; i < Held8<T>::WORDS; ++i)
                    held[r].w[i] = ok[r] ? held[r].w[i] : 0u;
        } else {
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r) {
                const int64_t in_m  = in_m0 + tile_row_of(rslot, r);
                const bool    valid = in_m < in_end;
                held[r].load_checked(x + in_m * N + gn, [&](int i) { return valid && gn + i < N; });
            }
        }
    } else {
        Held8<T> up[BQ_ROUNDS];
        float    pr[BQ_ROUNDS];
        bool     live[BQ_ROUNDS]; // the row exists and is not masked out
        if constexpr (VEC8) {
            int64_t ms[BQ_ROUNDS];
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r) {
                const int64_t in_m = in_m0 + tile_row_of(rslot, r);
                live[r]            = in_m < in_end;
                const bool ok      = live[r] && gn < N;
                ms[r]              = live[r] ? in_m : 0;
                const T *g         = x + (ok ? in_m * 2 * N + gn : 0);
                held[r].template load<true>(g);
                up[r].template load<true>(g + N);
                pr[r] = a.probs[ms[r]];
            }
            if (a.row_mask != nullptr) {
                int64_t keep[BQ_ROUNDS];
#pragma unroll
                for (int r = 0; r < BQ_ROUNDS; ++r)
                    keep[r] = a.row_mask[ms[r]];
#pragma unroll
                for (int r = 0; r < BQ_ROUNDS; ++r)
                    live[r] = live[r] && keep[r] != 0;
            }
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r)
                live[r] = live[r] && gn < N;
        } else {
#pragma unroll
            for (int r = 0; r < BQ_ROUNDS; ++r) {
                const int64_t in_m  = in_m0 + tile_row_of(rslot, r);
                const bool    valid = in_m < in_end;
                const T      *g     = x + in_m * 2 * N + gn;
                held[r].load_checked(g, [&](int i) { return valid && gn + i < N; });
                up[r].load_checked(g + N, [&](int i) { return valid && gn + i < N; });
                live[r] = valid && (a.row_mask == nullptr || a.row_mask[in_m] != 0);
                pr[r]   = live[r] ? a.probs[in_m] : 0.f;
            }
        }
#pragma unroll
        for (int r = 0; r < BQ_ROUNDS; ++r) {
            float fg[8], fu[8];
            held[r].get(fg);
            up[r].get(fu);
#pragma unroll
            for (int i = 0; i < 8; ++i) // (padding columns hold zeros: act(0) * 0 = 0)
                fg[i] = live[r] ? act_fwd<GLU - 1>(fg[i]) * fu[i] * pr[r] : 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                held[r].w[i] = pack2<T>(fg[2 * i], fg[2 * i + 1]);
        }
    }

    float col_amax[BQ_PACK];
    float tile_amax = 0.f;
#pragma unroll
    for (int i = 0; i < BQ_PACK; ++i)
        col_amax[i] = 0.f;

#pragma unroll
    for (int r = 0; r < BQ_ROUNDS; ++r) {
        const int     lm    = tile_row_of(rslot, r);
        const int64_t in_m  = in_m0 + lm;
        const bool    valid = in_m < in_end;
        float         vals[BQ_PACK];
        held[r].get(vals);
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < BQ_PACK; ++i) {
            const float av = fabsf(vals[i]);
            amax           = fmaxf(amax, av);
            if constexpr (MODE & MODE_COL)
                col_amax[i] = fmaxf(col_amax[i], av);
        }
        if constexpr (MODE & MODE_TILE)
            tile_amax = fmaxf(tile_amax, amax);
        if constexpr (MODE & MODE_ROW) {
            amax              = row16_max(amax); // the 16 lanes of this tile row
            const float scale = qmax / fmaxf(amax, BQ_EPS);
            if (valid) {
                const float s[8] = {scale, scale, scale, scale, scale, scale, scale, scale};
                store8<true>(a.q_row + batch * M * N + in_m * N + gn, quant8<E5M2>(vals, s, qmax), full, gn, N);
                if (cseg == 0)
                    a.s_row[in_m * a.rs_m + tn * a.rs_n] = 1.0f / scale;
            }
        }
    }

    if constexpr (MODE & MODE_TILE) {
        __shared__ float s_red[4];
        tile_amax         = block_max(tile_amax, s_red);
        const float scale = qmax / fmaxf(tile_amax, BQ_EPS);
        if (tid == 0)
            a.s_row[(batch * gridDim.y + tm) * gridDim.x + tn] = 1.0f / scale;
        const float s[8] = {scale, scale, scale, scale, scale, scale, scale, scale};
        [[maybe_unused]] u32x2 code4[4];
#pragma unroll
        for (int r = 0; r < BQ_ROUNDS; ++r) {
            const int64_t in_m = in_m0 + tile_row_of(rslot, r);
            float         vals[BQ_PACK];
            held[r].get(vals);
            const u32x2 code = quant8<E5M2>(vals, s, qmax); // rows beyond the matrix hold zeros: code 0
            if (in_m < in_end)
                store8<true>(a.q_row + batch * M * N + in_m * N + gn, code, full, gn, N);
            if constexpr (TRANS) {
                code4[r & 3] = code;
                if ((r & 3) == 3)
                    stage_transposed(s_tr, code4, cseg, rslot + 16 * (r >> 2));
            }
        }
        if constexpr (TRANS) {
            __syncthreads();
            flush_transposed(s_tr, a.q_t + batch * N * a.ldt, a.ldt, tn * BQ, N, tm * BQ, M, tid);
        }
    }

    if constexpr (MODE & MODE_COL) {
        __shared__ float s_part[16][BQ];
        __shared__ float s_cscale[BQ];
#pragma unroll
        for (int i = 0; i < BQ_PACK; ++i)
            s_part[rslot][cseg * BQ_PACK + i] = col_amax[i];
        __syncthreads();
        if (tid < BQ) {
            float m = 0.f;
#pragma unroll
            for (int k = 0; k < 16; ++k)
                m = fmaxf(m, s_part[k][tid]);
            const float scale = qmax / fmaxf(m, BQ_EPS);
            s_cscale[tid]     = scale;
            const int64_t c   = tn * BQ + tid;
            if (c < N)
                a.s_col[tm * N + c] = 1.0f / scale;
        }
        __syncthreads();
        float s[8];
#pragma unroll
        for (int i = 0; i < BQ_PACK; ++i)
            s[i] = s_cscale[cseg * BQ_PACK + i];
        [[maybe_unused]] u32x2 code4[4];
#pragma unroll
        for (int r = 0; r < BQ_ROUNDS; ++r) {
            const int64_t out_m = tm * BQ + tile_row_of(rslot, r);
            float         vals[BQ_PACK];
            held[r].get(vals);
            const u32x2 code = quant8<E5M2>(vals, s, qmax); // grouped: pad rows carry zeros -> code 0
            if (a.q_col != nullptr && out_m < M_out)
                store8<false>(a.q_col + out_m * N + gn, code, full, gn, N);
            if constexpr (TRANS) {
                code4[r & 3] = code;
                if ((r & 3) == 3)
                    stage_transposed(s_tr, code4, cseg, rslot + 16 * (r >> 2));
            }
        }
        if constexpr (TRANS) {
            __syncthreads();
            flush_transposed(s_tr, a.q_t, a.ldt, tn * BQ, N, tm * BQ, a.ldt, tid);
        }
    }
}

// Row blocks alone, rows of whole 16-byte pieces: a stream without LDS, same bytes as the tile
// kernel. A workgroup takes 16 rows of four neighbouring 128-column blocks, a wavefront four of
// those rows (runs of 1 KB): 16 lanes quantize one row of one block, a load covers one block of
// the four rows, and all four loads of a lane are requested before the first is used. The 16
// scales of a wavefront leave as 16 bytes per row (row-major scales, [M, N / 128]) or as 16 bytes
// per block (block-major scales, [N / 128, M]).
template <typename T, bool E5M2>
__global__ __launch_bounds__(256) void quant_rows128_kernel(const BlockQuantArgs a, const int64_t col_groups) {
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int     cseg = lane & 15, g = lane >> 4;
    const int64_t cg = blockIdx.x % col_groups, rg = blockIdx.x / col_groups;
    const bool    block_major = a.rs_n != 1;
    const T      *x = static_cast<const T *>(a.x);
    Held8<T>      held[4];
    bool          ok[4];
    int64_t       row[4], tn[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        row[k]           = rg * 16 + 4 * wave + g;
        tn[k]            = cg * 4 + k;
        const int64_t gn = tn[k] * BQ + cseg * BQ_PACK;
        ok[k]            = gn < a.N && row[k] < a.M; // (N is a multiple of 8: a piece is inside or outside as a whole)
        held[k].template load<true>(x + (ok[k] ? row[k] * a.N + gn : 0));
    }
    float inv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        float vals[BQ_PACK];
        held[k].get(vals);
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < BQ_PACK; ++i) {
            vals[i] = ok[k] ? vals[i] : 0.f;
            amax    = fmaxf(amax, fabsf(vals[i]));
        }
        amax              = row16_max(amax); // the 16 lanes of this row's block
        const float scale = a.qmax / fmaxf(amax, BQ_EPS);
        inv[k]            = 1.0f / scale;
        if (ok[k]) {
            const float s[8] = {scale, scale, scale, scale, scale, scale, scale, scale};
            st64_nt(a.q_row + row[k] * a.N + tn[k] * BQ + cseg * BQ_PACK, quant8<E5M2>(vals, s, a.qmax));
        }
    }
    if (block_major) {
        // lane L < 16 writes the scale of block L >> 2 and row L & 3, which the lanes 16 (L & 3) .. hold
        float mine = 0.f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float v = __shfl(inv[k], 16 * (lane & 3), 64);
            mine          = (lane >> 2) == k ? v : mine;
        }
        const int64_t r = rg * 16 + 4 * wave + (lane & 3), t = cg * 4 + (lane >> 2);
        if (lane < 16 && r < a.M && t * BQ < a.N)
            a.s_row[r * a.rs_m + t * a.rs_n] = mine;
    } else if (cseg == 0 && row[0] < a.M) {
        float *p = a.s_row + row[0] * a.rs_m + tn[0];
        if ((tn[3] + 1) * BQ - BQ < a.N && (reinterpret_cast<uintptr_t>(p) & 15) == 0) {
            st128(p, u32x4{__float_as_uint(inv[0]), __float_as_uint(inv[1]), __float_as_uint(inv[2]), __float_as_uint(inv[3])});
        } else {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (tn[k] * BQ < a.N)
                    p[k] = inv[k];
        }
    }
}

template <typename T, bool E5M2, int MODE, bool GROUPED, bool VEC8, bool TRANS = false, int GLU = 0>
__global__ __launch_bounds__(256) void quant_block128_kernel(const BlockQuantArgs a) {
    quant_block128_tile<T, E5M2, MODE, GROUPED, VEC8, TRANS, GLU>(a);
}
// The same tile with the registers capped for four workgroups per CU (the compiler takes 155 when
// left alone, three workgroups). Measured per form: the grouped row + column quantizer without the
// transposed copy gains (32768 x 7168: 188 -> 173 us), with the copy it makes no difference (146
// against 147 us), the dense row + column form loses (91 -> 95 us) and so does the gated one
// (93 -> 100 us): only the first is launched this way.
template <typename T, bool E5M2, int MODE, bool VEC8>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void quant_block128_occ4_kernel(const BlockQuantArgs a) {
    quant_block128_tile<T, E5M2, MODE, true, VEC8, false, 0>(a);
}

template <typename T, bool E5M2, int MODE, bool GROUPED, int GLU = 0>
static int launch_block128(const BlockQuantArgs &a, int64_t tiles_m, int64_t tiles_n, int64_t batch,
                           bool vec, hipStream_t stream) {
    if (tiles_m * tiles_n * batch == 0)
        return PT_OK;
    dim3 g(static_cast<unsigned>(tiles_n), static_cast<unsigned>(tiles_m),
           static_cast<unsigned>(batch));
    if constexpr (GLU != 0) {
        if (a.q_t != nullptr) {
            if (vec)
                quant_block128_kernel<T, E5M2, MODE, GROUPED, true, true, GLU><<<g, 256, 0, stream>>>(a);
            else
                quant_block128_kernel<T, E5M2, MODE, GROUPED, false, true, GLU><<<g, 256, 0, stream>>>(a);
        } else {
            if (vec)
                quant_block128_kernel<T, E5M2, MODE, GROUPED, true, false, GLU><<<g, 256, 0, stream>>>(a);
            else
                quant_block128_kernel<T, E5M2, MODE, GROUPED, false, false, GLU><<<g, 256, 0, stream>>>(a);
        }
        return check_launch("quant_block128_kernel");
    }
    if constexpr (MODE == MODE_TILE || MODE == (MODE_ROW | MODE_COL)) {
        if (a.q_t != nullptr) {
            if (vec)
                quant_block128_kernel<T, E5M2, MODE, GROUPED, true, true><<<g, 256, 0, stream>>>(a);
            else
                quant_block128_kernel<T, E5M2, MODE, GROUPED, false, true><<<g, 256, 0, stream>>>(a);
            return check_launch("quant_block128_kernel");
        }
    }
    if constexpr (GROUPED && MODE == (MODE_ROW | MODE_COL)) {
        if (vec)
            quant_block128_occ4_kernel<T, E5M2, MODE, true><<<g, 256, 0, stream>>>(a);
        else
            quant_block128_occ4_kernel<T, E5M2, MODE, false><<<g, 256, 0, stream>>>(a);
        return check_launch("quant_block128_kernel");
    }
    if (vec)
        quant_block128_kernel<T, E5M2, MODE, GROUPED, true><<<g, 256, 0, stream>>>(a);
    else
        quant_block128_kernel<T, E5M2, MODE, GROUPED, false><<<g, 256, 0, stream>>>(a);
    return check_launch("quant_block128_kernel");
}

// ---------------------------------------------------------------------------
// De-quantize with one fp32 scale per (bm x bn) block:
//   y[b, m, n] = T(float(q[b, m, n]) * s[b, m / bm, n / bn])
// (bm, bn) = (1, 128) row blocks, (128, 1) column blocks, (128, 128) tiles.
// ---------------------------------------------------------------------------
template <typename T, bool E5M2>
__global__ __launch_bounds__(256) void dequant_block_kernel(
    const uint8_t *__restrict__ q, const float *__restrict__ s, T *__restrict__ y, const int64_t B,
    const int64_t M, const int64_t N, const int bm, const int bn) {
    const int64_t sm = (M + bm - 1) / bm, sn = (N + bn - 1) / bn;
    const int64_t total  = B * M * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += stride) {
        const int64_t n = i % N, m = (i / N) % M, b = i / (M * N);
        const float   sc = s[(b * sm + m / bm) * sn + n / bn];
        y[i]             = HP<T>::from_f32(fp8_to_f32<E5M2>(q[i], 0) * sc);
    }
}

// 16 consecutive columns per thread; requires N % 16 == 0 and 16-byte aligned q / y.
template <typename T, bool E5M2, bool PER_COL>
__global__ __launch_bounds__(256) void dequant_block_vec_kernel(
    const uint8_t *__restrict__ q, const float *__restrict__ s, T *__restrict__ y, const int64_t B,
    const int64_t M, const int64_t N, const int bm, const int bn) {
    const int64_t sm = (M + bm - 1) / bm, sn = (N + bn - 1) / bn;
    const int64_t units  = B * M * N / 16;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t u = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; u < units;
         u += stride) {
        const int64_t  i = u * 16;
        const int64_t  n = i % N, m = (i / N) % M, b = i / (M * N);
        const u32x4    w = ld128_nt(q + i);
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
        float          f[16];
        if constexpr (PER_COL) { // bn == 1: sixteen different scales
            const float *sp = s + (b * sm + m / bm) * sn + n;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                f[4 * k + 0] = fp8_to_f32<E5M2>(ww[k], 0) * sp[4 * k + 0];
                f[4 * k + 1] = fp8_to_f32<E5M2>(ww[k], 1) * sp[4 * k + 1];
                f[4 * k + 2] = fp8_to_f32<E5M2>(ww[k], 2) * sp[4 * k + 2];
                f[4 * k + 3] = fp8_to_f32<E5M2>(ww[k], 3) * sp[4 * k + 3];
            }
        } else { // bn == 128: one scale for the 16 columns
            const float sc = s[(b * sm + m / bm) * sn + n / bn];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                f[4 * k + 0] = fp8_to_f32<E5M2>(ww[k], 0) * sc;
                f[4 * k + 1] = fp8_to_f32<E5M2>(ww[k], 1) * sc;
                f[4 * k + 2] = fp8_to_f32<E5M2>(ww[k], 2) * sc;
                f[4 * k + 3] = fp8_to_f32<E5M2>(ww[k], 3) * sc;
            }
        }
        char *dst = reinterpret_cast<char *>(y + i);
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                st128_nt(dst + 16 * k,
                      u32x4{__float_as_uint(f[4 * k]), __float_as_uint(f[4 * k + 1]),
                            __float_as_uint(f[4 * k + 2]), __float_as_uint(f[4 * k + 3])});
        } else {
#pragma unroll
            for (int k = 0; k < 2; ++k)
                st128_nt(dst + 16 * k,
                      u32x4{pack2<T>(f[8 * k], f[8 * k + 1]), pack2<T>(f[8 * k + 2], f[8 * k + 3]),
                            pack2<T>(f[8 * k + 4], f[8 * k + 5]),
                            pack2<T>(f[8 * k + 6], f[8 * k + 7])});
        }
    }
}

// ---------------------------------------------------------------------------
// Group offsets: offs[0] = 0, offs[i+1] = offs[i] + round_up(lens[i], align).
// One wavefront; each lane owns a strided slice, partial sums meet in LDS.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void group_offs_kernel(const int64_t *__restrict__ lens,
                                                        int64_t *__restrict__ padded_lens,
                                                        int64_t *__restrict__ offs, const int G,
                                                        const int64_t align) {
    __shared__ int64_t s_sum[64];
    const int          lane  = threadIdx.x;
    const int          chunk = (G + 63) / 64;
    const int          i0 = lane * chunk, i1 = (i0 + chunk < G) ? i0 + chunk : G;
    int64_t            sum = 0;
    for (int i = i0; i < i1; ++i)
        sum += (lens[i] + align - 1) / align * align;
    s_sum[lane] = sum;
    __syncthreads();
    int64_t base = 0;
    for (int k = 0; k < lane; ++k)
        base += s_sum[k];
    if (lane == 0)
        offs[0] = 0;
    for (int i = i0; i < i1; ++i) {
        const int64_t p = (lens[i] + align - 1) / align * align;
        if (padded_lens)
            padded_lens[i] = p;
        base += p;
        offs[i + 1] = base;
    }
}

#define PT_DISPATCH_T_E5(hp, fp8, CALL)                                                            \
    do {                                                                                           \
        if (hp == PT_DTYPE_BF16 && fp8 == PT_DTYPE_E4M3) { CALL(bf16_t, false); }                  \
        else if (hp == PT_DTYPE_BF16 && fp8 == PT_DTYPE_E5M2) { CALL(bf16_t, true); }              \
        else if (hp == PT_DTYPE_F16 && fp8 == PT_DTYPE_E4M3) { CALL(f16_t, false); }               \
        else if (hp == PT_DTYPE_F16 && fp8 == PT_DTYPE_E5M2) { CALL(f16_t, true); }                \
        else if (hp == PT_DTYPE_F32 && fp8 == PT_DTYPE_E4M3) { CALL(float, false); }               \
        else { CALL(float, true); }                                                                \
    } while (0)

static bool vec_ok(const BlockQuantArgs &a, int elem_bytes) {
    return a.N % 8 == 0 && aligned_to(a.x, 16) && (a.q_row == nullptr || aligned_to(a.q_row, 8)) &&
           (a.q_col == nullptr || aligned_to(a.q_col, 8)) && elem_bytes > 0;
}

} // namespace pt

using namespace pt;

extern "C" {

static int quantize_blocks(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, void *q_row,
                           float *scale_inv_row, void *q_col, void *q_col_t, int64_t ldt, float *scale_inv_col,
                           void *stream, bool row_scales_kmajor = false) {
    PT_REQUIRE(is_hp_dtype(x_dtype), "input must be bf16, fp16 or fp32");
    PT_REQUIRE(is_fp8_dtype(q_dtype), "output must be e4m3 or e5m2");
    PT_REQUIRE(M >= 0 && N >= 0, "dimensions must be non-negative");
    const bool row = q_row != nullptr, col = q_col != nullptr || q_col_t != nullptr;
    PT_REQUIRE(row || col, "at least one of q_row / q_col must be given");
    PT_REQUIRE(!row || scale_inv_row, "scale_inv_row must accompany q_row");
    PT_REQUIRE(!col || scale_inv_col, "scale_inv_col must accompany q_col");
    if (M * N == 0)
        return PT_OK;
    PT_REQUIRE(x != nullptr, "x must not be NULL");
    const int64_t tm = cdiv(M, BQ), tn = cdiv(N, BQ);
    PT_REQUIRE(tm < 65536, "too many row tiles");
    if (q_col_t != nullptr)
        PT_REQUIRE(row && ldt == tm * BQ && aligned_to(q_col_t, 16),
                   "the transposed column output comes with the row output, at a 16-byte aligned pitch of M rounded up to 128");
    BlockQuantArgs a{};
    a.x = x;
    a.q_row = static_cast<uint8_t *>(q_row);
    a.s_row = scale_inv_row;
    a.q_col = static_cast<uint8_t *>(q_col);
    a.s_col = scale_inv_col;
    a.q_t = static_cast<uint8_t *>(q_col_t);
    a.ldt = ldt;
    a.M = M;
    a.N = N;
    a.rs_m = row_scales_kmajor ? 1 : tn; // [M, N / 128], or block-major [N / 128, M]
    a.rs_n = row_scales_kmajor ? M : 1;
    a.qmax = fp8_max_of(q_dtype);
    auto       st  = static_cast<hipStream_t>(stream);
    const bool vec = vec_ok(a, 1);
    if (row && !col && vec) {
        const int64_t col_groups = cdiv(tn, 4), row_groups = cdiv(M, 16);
        PT_REQUIRE(col_groups * row_groups < (1LL << 31), "too many blocks");
        const dim3 grid(static_cast<unsigned>(col_groups * row_groups));
#define CALL(T, E5)                                                                                \
    do {                                                                                           \
        quant_rows128_kernel<T, E5><<<grid, 256, 0, st>>>(a, col_groups);                          \
        return check_launch("quant_rows128_kernel");                                               \
    } while (0)
        PT_DISPATCH_T_E5(x_dtype, q_dtype, CALL);
#undef CALL
    }
#define CALL(T, E5)                                                                                \
    do {                                                                                           \
        if (row && col)                                                                            \
            return launch_block128<T, E5, MODE_ROW | MODE_COL, false>(a, tm, tn, 1, vec, st);      \
        if (row)                                                                                   \
            return launch_block128<T, E5, MODE_ROW, false>(a, tm, tn, 1, vec, st);                 \
        return launch_block128<T, E5, MODE_COL, false>(a, tm, tn, 1, vec, st);                     \
    } while (0)
    PT_DISPATCH_T_E5(x_dtype, q_dtype, CALL);
#undef CALL
}

int pt_quantize_fp8_blockwise(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                              void *q_row, float *scale_inv_row, void *q_col, float *scale_inv_col,
                              void *stream) {
    return quantize_blocks(x, x_dtype, M, N, q_dtype, q_row, scale_inv_row, q_col, nullptr, 0, scale_inv_col, stream);
}

int pt_quantize_fp8_blockwise_t(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, void *q_row,
                                float *scale_inv_row, void *q_col, void *q_col_t, int64_t ldt, float *scale_inv_col,
                                void *stream) {
    PT_REQUIRE(q_col_t != nullptr || M * N == 0, "q_col_t must not be NULL");
    return quantize_blocks(x, x_dtype, M, N, q_dtype, q_row, scale_inv_row, q_col, q_col_t, ldt, scale_inv_col, stream);
}

int pt_quantize_fp8_blockwise_kmajor(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, void *q_row,
                                     float *scale_inv_row_kmajor, void *q_col_t, int64_t ldt, float *scale_inv_col,
                                     void *stream) {
    PT_REQUIRE(q_row != nullptr || M * N == 0, "q_row must not be NULL");
    return quantize_blocks(x, x_dtype, M, N, q_dtype, q_row, scale_inv_row_kmajor, nullptr, q_col_t, ldt, scale_inv_col, stream,
                           true);
}

static int quantize_weight_tiles(const void *w, int w_dtype, int64_t B, int64_t M, int64_t N, void *q, void *q_t,
                                 int64_t ldt, int q_dtype, float *scale_inv, void *stream) {
    PT_REQUIRE(is_hp_dtype(w_dtype), "input must be bf16, fp16 or fp32");
    PT_REQUIRE(is_fp8_dtype(q_dtype), "output must be e4m3 or e5m2");
    PT_REQUIRE(B >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    if (B * M * N == 0)
        return PT_OK;
    PT_REQUIRE(w && q && scale_inv, "NULL tensor pointer");
    if (q_t != nullptr)
        PT_REQUIRE(M % 16 == 0 && ldt >= M && ldt % 16 == 0 && aligned_to(q_t, 16),
                   "the transposed output needs M % 16 == 0 and a 16-byte aligned pitch >= M");
    const int64_t tm = cdiv(M, BQ), tn = cdiv(N, BQ);
    PT_REQUIRE(tm < 65536 && B < 65536, "too many tiles / batches");
    BlockQuantArgs a{};
    a.x = w;
    a.q_row = static_cast<uint8_t *>(q);
    a.s_row = scale_inv;
    a.q_t = static_cast<uint8_t *>(q_t);
    a.ldt = ldt;
    a.M = M;
    a.N = N;
    a.qmax = fp8_max_of(q_dtype);
    auto       st  = static_cast<hipStream_t>(stream);
    const bool vec = vec_ok(a, 1) && (M * N) % 8 == 0;
#define CALL(T, E5) return launch_block128<T, E5, MODE_TILE, false>(a, tm, tn, B, vec, st)
    PT_DISPATCH_T_E5(w_dtype, q_dtype, CALL);
#undef CALL
}

int pt_quantize_fp8_blockwise_weight(const void *w, int w_dtype, int64_t B, int64_t M, int64_t N,
                                     void *q, int q_dtype, float *scale_inv, void *stream) {
    return quantize_weight_tiles(w, w_dtype, B, M, N, q, nullptr, 0, q_dtype, scale_inv, stream);
}

int pt_quantize_fp8_blockwise_weight_dual(const void *w, int w_dtype, int64_t B, int64_t M, int64_t N, void *q,
                                          void *q_t, int64_t ldt, int q_dtype, float *scale_inv, void *stream) {
    PT_REQUIRE(q_t != nullptr || B * M * N == 0, "q_t must not be NULL");
    return quantize_weight_tiles(w, w_dtype, B, M, N, q, q_t, ldt, q_dtype, scale_inv, stream);
}

int pt_compute_group_offs(const int64_t *group_lens, int64_t num_groups, int64_t align,
                          int64_t *padded_lens, int64_t *group_offs, void *stream) {
    PT_REQUIRE(num_groups >= 0 && num_groups < (1 << 24), "bad group count");
    PT_REQUIRE(align >= 1, "align must be >= 1");
    PT_REQUIRE(group_offs != nullptr && (num_groups == 0 || group_lens != nullptr),
               "NULL tensor pointer");
    group_offs_kernel<<<1, 64, 0, static_cast<hipStream_t>(stream)>>>(
        group_lens, padded_lens, group_offs, static_cast<int>(num_groups), align);
    return check_launch("group_offs_kernel");
}

static int quantize_segment_m(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype, const int64_t *group_offs,
                              const int64_t *padded_group_offs, int64_t num_groups, void *q_row, float *scale_inv_row,
                              void *q_col_padded, void *q_col_t, int64_t ldt, float *scale_inv_col_padded,
                              void *stream, int glu = 0, const float *probs = nullptr,
                              const int64_t *row_mask = nullptr) {
    PT_REQUIRE(is_hp_dtype(x_dtype), "input must be bf16, fp16 or fp32");
    PT_REQUIRE(glu == 0 || ((x_dtype == PT_DTYPE_BF16 || x_dtype == PT_DTYPE_F16) && probs != nullptr),
               "the gated input must be bf16 or fp16 and needs the router probabilities");
    PT_REQUIRE(is_fp8_dtype(q_dtype), "output must be e4m3 or e5m2");
    PT_REQUIRE(M >= 0 && N >= 0 && num_groups >= 1, "bad dimensions");
    PT_REQUIRE(group_offs && padded_group_offs, "group offsets must not be NULL");
    PT_REQUIRE(q_row && scale_inv_row && (q_col_padded || q_col_t) && scale_inv_col_padded, "NULL output pointer");
    if (N == 0)
        return PT_OK;
    PT_REQUIRE(x != nullptr || M == 0, "x must not be NULL");
    const int64_t tm = cdiv(M + num_groups * BQ, BQ), tn = cdiv(N, BQ);
    PT_REQUIRE(tm < 65536, "too many row tiles");
    if (q_col_t != nullptr)
        PT_REQUIRE(ldt >= tm * BQ && ldt % 16 == 0 && aligned_to(q_col_t, 16),
                   "the transposed column output needs a 16-byte aligned pitch that holds every padded group");
    BlockQuantArgs a{};
    a.x = x;
    a.q_row = static_cast<uint8_t *>(q_row);
    a.s_row = scale_inv_row;
    a.q_col = static_cast<uint8_t *>(q_col_padded);
    a.s_col = scale_inv_col_padded;
    a.q_t = static_cast<uint8_t *>(q_col_t);
    a.ldt = ldt;
    a.M = M;
    a.N = N;
    a.rs_m = 1; // row scales are stored transposed: [N / 128, M]
    a.rs_n = M;
    a.group_offs = group_offs;
    a.padded_offs = padded_group_offs;
    a.num_groups = static_cast<int>(num_groups);
    a.qmax = fp8_max_of(q_dtype);
    a.probs    = probs;
    a.row_mask = row_mask;
    auto       st  = static_cast<hipStream_t>(stream);
    const bool vec = vec_ok(a, 1);
    if (glu != 0) {
        const bool e5 = q_dtype == PT_DTYPE_E5M2;
#define CALL_GLU(T, E5, ACT) return launch_block128<T, E5, MODE_ROW | MODE_COL, true, 1 + ACT>(a, tm, tn, 1, vec, st)
        if (x_dtype == PT_DTYPE_BF16) {
            if (glu == 1 + ACT_SILU) { if (e5) CALL_GLU(bf16_t, true, ACT_SILU); else CALL_GLU(bf16_t, false, ACT_SILU); }
            else { if (e5) CALL_GLU(bf16_t, true, ACT_GELU); else CALL_GLU(bf16_t, false, ACT_GELU); }
        } else {
            if (glu == 1 + ACT_SILU) { if (e5) CALL_GLU(f16_t, true, ACT_SILU); else CALL_GLU(f16_t, false, ACT_SILU); }
            else { if (e5) CALL_GLU(f16_t, true, ACT_GELU); else CALL_GLU(f16_t, false, ACT_GELU); }
        }
#undef CALL_GLU
    }
#define CALL(T, E5) return launch_block128<T, E5, MODE_ROW | MODE_COL, true>(a, tm, tn, 1, vec, st)
    PT_DISPATCH_T_E5(x_dtype, q_dtype, CALL);
#undef CALL
}

int pt_quantize_fp8_blockwise_segment_m_row_col(const void *x, int x_dtype, int64_t M, int64_t N,
                                                int q_dtype, const int64_t *group_offs,
                                                const int64_t *padded_group_offs,
                                                int64_t num_groups, void *q_row,
                                                float *scale_inv_row, void *q_col_padded,
                                                float *scale_inv_col_padded, void *stream) {
    PT_REQUIRE(q_col_padded != nullptr, "NULL output pointer");
    return quantize_segment_m(x, x_dtype, M, N, q_dtype, group_offs, padded_group_offs, num_groups, q_row, scale_inv_row,
                              q_col_padded, nullptr, 0, scale_inv_col_padded, stream);
}

int pt_quantize_fp8_blockwise_segment_m_row_col_t(const void *x, int x_dtype, int64_t M, int64_t N, int q_dtype,
                                                  const int64_t *group_offs, const int64_t *padded_group_offs,
                                                  int64_t num_groups, void *q_row, float *scale_inv_row,
                                                  void *q_col_padded, void *q_col_t, int64_t ldt,
                                                  float *scale_inv_col_padded, void *stream) {
    PT_REQUIRE(q_col_t != nullptr, "q_col_t must not be NULL");
    return quantize_segment_m(x, x_dtype, M, N, q_dtype, group_offs, padded_group_offs, num_groups, q_row, scale_inv_row,
                              q_col_padded, q_col_t, ldt, scale_inv_col_padded, stream);
}

int pt_glu_quantize_fp8_blockwise_segment_m_row_col(const void *x, int x_dtype, const float *probs,
                                                    const int64_t *row_mask, int act, int64_t M, int64_t N, int q_dtype,
                                                    const int64_t *group_offs, const int64_t *padded_group_offs,
                                                    int64_t num_groups, void *q_row, float *scale_inv_row,
                                                    void *q_col_padded, void *q_col_t, int64_t ldt,
                                                    float *scale_inv_col_padded, void *stream) {
    PT_REQUIRE(act == ACT_SILU || act == ACT_GELU, "act must be 0 (SiLU) or 1 (GELU)");
    PT_REQUIRE(q_col_padded != nullptr || q_col_t != nullptr, "NULL output pointer");
    return quantize_segment_m(x, x_dtype, M, N, q_dtype, group_offs, padded_group_offs, num_groups, q_row, scale_inv_row,
                              q_col_padded, q_col_t, ldt, scale_inv_col_padded, stream, 1 + act, probs, row_mask);
}

int pt_dequantize_fp8_block(const void *q, int q_dtype, int64_t B, int64_t M, int64_t N,
                            const float *scale_inv, int64_t block_m, int64_t block_n, void *y,
                            int y_dtype, void *stream) {
    PT_REQUIRE(is_fp8_dtype(q_dtype), "input must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(y_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(B >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    PT_REQUIRE(block_m >= 1 && block_n >= 1, "block sizes must be positive");
    if (B * M * N == 0)
        return PT_OK;
    PT_REQUIRE(q && y && scale_inv, "NULL tensor pointer");
    auto          st    = static_cast<hipStream_t>(stream);
    const int64_t total = B * M * N;
    const bool    vec   = N % 16 == 0 && aligned_to(q, 16) && aligned_to(y, 16) &&
                     (block_n == 1 || block_n % 16 == 0);
    const int bm = static_cast<int>(block_m), bn = static_cast<int>(block_n);
    int64_t   grid = cdiv(vec ? total / 16 : total, 256);
    if (grid > 16384)
        grid = 16384;
    const unsigned g = static_cast<unsigned>(grid);
#define CALL(T, E5)                                                                                \
    do {                                                                                           \
        if (vec && bn == 1)                                                                        \
            dequant_block_vec_kernel<T, E5, true><<<g, 256, 0, st>>>(                              \
                static_cast<const uint8_t *>(q), scale_inv, static_cast<T *>(y), B, M, N, bm, bn); \
        else if (vec)                                                                              \
            dequant_block_vec_kernel<T, E5, false><<<g, 256, 0, st>>>(                             \
                static_cast<const uint8_t *>(q), scale_inv, static_cast<T *>(y), B, M, N, bm, bn); \
        else                                                                                       \
            dequant_block_kernel<T, E5><<<g, 256, 0, st>>>(                                        \
                static_cast<const uint8_t *>(q), scale_inv, static_cast<T *>(y), B, M, N, bm, bn); \
        return check_launch("dequant_block_kernel");                                               \
    } while (0)
    PT_DISPATCH_T_E5(y_dtype, q_dtype, CALL);
#undef CALL
}

} // extern "C"
