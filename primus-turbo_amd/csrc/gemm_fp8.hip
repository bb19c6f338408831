// Scaled FP8 GEMM entry points: operand preparation (transposes / K padding), the
// VECTOR-scale (tensorwise, rowwise) kernel instantiations and the C ABI. The BLOCK-scale
// instantiations live in gemm_fp8_block.hip, which is compiled with MFMA results in VGPRs.
#include "gemm_fp8_kernel.h"

namespace pt {


// ---------------------------------------------------------------------------
// fp8 byte matrix transpose in[R, C] -> out[C, ldo] through a padded 64 x 64 LDS tile;
// columns [R, ldo) of every output row are zero-filled. Brings operands whose reduction
// axis is not contiguous into NT form (and pads K to a multiple of 128 on the way).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose_u8_kernel(const uint8_t *__restrict__ in,
                                                           uint8_t *__restrict__ out,
                                                           const int64_t R, const int64_t C,
                                                           const int64_t ldo) {
    __shared__ uint8_t t[64][64 + 4];
    const int64_t      r0 = static_cast<int64_t>(blockIdx.y) * 64, c0 = static_cast<int64_t>(blockIdx.x) * 64;
    const int64_t      bi = static_cast<int64_t>(blockIdx.z) * R * C, bo = static_cast<int64_t>(blockIdx.z) * C * ldo;
    const int          tx = threadIdx.x & 15, ty = threadIdx.x >> 4; // 16 x 16 threads, 4 bytes each
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     r  = ty + 16 * p;
        const int64_t gr = r0 + r, gc = c0 + tx * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            t[r][tx * 4 + e] = (gr < R && gc + e < C) ? in[bi + gr * C + gc + e] : 0;
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     c  = ty + 16 * p; // output row = input column
        const int64_t gc = c0 + c, gr = r0 + tx * 4;
        if (gc < C) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (gr + e < ldo)
                    out[bo + gc * ldo + gr + e] = t[tx * 4 + e][c]; // rows >= R were loaded as 0
        }
    }
}

// in[R, C] -> out[R, ldo], columns [C, ldo) zero-filled (K padding of a K-contiguous operand)
__global__ __launch_bounds__(256) void pad_rows_u8_kernel(const uint8_t *__restrict__ in,
                                                          uint8_t *__restrict__ out, const int64_t R,
                                                          const int64_t C, const int64_t ldo) {
    const int64_t total  = R * ldo;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / ldo, c = i % ldo;
        out[i]          = c < C ? in[r * C + c] : 0;
    }
}

// The same for 16-byte aligned shapes: a workgroup moves a 128 x 128 byte tile. A thread loads
// 16 bytes from each of four consecutive rows, transposes the four 4 x 4 byte blocks in
// registers (v_perm_b32) and writes 16 words "four rows of one column" into the LDS tile, which
// is then written out as full 128-byte rows.
__global__ __launch_bounds__(256) void transpose_u8_tile128_kernel(const uint8_t *__restrict__ in,
                                                                   uint8_t *__restrict__ out, const int64_t R,
                                                                   const int64_t C, const int64_t ldo) {
    constexpr int  P = 33; // words per LDS row: conflict-free 16-byte row reads, 2-way column writes
    __shared__ uint32_t t[128 * P];
    const int64_t  r0 = static_cast<int64_t>(blockIdx.y) * 128, c0 = static_cast<int64_t>(blockIdx.x) * 128;
    const int64_t  bi = static_cast<int64_t>(blockIdx.z) * R * C, bo = static_cast<int64_t>(blockIdx.z) * C * ldo;
    const int      tid = threadIdx.x;
    {
        const int     cc = tid & 7, rg = tid >> 3; // 16-byte column chunk, group of four rows
        const int64_t gc = c0 + cc * 16;
        u32x4         a[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t gr = r0 + rg * 4 + e;
            a[e] = (gr < R && gc < C) ? *reinterpret_cast<const u32x4 *>(in + bi + gr * C + gc) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) { // word w of the four rows = columns 4w .. 4w+3
            const uint32_t t0 = __builtin_amdgcn_perm(a[1][w], a[0][w], 0x05010400u);
            const uint32_t t1 = __builtin_amdgcn_perm(a[1][w], a[0][w], 0x07030602u);
            const uint32_t t2 = __builtin_amdgcn_perm(a[3][w], a[2][w], 0x05010400u);
            const uint32_t t3 = __builtin_amdgcn_perm(a[3][w], a[2][w], 0x07030602u);
            const int      c  = cc * 16 + w * 4;
            t[(c + 0) * P + rg] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
            t[(c + 1) * P + rg] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
            t[(c + 2) * P + rg] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
            t[(c + 3) * P + rg] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
        }
    }
    __syncthreads();
    const int j = tid & 7; // 16-byte chunk of an output row
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int     c  = (tid >> 3) + 32 * p; // output row = input column
        const int64_t gc = c0 + c, gr = r0 + j * 16;
        if (gc < C && gr < ldo) {
            u32x4 v;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                v[k] = t[c * P + j * 4 + k];
            *reinterpret_cast<u32x4 *>(out + bo + gc * ldo + gr) = v; // rows >= R were loaded as 0
        }
    }
}

// out[b, c, r] = in[b, r, c] for 2-, 4- and 8-byte elements through a padded 32 x 32 LDS tile
// (coalesced rows on both sides).
template <typename E>
__global__ __launch_bounds__(256) void transpose_elem_kernel(const E *__restrict__ in, E *__restrict__ out, const int64_t R,
                                                             const int64_t C) {
    __shared__ E  t[32][33];
    const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 32, c0 = static_cast<int64_t>(blockIdx.x) * 32;
    const int64_t b  = static_cast<int64_t>(blockIdx.z) * R * C;
    const int     tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8 threads
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int64_t r = r0 + ty + 8 * p, c = c0 + tx;
        if (r < R && c < C)
            t[ty + 8 * p][tx] = in[b + r * C + c];
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int64_t c = c0 + ty + 8 * p, r = r0 + tx;
        if (c < C && r < R)
            out[b + c * R + r] = t[tx][ty + 8 * p];
    }
}

void launch_transpose(const uint8_t *in, uint8_t *out, int64_t batch, int64_t R, int64_t C,
                      int64_t ldo, hipStream_t st) {
    if (batch <= 0 || C <= 0 || ldo <= 0)
        return;
    // the grids cover ldo (>= R) input-row positions so that the zero tail gets written too
    const bool aligned = C % 16 == 0 && ldo % 16 == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 &&
                         reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (aligned) {
        dim3 g(static_cast<unsigned>(cdiv(C, 128)), static_cast<unsigned>(cdiv(ldo, 128)), static_cast<unsigned>(batch));
        transpose_u8_tile128_kernel<<<g, 256, 0, st>>>(in, out, R, C, ldo);
        return;
    }
    dim3 g(static_cast<unsigned>(cdiv(C, 64)), static_cast<unsigned>(cdiv(ldo, 64)),
           static_cast<unsigned>(batch));
    transpose_u8_kernel<<<g, 256, 0, st>>>(in, out, R, C, ldo);
}

// out[w, r] = in[r * pitch + w] for w < W: the scale words of one K position of all rows made
// contiguous (32 x 32 word tiles through LDS, coalesced on both sides)
__global__ __launch_bounds__(256) void transpose_words_kernel(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                                              const int64_t R, const int64_t W, const int64_t pitch) {
    __shared__ uint32_t t[32][33];
    in += static_cast<int64_t>(blockIdx.z) * R * pitch; // batch of matrices, each transposed on its own
    out += static_cast<int64_t>(blockIdx.z) * W * R;
    const int64_t w0 = static_cast<int64_t>(blockIdx.x) * 32;
    const int     tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    // (the row tiles are walked with the grid's y extent as the stride: it is capped at 65535)
    for (int64_t r0 = static_cast<int64_t>(blockIdx.y) * 32; r0 < R; r0 += static_cast<int64_t>(gridDim.y) * 32) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int64_t r = r0 + ty + 8 * p, w = w0 + tx;
            if (r < R && w < W)
                t[ty + 8 * p][tx] = in[r * pitch + w];
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int64_t w = w0 + ty + 8 * p, r = r0 + tx;
            if (w < W && r < R)
                out[w * R + r] = t[tx][ty + 8 * p];
        }
        __syncthreads();
    }
}

int launch_transpose_words(const uint32_t *in, uint32_t *out, int64_t R, int64_t W, int64_t pitch, hipStream_t st,
                           int64_t batch) {
    if (R * W * batch == 0)
        return PT_OK;
    if (batch > 65535)
        return fail(PT_ERR_INVALID_ARGUMENT, "transpose_words: more than 65535 matrices in a batch");
    const int64_t gy = cdiv(R, 32) < 65535 ? cdiv(R, 32) : 65535;
    dim3 g(static_cast<unsigned>(cdiv(W, 32)), static_cast<unsigned>(gy), static_cast<unsigned>(batch));
    transpose_words_kernel<<<g, 256, 0, st>>>(in, out, R, W, pitch);
    return check_launch("transpose_words_kernel");
}

template <int FA, int FB>
static int launch_vector_tiles(const GemmArgs &a, int tile_cfg, hipStream_t stream) {
    // tile_cfg: 0 = auto, 1 = 256x256, 2 = 256x128, 3 = 128x128
    if (tile_cfg == 0)
        tile_cfg = (a.M >= 2048 && a.N >= 2048) ? 1 : 3;
    if (tile_cfg == 1 || tile_cfg == 4)
        return launch_gemm_cfg<8, 8, SCALE_VECTOR, false, FA, FB>(a, stream);
    if (tile_cfg == 2)
        return launch_gemm_cfg<8, 4, SCALE_VECTOR, false, FA, FB>(a, stream);
    return launch_gemm_cfg<4, 4, SCALE_VECTOR, false, FA, FB>(a, stream);
}

static int launch_gemm_vector(const GemmArgs &a, int fa, int fb, int tile_cfg, hipStream_t stream) {
    if (fa == 0 && fb == 0)
        return launch_vector_tiles<0, 0>(a, tile_cfg, stream);
    if (fa == 0 && fb == 1)
        return launch_vector_tiles<0, 1>(a, tile_cfg, stream);
    if (fa == 1 && fb == 0)
        return launch_vector_tiles<1, 0>(a, tile_cfg, stream);
    return launch_vector_tiles<1, 1>(a, tile_cfg, stream);
}

// in[R, C] with row pitch ldi -> out[R, ldo], columns [C, ldo) zero-filled
__global__ __launch_bounds__(256) void pad_rows2_u8_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                           const int64_t R, const int64_t C, const int64_t ldi,
                                                           const int64_t ldo) {
    const int64_t total  = R * ldo;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / ldo, c = i % ldo;
        out[i]          = c < C ? in[r * ldi + c] : 0;
    }
}

void launch_pad_rows2(const uint8_t *in, uint8_t *out, int64_t R, int64_t C, int64_t ldi, int64_t ldo, hipStream_t st) {
    if (R * ldo > 0)
        pad_rows2_u8_kernel<<<static_cast<unsigned>(cdiv(R * ldo, 256 * 16)), 256, 0, st>>>(in, out, R, C, ldi, ldo);
}

void launch_pad_rows(const uint8_t *in, uint8_t *out, int64_t R, int64_t C, int64_t ldo, hipStream_t st) {
    pad_rows_u8_kernel<<<static_cast<unsigned>(cdiv(R * ldo, 256 * 16)), 256, 0, st>>>(in, out, R, C, ldo);
}

// zero `bytes` bytes at a 16-byte aligned address (a fill kernel rather than a memset node,
// so that callers may capture the launch in a graph)
__global__ __launch_bounds__(256) void zero16_kernel(u32x4 *p, int64_t n16, int64_t bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n16) {
        if ((i + 1) * 16 <= bytes) {
            p[i] = u32x4{0u, 0u, 0u, 0u};
        } else {
            uint8_t *b = reinterpret_cast<uint8_t *>(p);
            for (int64_t k = i * 16; k < bytes; ++k)
                b[k] = 0;
        }
    }
}

} // namespace pt

using namespace pt;

extern "C" {

// Block-scale GEMMs whose A scales are stored one row of K blocks per matrix row ([M, K / 128],
// the 1 x 128 activation quantizer's layout) get a copy with the scales of one K block of all rows
// contiguous ([K / 128, M]): a scale copy of the kernel (64 rows per instruction) then reads two
// cache lines instead of sixty-four.
static bool block_scale_copy_pays(int64_t M, int64_t N, int64_t K) {
    return M >= 1024 && N >= 1024 && K >= 1024;
}

size_t pt_gemm_fp8_workspace_bytes(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b) {
    // An operand is copied into the workspace when its reduction axis is not contiguous
    // (transpose) or when K is not a multiple of 128 (zero padding of the K tail).
    const int64_t Kp    = padded_k(K);
    const bool    pad   = Kp != K;
    size_t        bytes = 0;
    if (block_scale_copy_pays(M, N, K))
        bytes += static_cast<size_t>(round_up(M * cdiv(K, 128) * 4, 256));
    if (trans_a || pad)
        bytes += static_cast<size_t>(round_up(M * Kp, 256));
    if (!trans_b || pad)
        bytes += static_cast<size_t>(round_up(N * Kp, 256));
    return bytes;
}

int pt_gemm_fp8(const void *a, int a_dtype, const float *a_scale, const void *b, int b_dtype,
                const float *b_scale, void *c, int c_dtype, int64_t M, int64_t N, int64_t K,
                int trans_a, int trans_b, int scale_mode, int64_t sa_m, int64_t sa_k, int64_t sb_n,
                int64_t sb_k, int sa_block, int sb_block, int accumulate, void *workspace,
                size_t workspace_bytes, int tile_cfg, void *stream) {
    PT_REQUIRE(is_fp8_dtype(a_dtype) && is_fp8_dtype(b_dtype), "operands must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(c_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(M >= 0 && N >= 0 && K >= 0, "dimensions must be non-negative");
    PT_REQUIRE(scale_mode == SCALE_VECTOR || scale_mode == SCALE_BLOCK, "unknown scale mode");
    PT_REQUIRE(scale_mode != SCALE_BLOCK || ((sa_block == 1 || sa_block == 128) && (sb_block == 1 || sb_block == 128)),
               "sa_block / sb_block must be 1 or 128");
    PT_REQUIRE(tile_cfg >= 0 && tile_cfg <= 4, "tile_cfg must be 0..4");
    if (M == 0 || N == 0)
        return PT_OK;
    PT_REQUIRE(a && b && c && a_scale && b_scale, "NULL tensor pointer");
    PT_REQUIRE(aligned_to(a, 16) && aligned_to(b, 16) && aligned_to(c, 16), "operands must be 16-byte aligned");
    PT_REQUIRE(cdiv(M, 128) * cdiv(N, 128) < (1LL << 31), "too many tiles");
    // the kernel addresses a tile's rows with 32-bit byte offsets: 255 rows x K must fit
    PT_REQUIRE(K < (1LL << 24), "K must be below 2^24");
    auto st = static_cast<hipStream_t>(stream);
    if (K == 0) { // empty sum
        if (!accumulate) {
            const int64_t n16 = cdiv(M * N * (c_dtype == PT_DTYPE_F32 ? 4 : 2), 16);
            zero16_kernel<<<static_cast<unsigned>(cdiv(n16, 256)), 256, 0, st>>>(static_cast<u32x4 *>(c), n16, M * N * (c_dtype == PT_DTYPE_F32 ? 4 : 2));
            return check_launch("zero16_kernel");
        }
        return PT_OK;
    }

    const int64_t  Kp  = padded_k(K);
    const bool     pad = Kp != K;
    const uint8_t *A   = static_cast<const uint8_t *>(a);
    const uint8_t *B   = static_cast<const uint8_t *>(b);
    // workspace layout: [scale area of block_scale_copy_pays problems][operand copies]
    const int64_t KB         = cdiv(K, 128);
    const size_t  full       = pt_gemm_fp8_workspace_bytes(M, N, K, trans_a, trans_b);
    const bool    have_ws    = workspace != nullptr && aligned_to(workspace, 16) && workspace_bytes >= full;
    const size_t  scale_area = block_scale_copy_pays(M, N, K) ? static_cast<size_t>(round_up(M * KB * 4, 256)) : 0;
    // per-row A scales stored [M, K / 128] (sa_k == 1): hand the kernel a [K / 128, M] copy
    if (have_ws && scale_area != 0 && scale_mode == SCALE_BLOCK && sa_block == 1 && sa_k == 1 && sa_m >= KB) {
        if (const int rc = launch_transpose_words(reinterpret_cast<const uint32_t *>(a_scale), static_cast<uint32_t *>(workspace), M, KB, sa_m, st))
            return rc;
        a_scale = static_cast<const float *>(workspace);
        sa_m    = 1;
        sa_k    = M;
    }
    if (trans_a || !trans_b || pad) {
        if (!have_ws)
            return fail(PT_ERR_WORKSPACE, "pt_gemm_fp8: workspace missing, too small or misaligned");
        uint8_t *ws = static_cast<uint8_t *>(workspace) + scale_area;
        if (trans_a || pad) {
            if (M * Kp > 0) {
                if (trans_a) // stored [K, M] -> [M, Kp]
                    launch_transpose(A, ws, 1, K, M, Kp, st);
                else
                    launch_pad_rows(A, ws, M, K, Kp, st);
            }
            A = ws;
            ws += round_up(M * Kp, 256);
        }
        if (!trans_b || pad) {
            if (N * Kp > 0) {
                if (!trans_b) // stored [K, N] -> [N, Kp]
                    launch_transpose(B, ws, 1, K, N, Kp, st);
                else
                    launch_pad_rows(B, ws, N, K, Kp, st);
            }
            B = ws;
        }
    }

    GemmArgs g{};
    g.A = A;
    g.B = B;
    g.C = c;
    g.sA = a_scale;
    g.sB = b_scale;
    g.M = M;
    g.N = N;
    g.K = Kp;
    g.lda = Kp;
    g.ldb = Kp;
    g.sa_m = sa_m;
    g.sa_k = sa_k;
    g.sb_n = sb_n;
    g.sb_k = sb_k;
    g.sa_shift = sa_block == 128 ? 7 : 0;
    g.sb_shift = sb_block == 128 ? 7 : 0;
    g.kb_valid = static_cast<int>(cdiv(K, 128));
    g.out_dtype = c_dtype;
    g.accumulate = accumulate;
    const int fa = a_dtype == PT_DTYPE_E5M2 ? 1 : 0, fb = b_dtype == PT_DTYPE_E5M2 ? 1 : 0;
    if (scale_mode == SCALE_VECTOR)
        return launch_gemm_vector(g, fa, fb, tile_cfg, st);
    return launch_gemm_block(g, fa, fb, sb_block == 1, tile_cfg, st);
}

int pt_transpose_2d(const void *in, void *out, int64_t batch, int64_t R, int64_t C, int elem_bytes, void *stream) {
    PT_REQUIRE(batch >= 0 && R >= 0 && C >= 0, "dimensions must be non-negative");
    PT_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8, "element size must be 1, 2, 4 or 8 bytes");
    if (elem_bytes == 1)
        return pt_transpose_u8(in, out, batch, R, C, stream);
    if (batch * R * C == 0)
        return PT_OK;
    PT_REQUIRE(in && out, "NULL tensor pointer");
    PT_REQUIRE(batch < 65536 && cdiv(R, 32) < 65536, "grid dimension out of range");
    dim3 g(static_cast<unsigned>(cdiv(C, 32)), static_cast<unsigned>(cdiv(R, 32)), static_cast<unsigned>(batch));
    auto st = static_cast<hipStream_t>(stream);
    if (elem_bytes == 2)
        transpose_elem_kernel<uint16_t><<<g, 256, 0, st>>>(static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), R, C);
    else if (elem_bytes == 4)
        transpose_elem_kernel<uint32_t><<<g, 256, 0, st>>>(static_cast<const uint32_t *>(in), static_cast<uint32_t *>(out), R, C);
    else
        transpose_elem_kernel<uint64_t><<<g, 256, 0, st>>>(static_cast<const uint64_t *>(in), static_cast<uint64_t *>(out), R, C);
    return check_launch("transpose_elem_kernel");
}

int pt_transpose_u8(const void *in, void *out, int64_t batch, int64_t R, int64_t C, void *stream) {
    PT_REQUIRE(batch >= 0 && R >= 0 && C >= 0, "dimensions must be non-negative");
    if (batch * R * C == 0)
        return PT_OK;
    PT_REQUIRE(in && out, "NULL tensor pointer");
    PT_REQUIRE(batch < 65536 && cdiv(R, 64) < 65536, "grid dimension out of range");
    launch_transpose(static_cast<const uint8_t *>(in), static_cast<uint8_t *>(out), batch, R, C, R,
                     static_cast<hipStream_t>(stream));
    return check_launch("transpose_u8_kernel");
}

} // extern "C"
