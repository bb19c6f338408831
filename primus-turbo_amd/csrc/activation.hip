// Gated activations of an MoE expert MLP between its two grouped GEMMs:
//   out[t, c] = act(x[t, c]) * x[t, H + c] * probs[t]          act = SiLU or exact (erf) GELU
// and their backward, following Primus-Turbo's swiglu_with_probs / geglu_with_probs
// (primus_turbo/triton/activation/swiglu_kernel.py:11-248, geglu_kernel.py, utils/gelu.py:24-49;
// host side primus_turbo/pytorch/kernels/activation/swiglu_impl.py:20-117). HBM-bound: one
// workgroup per token row, 16-byte loads and stores, fp32 arithmetic, the per-row gradient of
// the router probability reduced through DPP and a few LDS words.
//
// Differences, both outside what the reference's own test observes: rows whose row_mask is 0
// are written as zeros (the reference leaves them unwritten), and the GELU gradient of the gate
// is grad_out * probs * up * gelu'(gate) (the reference multiplies by grad_out once more, which
// only agrees for grad_out = 1).
#include "pt_activation.h"

namespace pt {

// -> (act(g), act'(g))
template <int ACT> __device__ __forceinline__ void act_both(float g, float &a, float &da) {
    if constexpr (ACT == ACT_SILU) {
        const float s = 1.0f / (1.0f + expf(-g));
        a             = s * g;
        da            = s * (1.0f + g * (1.0f - s));
    } else {
        const float e = erff(g * 0.7071067811f);
        a             = 0.5f * g * (1.0f + e);
        da            = 0.3989422803f * g * expf(-(0.7071067811f * g) * (0.7071067811f * g)) + 0.5f * e + 0.5f;
    }
}

template <typename T> __device__ __forceinline__ void unpack8(const u32x4 &w, float (&f)[8]) {
    unpack2<T>(w.x, f[0], f[1]);
    unpack2<T>(w.y, f[2], f[3]);
    unpack2<T>(w.z, f[4], f[5]);
    unpack2<T>(w.w, f[6], f[7]);
}
template <typename T> __device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    return u32x4{pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])};
}

// sum over the 64 lanes of a wavefront (DPP row reduction, then the four row totals)
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    float r = 0.f;
#pragma unroll
    for (int l = 0; l < 64; l += 16)
        r += __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), l));
    return r;
}

// VEC: H % 8 == 0 and 16-byte aligned rows
template <typename T, int ACT, bool VEC>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const T *__restrict__ x, const float *__restrict__ probs,
                                                      const int64_t *__restrict__ row_mask, T *__restrict__ out,
                                                      const int64_t rows, const int64_t H) {
    for (int64_t t = blockIdx.x; t < rows; t += gridDim.x) {
        const bool  live = row_mask == nullptr || row_mask[t] != 0;
        const float p    = live ? probs[t] : 0.f;
        const T    *g = x + t * 2 * H, *u = g + H;
        T          *o = out + t * H;
        if constexpr (VEC) {
            for (int64_t c = threadIdx.x * 8; c < H; c += 256 * 8) {
                float r[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (live) {
                    float fg[8], fu[8];
                    unpack8<T>(ld128_nt(g + c), fg);
                    unpack8<T>(ld128_nt(u + c), fu);
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        r[k] = act_fwd<ACT>(fg[k]) * fu[k] * p;
                }
                st128(o + c, pack8<T>(r));
            }
        } else {
            for (int64_t c = threadIdx.x; c < H; c += 256)
                o[c] = HP<T>::from_f32(live ? act_fwd<ACT>(HP<T>::to_f32(g[c])) * HP<T>::to_f32(u[c]) * p : 0.f);
        }
    }
}

template <typename T, int ACT, bool VEC>
__global__ __launch_bounds__(256) void glu_bwd_kernel(const T *__restrict__ grad_out, const T *__restrict__ x,
                                                      const float *__restrict__ probs,
                                                      const int64_t *__restrict__ row_mask, T *__restrict__ grad_x,
                                                      float *__restrict__ grad_probs, const int64_t rows,
                                                      const int64_t H) {
    __shared__ float s_part[4];
    for (int64_t t = blockIdx.x; t < rows; t += gridDim.x) {
        const bool  live = row_mask == nullptr || row_mask[t] != 0;
        const float p    = live ? probs[t] : 0.f;
        const T    *g = x + t * 2 * H, *u = g + H, *go = grad_out + t * H;
        T          *dg = grad_x + t * 2 * H, *du = dg + H;
        float       acc = 0.f; // sum over the row of grad_out * act(gate) * up
        if constexpr (VEC) {
            for (int64_t c = threadIdx.x * 8; c < H; c += 256 * 8) {
                float rg[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, ru[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (live) {
                    float fg[8], fu[8], fo[8];
                    unpack8<T>(ld128_nt(g + c), fg);
                    unpack8<T>(ld128_nt(u + c), fu);
                    unpack8<T>(ld128_nt(go + c), fo);
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        float a, da;
                        act_both<ACT>(fg[k], a, da);
                        acc += fo[k] * a * fu[k];
                        const float gp = fo[k] * p;
                        ru[k]          = gp * a;
                        rg[k]          = gp * (fu[k] * da);
                    }
                }
                st128_nt(dg + c, pack8<T>(rg)); // (streaming stores: the step's 198 -> 179 us; the forward
                st128_nt(du + c, pack8<T>(ru)); //  output keeps plain stores, its reader follows at once)
            }
        } else {
            for (int64_t c = threadIdx.x; c < H; c += 256) {
                float vg = 0.f, vu = 0.f;
                if (live) {
                    float a, da;
                    act_both<ACT>(HP<T>::to_f32(g[c]), a, da);
                    const float fo = HP<T>::to_f32(go[c]), fu = HP<T>::to_f32(u[c]);
                    acc += fo * a * fu;
                    vu = fo * p * a;
                    vg = fo * p * (fu * da);
                }
                dg[c] = HP<T>::from_f32(vg);
                du[c] = HP<T>::from_f32(vu);
            }
        }
        acc = wave_sum(acc);
        __syncthreads(); // the previous row's partial sums have been read
        if ((threadIdx.x & 63) == 0)
            s_part[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0)
            grad_probs[t] = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
    }
}

static unsigned glu_grid(int64_t rows) {
    const int64_t cap = 32L * device_cu_count();
    return static_cast<unsigned>(rows < cap ? rows : cap);
}

} // namespace pt

using namespace pt;

extern "C" {

int pt_glu_with_probs_fwd(const void *x, int x_dtype, const float *probs, const int64_t *row_mask, void *out,
                          int64_t rows, int64_t H, int act, void *stream) {
    PT_REQUIRE(x_dtype == PT_DTYPE_BF16 || x_dtype == PT_DTYPE_F16, "x must be bf16 or fp16");
    PT_REQUIRE(rows >= 0 && H >= 0, "dimensions must be non-negative");
    PT_REQUIRE(act == ACT_SILU || act == ACT_GELU, "act must be 0 (silu) or 1 (gelu)");
    if (rows == 0 || H == 0)
        return PT_OK;
    PT_REQUIRE(x && probs && out, "NULL tensor pointer");
    const bool vec = H % 8 == 0 && aligned_to(x, 16) && aligned_to(out, 16);
    auto       st  = static_cast<hipStream_t>(stream);
    const unsigned grid = glu_grid(rows);
#define CALL(T, A)                                                                                                        \
    do {                                                                                                                  \
        if (vec)                                                                                                          \
            glu_fwd_kernel<T, A, true><<<grid, 256, 0, st>>>(static_cast<const T *>(x), probs, row_mask,                 \
                                                             static_cast<T *>(out), rows, H);                            \
        else                                                                                                              \
            glu_fwd_kernel<T, A, false><<<grid, 256, 0, st>>>(static_cast<const T *>(x), probs, row_mask,                \
                                                              static_cast<T *>(out), rows, H);                           \
    } while (0)
    if (x_dtype == PT_DTYPE_BF16) {
        if (act == ACT_SILU) CALL(bf16_t, ACT_SILU); else CALL(bf16_t, ACT_GELU);
    } else {
        if (act == ACT_SILU) CALL(f16_t, ACT_SILU); else CALL(f16_t, ACT_GELU);
    }
#undef CALL
    return check_launch("glu_fwd_kernel");
}

int pt_glu_with_probs_bwd(const void *grad_out, const void *x, int x_dtype, const float *probs, const int64_t *row_mask,
                          void *grad_x, float *grad_probs, int64_t rows, int64_t H, int act, void *stream) {
    PT_REQUIRE(x_dtype == PT_DTYPE_BF16 || x_dtype == PT_DTYPE_F16, "x must be bf16 or fp16");
    PT_REQUIRE(rows >= 0 && H >= 0, "dimensions must be non-negative");
    PT_REQUIRE(act == ACT_SILU || act == ACT_GELU, "act must be 0 (silu) or 1 (gelu)");
    if (rows == 0)
        return PT_OK;
    PT_REQUIRE(probs && grad_probs && (H == 0 || (grad_out && x && grad_x)), "NULL tensor pointer");
    const bool vec = H % 8 == 0 && aligned_to(x, 16) && aligned_to(grad_out, 16) && aligned_to(grad_x, 16);
    auto       st  = static_cast<hipStream_t>(stream);
    const unsigned grid = glu_grid(rows);
#define CALL(T, A)                                                                                                        \
    do {                                                                                                                  \
        if (vec)                                                                                                          \
            glu_bwd_kernel<T, A, true><<<grid, 256, 0, st>>>(static_cast<const T *>(grad_out), static_cast<const T *>(x), \
                                                             probs, row_mask, static_cast<T *>(grad_x), grad_probs,      \
                                                             rows, H);                                                   \
        else                                                                                                              \
            glu_bwd_kernel<T, A, false><<<grid, 256, 0, st>>>(static_cast<const T *>(grad_out),                          \
                                                              static_cast<const T *>(x), probs, row_mask,                \
                                                              static_cast<T *>(grad_x), grad_probs, rows, H);            \
    } while (0)
    if (x_dtype == PT_DTYPE_BF16) {
        if (act == ACT_SILU) CALL(bf16_t, ACT_SILU); else CALL(bf16_t, ACT_GELU);
    } else {
        if (act == ACT_SILU) CALL(f16_t, ACT_SILU); else CALL(f16_t, ACT_GELU);
    }
#undef CALL
    return check_launch("glu_bwd_kernel");
}

} // extern "C"
