// Shared device/host helpers for the gfx950 low-precision kernels.
//
// Everything here is written for CDNA4 only: 64-lane wavefronts, OCP FP8
// conversion instructions (v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32), DPP row
// operations for wavefront reductions and 128-bit global memory accesses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>

#include "../../include/primus_turbo_amd.h"

namespace pt {

// ---------------------------------------------------------------------------
// Host-side error plumbing (thread-local message, negative status codes)
// ---------------------------------------------------------------------------
void set_error(const std::string &msg);
int  fail(int code, const std::string &msg);
int  check_launch(const char *what);

#define PT_REQUIRE(cond, msg)                                                                      \
    do {                                                                                           \
        if (!(cond))                                                                               \
            return ::pt::fail(PT_ERR_INVALID_ARGUMENT, std::string(__func__) + ": " + (msg));      \
    } while (0)

int device_cu_count();

static inline int64_t cdiv(int64_t a, int64_t b) {
    return (a + b - 1) / b;
}

static inline bool is_hp_dtype(int d) {
    return d == PT_DTYPE_BF16 || d == PT_DTYPE_F16 || d == PT_DTYPE_F32;
}
static inline bool is_fp8_dtype(int d) {
    return d == PT_DTYPE_E4M3 || d == PT_DTYPE_E5M2;
}
static inline float fp8_max_of(int d) {
    return d == PT_DTYPE_E4M3 ? 448.0f : 57344.0f;
}
static inline bool aligned_to(const void *p, uintptr_t a) {
    return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

// ---------------------------------------------------------------------------
// Element types
// ---------------------------------------------------------------------------
struct bf16_t {
    uint16_t bits;
};
struct f16_t {
    _Float16 v;
};

template <typename T> struct HP; // high-precision element traits
template <> struct HP<bf16_t> {
    static __device__ __forceinline__ float to_f32(bf16_t x) {
        return __uint_as_float(static_cast<uint32_t>(x.bits) << 16);
    }
    // round-to-nearest-even in hardware (v_cvt_pk_bf16_f32), NaN stays NaN
    static __device__ __forceinline__ bf16_t from_f32(float f) {
        bf16_t r;
        r.bits = __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
        return r;
    }
};
template <> struct HP<f16_t> {
    static __device__ __forceinline__ float to_f32(f16_t x) { return static_cast<float>(x.v); }
    static __device__ __forceinline__ f16_t from_f32(float f) {
        f16_t r;
        r.v = static_cast<_Float16>(f);
        return r;
    }
};
template <> struct HP<float> {
    static __device__ __forceinline__ float to_f32(float x) { return x; }
    static __device__ __forceinline__ float from_f32(float f) { return f; }
};

// ---------------------------------------------------------------------------
// FP8 (OCP) conversions. `E5M2` selects the bf8 instruction.
// The value must already be clamped to the finite range: the converter rounds
// to nearest even and a value above the largest finite code would become NaN.
// ---------------------------------------------------------------------------
template <bool E5M2>
__device__ __forceinline__ uint32_t cvt_pk_fp8(float a, float b, uint32_t old, bool hi) {
    if constexpr (E5M2) {
        return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true)
                  : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
    } else {
        return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true)
                  : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
    }
}

// four floats -> four fp8 bytes in one dword (byte i = value i)
template <bool E5M2>
__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
    uint32_t w = cvt_pk_fp8<E5M2>(a, b, 0u, false);
    return cvt_pk_fp8<E5M2>(c, d, w, true);
}

// y = clamp(x * scale, -qmax, qmax); NaN maps to +qmax (fminf drops the NaN).
__device__ __forceinline__ float scale_clamp(float x, float scale, float qmax) {
    return fmaxf(fminf(x * scale, qmax), -qmax);
}

template <bool E5M2> __device__ __forceinline__ float fp8_to_f32(uint32_t word, int byte) {
    // byte select must be an immediate
    if constexpr (E5M2) {
        switch (byte) {
        case 0: return __builtin_amdgcn_cvt_f32_bf8(word, 0);
        case 1: return __builtin_amdgcn_cvt_f32_bf8(word, 1);
        case 2: return __builtin_amdgcn_cvt_f32_bf8(word, 2);
        default: return __builtin_amdgcn_cvt_f32_bf8(word, 3);
        }
    } else {
        switch (byte) {
        case 0: return __builtin_amdgcn_cvt_f32_fp8(word, 0);
        case 1: return __builtin_amdgcn_cvt_f32_fp8(word, 1);
        case 2: return __builtin_amdgcn_cvt_f32_fp8(word, 2);
        default: return __builtin_amdgcn_cvt_f32_fp8(word, 3);
        }
    }
}

// ---------------------------------------------------------------------------
// Wavefront reductions on DPP (no LDS traffic). Values are non-negative
// floats (abs-max), so the exchange order never matters.
// ---------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return __uint_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_uint(v), CTRL, 0xf, 0xf, true));
}

// max over each aligned group of 16 lanes (one DPP row); every lane gets it.
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));  // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_f32<0x4E>(v));  // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_f32<0x141>(v)); // row_half_mirror
    v = fmaxf(v, dpp_f32<0x140>(v)); // row_mirror
    return v;
}

// max over aligned groups of 8 lanes; every lane gets it.
__device__ __forceinline__ float lane8_max(float v) {
    v = fmaxf(v, dpp_f32<0xB1>(v));
    v = fmaxf(v, dpp_f32<0x4E>(v));
    v = fmaxf(v, dpp_f32<0x141>(v));
    return v;
}

// max over the whole 64-lane wavefront, returned uniformly.
__device__ __forceinline__ float wave_max(float v) {
    v        = row16_max(v);
    float r0 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 0));
    float r1 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 16));
    float r2 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 32));
    float r3 = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Block-wide max of non-negative floats; `smem` holds >= blockDim/64 floats.
// All threads return the result.
__device__ __forceinline__ float block_max(float v, float *smem) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nw   = (blockDim.x + 63) >> 6;
    v              = wave_max(v);
    __syncthreads();
    if (lane == 0)
        smem[wave] = v;
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < nw; ++i)
        r = fmaxf(r, smem[i]);
    return r;
}

// ---------------------------------------------------------------------------
// The group g with offs[g] <= pos < offs[g + 1] (offs ascending, G + 1 entries; empty groups are
// never returned; 0 when no group holds pos). Every lane of the calling wavefront must take part;
// lane i looks at group i (+ 64, + 128, ...), so the offsets arrive in one round trip per 64
// groups instead of one per group.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int find_group(const int64_t *__restrict__ offs, int G, int64_t pos) {
    const int lane = threadIdx.x & 63;
    int       g    = 0;
    for (int base = 0; base < G; base += 64) {
        const int  i   = base + lane;
        const bool hit = i < G && pos >= offs[i < G ? i : 0] && pos < offs[i < G ? i + 1 : 1];
        const unsigned long long m = __ballot(hit);
        if (m != 0)
            g = base + __builtin_ctzll(m);
    }
    return __builtin_amdgcn_readfirstlane(g);
}

// ---------------------------------------------------------------------------
// Tile order of the tiled quantizers. Workgroups go to the eight XCDs (each with its own L2)
// round-robin in launch order. The tile grid (gridDim.x by gridDim.y, per blockIdx.z) is walked
// in blocks of 8 x 8 tiles, and in every aligned run of 512 workgroups each XCD gets one whole
// block: the 4-byte scale words of eight tiles side by side or on top of each other then fill
// whole 32-byte units in one L2 instead of leaving eight L2s as masked partial writes. Grids
// that are no multiple of 8 tiles in a direction keep the launch order, with eight tiles of a
// row per XCD where that fits.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void xcd_block_tile(uint32_t &tile_x, uint32_t &tile_y) {
    const uint32_t gx = gridDim.x, gy = gridDim.y, per_z = gx * gy;
    const uint32_t wg0 = blockIdx.y * gx + blockIdx.x;
    tile_x = blockIdx.x;
    tile_y = blockIdx.y;
    if ((gx & 7) == 0 && (gy & 7) == 0) {
        uint32_t blk = wg0 >> 6, j = wg0 & 63;
        if ((wg0 | 511u) < per_z) {
            const uint32_t r = wg0 & 511u;
            blk              = ((wg0 >> 9) << 3) + (r & 7u);
            j                = r >> 3;
        }
        const uint32_t nbx = gx >> 3;
        tile_x             = (blk % nbx) * 8 + (j & 7u);
        tile_y             = (blk / nbx) * 8 + (j >> 3);
    } else if ((gx & 7) == 0 && (wg0 | 63u) < per_z) {
        const uint32_t t = (wg0 & ~63u) + ((wg0 & 7u) << 3) + ((wg0 >> 3) & 7u);
        tile_x           = t % gx;
        tile_y           = t / gx;
    }
}

// ---------------------------------------------------------------------------
// 128-bit global memory helpers
// ---------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ u32x4 ld128(const void *p) {
    return *reinterpret_cast<const u32x4 *>(p);
}
__device__ __forceinline__ void st128(void *p, u32x4 v) {
    *reinterpret_cast<u32x4 *>(p) = v;
}
// streaming store: output is not re-read by this kernel
__device__ __forceinline__ void st128_nt(void *p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ void st64_nt(void *p, u32x2 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(p));
}
__device__ __forceinline__ void st32_nt(void *p, uint32_t v) {
    __builtin_nontemporal_store(v, reinterpret_cast<uint32_t *>(p));
}
// streaming load: input is read once by this kernel
__device__ __forceinline__ u32x4 ld128_nt(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

__device__ __forceinline__ float bf16lo(uint32_t w) {
    return __uint_as_float(w << 16);
}
__device__ __forceinline__ float bf16hi(uint32_t w) {
    return __uint_as_float(w & 0xffff0000u);
}

// unpack two packed 16-bit elements of type T from one dword
template <typename T> __device__ __forceinline__ void unpack2(uint32_t w, float &a, float &b);
template <> __device__ __forceinline__ void unpack2<bf16_t>(uint32_t w, float &a, float &b) {
    a = bf16lo(w);
    b = bf16hi(w);
}
template <> __device__ __forceinline__ void unpack2<f16_t>(uint32_t w, float &a, float &b) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2               h = __builtin_bit_cast(h2, w);
    a                = static_cast<float>(h.x);
    b                = static_cast<float>(h.y);
}

template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
    typedef float  f2 __attribute__((ext_vector_type(2)));
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, b2));
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
    typedef float    f2 __attribute__((ext_vector_type(2)));
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f2{a, b}, h2));
}

} // namespace pt
