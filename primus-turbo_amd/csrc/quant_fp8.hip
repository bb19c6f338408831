// FP8 tensorwise and rowwise quantize / dequantize for gfx950.
//
// Numerics follow Primus-Turbo's device quantizer
// (csrc/include/primus_turbo/device/quant_utils.cuh:33-74,
//  csrc/kernels/quantization/quantization_tensorwise.cu:51-154,
//  csrc/kernels/quantization/quantization_rowwise.cu:59-503):
//   scale = qmax / max(amax, 1e-12), scale_inv = 1.0f / scale,
//   q = fp8_rne(clamp(float(x) * scale, -qmax, qmax)), y = T(float(q) * scale_inv).
// The launch structure is this library's own: the tensorwise quantizer is one
// persistent launch whose workgroups park their slice of x in VGPRs while the
// amax crosses the grid, so HBM sees x exactly once.
#include "pt_common.h"

#include <mutex>

// Timing probes for kernel development: a test translation unit may define this macro to record
// timestamps; in the library it expands to nothing.
#ifndef PT_TW_TRACE_POINT
#define PT_TW_TRACE_POINT(id)
#endif

namespace pt {

// ===========================================================================
// Tensorwise quantize: fused amax + scale + cast
// ===========================================================================
constexpr int TW_THREADS = 1024;
constexpr int TW_VEC     = 16; // elements per thread per unit (16 fp8 bytes = one 128-bit store)

// Grid-wide abs-max exchange without read-modify-write atomics (same-address
// device-scope atomics serialise at ~12 ns each on this part, far too slow for a
// 256-workgroup launch). Workspace layout, in 64-bit words (zero-filled before its
// first use, maintained by the kernels from then on):
//   [WS_GEN]       generation g: the tag of the last launch that completed its exchange
//   [WS_GAVE_UP]   tag of the last launch in which a workgroup gave up waiting
//   [WS_SLOTS + b] slot of workgroup b: (tag << 32) | abs-max bits
// A launch takes tag = g + 1 (never 0). Thread 0 of every workgroup reads g BEFORE it
// publishes (the published word depends on the value read, so the two cannot swap); it asks
// for g when the kernel starts (grid_generation), so that this round trip passes under the loads
// of the tensor, and hands the tag to its workgroup through LDS; wavefront 0 then polls the slots of all
// workgroups until each carries the tag. Slots of earlier launches carry older tags and
// need no clearing; workgroup 0 zeroes the slots this launch does not use, so a stale tag
// can never be 2^32 launches old. Workgroup 0 stores g = tag once its own poll is over,
// i.e. after every workgroup has read the old g. Successive launches that share a
// workspace must be ordered (one stream, or a graph's dependencies).
constexpr int WS_GEN = 0, WS_GAVE_UP = 1, WS_SLOTS = 8, WS_MAX_BLOCKS = 1024;
constexpr int WS_WORDS = WS_SLOTS + WS_MAX_BLOCKS;
// Probe bound of the poll (each probe sleeps ~64 cycles plus one memory round trip).
// Every workgroup of the launch is resident (grid <= CU count, one workgroup per
// CU), so the wait normally ends within microseconds; the bound only guarantees that
// every wave exits even if residency is broken by something outside this library (CU
// masking, a long kernel of another stream holding the CUs). A workgroup that gives up
// raises *status (when given) and WS_GAVE_UP; workgroup 0 then writes NaN into scale_inv,
// so the failure travels with the data: everything de-quantized from it is NaN.
constexpr uint32_t GRID_WAIT_MAX_PROBES = 1u << 21;
// Wavefronts of a workgroup that poll, and how far each starts behind the one before (units of
// s_sleep, 64 clocks). Measured on a 4096 x 4096 launch: one wavefront 14.5 us, two 1280 clocks
// apart 13.1, two 640 apart 13.7, four 640 apart 14.6, eight 320 apart 15.3 (more probes in
// flight delay the slots they wait for).
constexpr int GRID_POLL_WAVES = 2, GRID_POLL_STEP = 20;

struct GridWait {
    uint64_t *ws;         // workspace words
    int32_t  *status;     // optional device word, set to 1 by every workgroup that gives up
    uint32_t  max_probes; // probe bound
    uint32_t  wait_for;   // number of slots to wait for (the grid size; tests pass more)
};

// The generation word as thread 0 sees it when the kernel starts (other threads: 0, not used).
// The launch that wrote it has completed (launches that share a workspace are ordered), and
// workgroup 0 of this launch replaces it only after every workgroup has published, i.e. used it.
__device__ __forceinline__ uint32_t grid_generation(const GridWait &gw) {
    return threadIdx.x == 0
               ? static_cast<uint32_t>(__hip_atomic_load(&gw.ws[WS_GEN], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
               : 0u;
}

// Returns the grid-wide abs-max; g = grid_generation() of this launch. s_tag[1] != 0 afterwards
// when this workgroup's poll ended at the probe bound (the value returned is then only a partial
// maximum) or, in workgroup 0, when any workgroup of the launch is known to have given up.
__device__ __forceinline__ float grid_max_exchange(float block_amax, uint32_t g, const GridWait &gw,
                                                   float *s_red, uint32_t *s_tag) {
    uint64_t *slots = gw.ws + WS_SLOTS;
    if (threadIdx.x == 0) {
        const uint32_t tag = (g + 1u == 0u) ? 1u : g + 1u;
        s_tag[0]           = tag;
        s_tag[1]           = 0u;
        s_tag[2]           = 0u;
        __hip_atomic_store(&slots[blockIdx.x],
                           (static_cast<uint64_t>(tag) << 32) | __float_as_uint(block_amax),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const uint32_t tag = s_tag[0];
    if (blockIdx.x == 0)
        for (uint32_t t = gw.wait_for + threadIdx.x; t < WS_MAX_BLOCKS; t += blockDim.x)
            slots[t] = 0ull;
    float v = 0.f;
    if (threadIdx.x < 64 * GRID_POLL_WAVES) {
        // GRID_POLL_WAVES wavefronts poll, each a part of a round trip behind the one before, so
        // that a slot that arrives just after a probe has left is seen by the next wavefront's
        // probe instead of a whole round trip later. A lane takes four slots, 64 apart, and
        // requests them together (one memory round trip per round of probes, not four in a row;
        // each of the four requests of the wavefront covers 512 consecutive bytes).
        // The first wavefront that has seen every slot raises s_tag[2] and the others stop: what
        // they have seen so far are valid amax values and join the block's maximum.
        for (uint32_t i = 0; i < (threadIdx.x >> 6); ++i)
            __builtin_amdgcn_s_sleep(GRID_POLL_STEP);
        const uint32_t lane = threadIdx.x & 63;
        bool           bad = false, whole = true; // whole: this lane has seen all of its slots tagged
        for (uint32_t base = 0; base < gw.wait_for; base += 256) {
            const uint32_t t0     = base + lane;
            uint32_t       probes = 0;
            uint64_t       w[4];
            while (true) {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    w[k] = t0 + 64 * k < gw.wait_for
                               ? __hip_atomic_load(&slots[t0 + 64 * k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                               : static_cast<uint64_t>(tag) << 32;
                bool all = true;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    all = all && static_cast<uint32_t>(w[k] >> 32) == tag;
                if (all)
                    break;
                if (__hip_atomic_load(&s_tag[2], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0u) {
                    whole = false; // another wavefront has the whole picture
                    break;
                }
                if (++probes >= gw.max_probes) {
                    whole = false;
                    bad   = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (static_cast<uint32_t>(w[k] >> 32) == tag) // (a slot that never arrived contributes nothing)
                    v = fmaxf(v, __uint_as_float(static_cast<uint32_t>(w[k]) & 0x7fffffffu));
        }
        if (__all(whole) && lane == 0)
            __hip_atomic_store(&s_tag[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (bad)
            s_tag[1] = 1u; // same value from every lane that writes
    }
    v = block_max(v, s_red);
    if (threadIdx.x == 0) {
        if (s_tag[1] != 0u) {
            __hip_atomic_store(&gw.ws[WS_GAVE_UP], static_cast<uint64_t>(tag), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            if (gw.status != nullptr)
                __hip_atomic_store(gw.status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (blockIdx.x == 0) {
            // a workgroup that started late (after one that gave up had left) can find every
            // slot published although others quantized with a partial maximum: look at the flag
            if (static_cast<uint32_t>(__hip_atomic_load(&gw.ws[WS_GAVE_UP], __ATOMIC_RELAXED,
                                                        __HIP_MEMORY_SCOPE_AGENT)) == tag)
                s_tag[1] = 1u;
            __hip_atomic_store(&gw.ws[WS_GEN], static_cast<uint64_t>(tag), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    return v;
}

// Register image of one 16-element unit.
template <typename T> struct Unit16 {
    static constexpr int DW = 16 * sizeof(T) / 4; // 8 dwords (16-bit) or 16 dwords (fp32)
    u32x4                v[DW / 4];

    __device__ __forceinline__ void load(const T *p) {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i)
            v[i] = ld128(reinterpret_cast<const char *>(p) + 16 * i);
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i)
            v[i] = u32x4{0, 0, 0, 0};
    }
    __device__ __forceinline__ void get(float (&f)[16]) const {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f[4 * i + 0] = __uint_as_float(v[i].x);
                f[4 * i + 1] = __uint_as_float(v[i].y);
                f[4 * i + 2] = __uint_as_float(v[i].z);
                f[4 * i + 3] = __uint_as_float(v[i].w);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                unpack2<T>(v[i].x, f[8 * i + 0], f[8 * i + 1]);
                unpack2<T>(v[i].y, f[8 * i + 2], f[8 * i + 3]);
                unpack2<T>(v[i].z, f[8 * i + 4], f[8 * i + 5]);
                unpack2<T>(v[i].w, f[8 * i + 6], f[8 * i + 7]);
            }
        }
    }
    __device__ __forceinline__ float amax() const {
        float f[16];
        get(f);
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i)
            m = fmaxf(m, fabsf(f[i]));
        return m;
    }
    template <bool E5M2> __device__ __forceinline__ u32x4 quant(float scale, float qmax) const {
        float f[16];
        get(f);
#pragma unroll
        for (int i = 0; i < 16; ++i)
            f[i] = scale_clamp(f[i], scale, qmax);
        u32x4 o;
        o.x = cvt4_fp8<E5M2>(f[0], f[1], f[2], f[3]);
        o.y = cvt4_fp8<E5M2>(f[4], f[5], f[6], f[7]);
        o.z = cvt4_fp8<E5M2>(f[8], f[9], f[10], f[11]);
        o.w = cvt4_fp8<E5M2>(f[12], f[13], f[14], f[15]);
        return o;
    }
};

template <bool E5M2> __device__ __forceinline__ uint8_t quant1(float x, float scale, float qmax) {
    const float v = scale_clamp(x, scale, qmax);
    return static_cast<uint8_t>(cvt_pk_fp8<E5M2>(v, v, 0u, false) & 0xffu);
}

// VEC16 = true : x and q are 16-byte aligned; 128-bit accesses, RET units per
//                thread stay in registers between the amax pass and the cast.
// VEC16 = false: arbitrary alignment, scalar accesses, x re-read after the exchange.
// DYNAMIC = false: scale comes from scale_in, no amax pass and no grid exchange.
template <typename T, bool E5M2, bool VEC16, bool DYNAMIC, int RET>
__global__ __launch_bounds__(TW_THREADS) void quant_tensorwise_kernel(
    const T *__restrict__ x, uint8_t *__restrict__ q, const int64_t n,
    const float *__restrict__ scale_in, float *__restrict__ scale_inv_out, const GridWait gw,
    const float qmax) {
    __shared__ float    s_red[TW_THREADS / 64];
    __shared__ uint32_t s_tag[3];
    const int64_t    stride = static_cast<int64_t>(gridDim.x) * TW_THREADS;
    const int64_t    tid0   = static_cast<int64_t>(blockIdx.x) * TW_THREADS + threadIdx.x;

    PT_TW_TRACE_POINT(0);
    [[maybe_unused]] uint32_t gen = 0u;
    if constexpr (DYNAMIC)
        gen = grid_generation(gw);
    if constexpr (VEC16) {
        const int64_t units = n / TW_VEC;
        const int64_t tail0 = units * TW_VEC; // first element of the scalar tail
        Unit16<T>     held[RET > 0 ? RET : 1];
        float         amax = 0.f;
        if constexpr (DYNAMIC) {
#pragma unroll
            for (int it = 0; it < RET; ++it) {
                const int64_t u = tid0 + it * stride;
                if (u < units)
                    held[it].load(x + u * TW_VEC);
                else
                    held[it].zero();
            }
#pragma unroll
            for (int it = 0; it < RET; ++it)
                amax = fmaxf(amax, held[it].amax());
            for (int64_t u = tid0 + RET * stride; u < units; u += stride) {
                Unit16<T> t;
                t.load(x + u * TW_VEC);
                amax = fmaxf(amax, t.amax());
            }
            if (blockIdx.x == 0 && tail0 + threadIdx.x < n)
                amax = fmaxf(amax, fabsf(HP<T>::to_f32(x[tail0 + threadIdx.x])));
            amax = block_max(amax, s_red);
            PT_TW_TRACE_POINT(1);
            amax = grid_max_exchange(amax, gen, gw, s_red, s_tag);
            PT_TW_TRACE_POINT(2);
        }
        float scale;
        if constexpr (DYNAMIC)
            scale = qmax / fmaxf(amax, 1e-12f);
        else
            scale = scale_in[0];
        if (tid0 == 0)
            scale_inv_out[0] = (DYNAMIC && s_tag[1] != 0u) ? __builtin_nanf("") : 1.0f / scale;

        if constexpr (DYNAMIC) {
#pragma unroll
            for (int it = 0; it < RET; ++it) {
                const int64_t u = tid0 + it * stride;
                if (u < units) // (streaming stores: 13.1 -> 11.3 us at 4096 x 4096; streaming loads cost 0.8 us)
                    st128_nt(q + u * TW_VEC, held[it].template quant<E5M2>(scale, qmax));
            }
        }
        for (int64_t u = tid0 + (DYNAMIC ? RET : 0) * stride; u < units; u += stride) {
            Unit16<T> t;
            t.load(x + u * TW_VEC);
            st128_nt(q + u * TW_VEC, t.template quant<E5M2>(scale, qmax));
        }
        if (blockIdx.x == 0 && tail0 + threadIdx.x < n)
            q[tail0 + threadIdx.x] =
                quant1<E5M2>(HP<T>::to_f32(x[tail0 + threadIdx.x]), scale, qmax);
        PT_TW_TRACE_POINT(3);
    } else {
        float amax = 0.f;
        if constexpr (DYNAMIC) {
            for (int64_t i = tid0; i < n; i += stride)
                amax = fmaxf(amax, fabsf(HP<T>::to_f32(x[i])));
            amax = block_max(amax, s_red);
            amax = grid_max_exchange(amax, gen, gw, s_red, s_tag);
        }
        float scale;
        if constexpr (DYNAMIC)
            scale = qmax / fmaxf(amax, 1e-12f);
        else
            scale = scale_in[0];
        if (tid0 == 0)
            scale_inv_out[0] = (DYNAMIC && s_tag[1] != 0u) ? __builtin_nanf("") : 1.0f / scale;
        for (int64_t i = tid0; i < n; i += stride)
            q[i] = quant1<E5M2>(HP<T>::to_f32(x[i]), scale, qmax);
    }
}

template <typename T, bool E5M2>
static int launch_quant_tensorwise(const void *x, int64_t n, void *q, const float *scale_in,
                                   float *scale_inv, uint64_t *ws, int32_t *status,
                                   uint32_t max_probes, int64_t phantom_blocks, hipStream_t stream) {
    constexpr int RET   = 4;
    const float   qmax  = E5M2 ? 57344.0f : 448.0f;
    const bool    vec   = aligned_to(x, 16) && aligned_to(q, 16);
    const int     cus   = device_cu_count();
    const int64_t units = vec ? n / TW_VEC : n;
    int64_t       grid  = cdiv(units, TW_THREADS);
    if (grid < 1)
        grid = 1;
    if (grid > cus)
        grid = cus; // one workgroup per CU: all of them are resident at the grid exchange
    if (grid > WS_MAX_BLOCKS)
        grid = WS_MAX_BLOCKS;
    if (grid + phantom_blocks > WS_MAX_BLOCKS)
        return fail(PT_ERR_INVALID_ARGUMENT, "quant_tensorwise: phantom_blocks exceeds the slot count");
    const T       *xp = static_cast<const T *>(x);
    auto          *qp = static_cast<uint8_t *>(q);
    dim3           g(static_cast<unsigned>(grid)), b(TW_THREADS);
    const GridWait gw{ws, status, max_probes ? max_probes : GRID_WAIT_MAX_PROBES,
                      static_cast<uint32_t>(grid + phantom_blocks)};
    if (scale_in == nullptr) {
        if (vec)
            quant_tensorwise_kernel<T, E5M2, true, true, RET>
                <<<g, b, 0, stream>>>(xp, qp, n, nullptr, scale_inv, gw, qmax);
        else
            quant_tensorwise_kernel<T, E5M2, false, true, 0>
                <<<g, b, 0, stream>>>(xp, qp, n, nullptr, scale_inv, gw, qmax);
    } else {
        // no grid exchange: oversubscribe the CUs for latency hiding
        const int64_t full = cdiv(units, TW_THREADS);
        int64_t       gg   = full < 1 ? 1 : (full > 8L * cus ? 8L * cus : full);
        dim3          g2(static_cast<unsigned>(gg));
        if (vec)
            quant_tensorwise_kernel<T, E5M2, true, false, 0>
                <<<g2, b, 0, stream>>>(xp, qp, n, scale_in, scale_inv, gw, qmax);
        else
            quant_tensorwise_kernel<T, E5M2, false, false, 0>
                <<<g2, b, 0, stream>>>(xp, qp, n, scale_in, scale_inv, gw, qmax);
    }
    return check_launch("quant_tensorwise_kernel");
}

// ---------------------------------------------------------------------------
// Two-launch form of the tensorwise quantizer: per-workgroup abs-max into `partial`, then a
// second launch in which every workgroup takes the maximum of all partials, forms the scale and
// casts. No workgroup waits for another, so nothing depends on the launch being resident as a
// whole (other streams may hold CUs, CU masks, HIP-graph replays beside eager work), at the
// price of reading x twice (the second read finds a tensor of this size in the caches). The
// launch structure of Primus-Turbo's own op (csrc/pytorch/quantization/quantization.cpp:44-90:
// reduce, compute scale, cast) with the scale computation folded into the cast.
// `partial` needs no clearing: launch 1 writes every word that launch 2 reads.
// ---------------------------------------------------------------------------
template <typename T, bool VEC16>
__global__ __launch_bounds__(TW_THREADS) void tw_partial_amax_kernel(const T *__restrict__ x, const int64_t n,
                                                                     float *__restrict__ partial) {
    __shared__ float s_red[TW_THREADS / 64];
    const int64_t    stride = static_cast<int64_t>(gridDim.x) * TW_THREADS;
    const int64_t    tid0   = static_cast<int64_t>(blockIdx.x) * TW_THREADS + threadIdx.x;
    float            amax   = 0.f;
    if constexpr (VEC16) {
        const int64_t units = n / TW_VEC;
        const int64_t tail0 = units * TW_VEC;
        constexpr int UNR   = 4; // loads requested together
        int64_t       u     = tid0;
        for (; u + (UNR - 1) * stride < units; u += UNR * stride) {
            Unit16<T> t[UNR];
#pragma unroll
            for (int k = 0; k < UNR; ++k)
                t[k].load(x + (u + k * stride) * TW_VEC);
#pragma unroll
            for (int k = 0; k < UNR; ++k)
                amax = fmaxf(amax, t[k].amax());
        }
        for (; u < units; u += stride) {
            Unit16<T> t;
            t.load(x + u * TW_VEC);
            amax = fmaxf(amax, t.amax());
        }
        if (blockIdx.x == 0 && tail0 + threadIdx.x < n)
            amax = fmaxf(amax, fabsf(HP<T>::to_f32(x[tail0 + threadIdx.x])));
    } else {
        for (int64_t i = tid0; i < n; i += stride)
            amax = fmaxf(amax, fabsf(HP<T>::to_f32(x[i])));
    }
    amax = block_max(amax, s_red);
    if (threadIdx.x == 0)
        partial[blockIdx.x] = amax;
}

template <typename T, bool E5M2, bool VEC16>
__global__ __launch_bounds__(TW_THREADS) void tw_cast_from_partials_kernel(
    const T *__restrict__ x, uint8_t *__restrict__ q, const int64_t n, const float *__restrict__ partial,
    const int nparts, float *__restrict__ scale_inv_out, const float qmax) {
    __shared__ float s_red[TW_THREADS / 64];
    const int64_t    stride = static_cast<int64_t>(gridDim.x) * TW_THREADS;
    const int64_t    tid0   = static_cast<int64_t>(blockIdx.x) * TW_THREADS + threadIdx.x;
    float            amax   = 0.f;
    for (int t = threadIdx.x; t < nparts; t += TW_THREADS)
        amax = fmaxf(amax, partial[t]);
    amax              = block_max(amax, s_red);
    const float scale = qmax / fmaxf(amax, 1e-12f);
    if (tid0 == 0)
        scale_inv_out[0] = 1.0f / scale;
    if constexpr (VEC16) {
        const int64_t units = n / TW_VEC;
        const int64_t tail0 = units * TW_VEC;
        for (int64_t u = tid0; u < units; u += stride) {
            Unit16<T> t;
            t.load(x + u * TW_VEC);
            st128_nt(q + u * TW_VEC, t.template quant<E5M2>(scale, qmax));
        }
        if (blockIdx.x == 0 && tail0 + threadIdx.x < n)
            q[tail0 + threadIdx.x] = quant1<E5M2>(HP<T>::to_f32(x[tail0 + threadIdx.x]), scale, qmax);
    } else {
        for (int64_t i = tid0; i < n; i += stride)
            q[i] = quant1<E5M2>(HP<T>::to_f32(x[i]), scale, qmax);
    }
}

template <typename T, bool E5M2>
static int launch_quant_tensorwise_two_pass(const void *x, int64_t n, void *q, float *scale_inv, float *partial,
                                            hipStream_t stream) {
    const float   qmax  = E5M2 ? 57344.0f : 448.0f;
    const bool    vec   = aligned_to(x, 16) && aligned_to(q, 16);
    const int     cus   = device_cu_count();
    const int64_t units = vec ? n / TW_VEC : n;
    const int64_t full  = cdiv(units, TW_THREADS);
    int64_t       g1    = full < 1 ? 1 : (full > 2L * cus ? 2L * cus : full);
    if (g1 > WS_MAX_BLOCKS)
        g1 = WS_MAX_BLOCKS;
    const int64_t g2 = full < 1 ? 1 : (full > 8L * cus ? 8L * cus : full);
    const T      *xp = static_cast<const T *>(x);
    auto         *qp = static_cast<uint8_t *>(q);
    dim3          b(TW_THREADS);
    if (vec)
        tw_partial_amax_kernel<T, true><<<dim3(static_cast<unsigned>(g1)), b, 0, stream>>>(xp, n, partial);
    else
        tw_partial_amax_kernel<T, false><<<dim3(static_cast<unsigned>(g1)), b, 0, stream>>>(xp, n, partial);
    const int rc = check_launch("tw_partial_amax_kernel");
    if (rc != PT_OK)
        return rc;
    if (vec)
        tw_cast_from_partials_kernel<T, E5M2, true>
            <<<dim3(static_cast<unsigned>(g2)), b, 0, stream>>>(xp, qp, n, partial, static_cast<int>(g1), scale_inv, qmax);
    else
        tw_cast_from_partials_kernel<T, E5M2, false>
            <<<dim3(static_cast<unsigned>(g2)), b, 0, stream>>>(xp, qp, n, partial, static_cast<int>(g1), scale_inv, qmax);
    return check_launch("tw_cast_from_partials_kernel");
}

// y[8 u .. 8 u + 7] = T(fp8(q[8 u ..]) * s) for the pieces u = first, first + step, ... below
// `units`: 8 code bytes in, 16 or 32 bytes out per lane (whole lines per wavefront on both sides),
// four pieces per round requested together, streaming accesses (nothing here is read twice).
template <typename T, bool E5M2>
__device__ __forceinline__ void dequant_pieces8(const uint8_t *__restrict__ q, T *__restrict__ y, const float s,
                                                const int64_t first, const int64_t step, const int64_t units) {
    for (int64_t u0 = first; u0 < units; u0 += 4 * step) {
        u32x2 w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t u = u0 + k * step;
            w[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(q + 8 * (u < units ? u : u0)));
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t u = u0 + k * step;
            if (u >= units)
                break;
            const uint32_t ww[2] = {w[k].x, w[k].y};
            float          f[8];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f[4 * i + 0] = fp8_to_f32<E5M2>(ww[i], 0) * s;
                f[4 * i + 1] = fp8_to_f32<E5M2>(ww[i], 1) * s;
                f[4 * i + 2] = fp8_to_f32<E5M2>(ww[i], 2) * s;
                f[4 * i + 3] = fp8_to_f32<E5M2>(ww[i], 3) * s;
            }
            char *dst = reinterpret_cast<char *>(y + u * 8);
            if constexpr (sizeof(T) == 4) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    st128_nt(dst + 16 * i, u32x4{__float_as_uint(f[4 * i]), __float_as_uint(f[4 * i + 1]),
                                                 __float_as_uint(f[4 * i + 2]), __float_as_uint(f[4 * i + 3])});
            } else {
                st128_nt(dst, u32x4{pack2<T>(f[0], f[1]), pack2<T>(f[2], f[3]), pack2<T>(f[4], f[5]), pack2<T>(f[6], f[7])});
            }
        }
    }
}

// ===========================================================================
// Tensorwise dequantize
// ===========================================================================
template <typename T, bool E5M2, bool VEC16>
__global__ __launch_bounds__(256) void dequant_tensorwise_kernel(
    const uint8_t *__restrict__ q, T *__restrict__ y, const int64_t n,
    const float *__restrict__ scale_inv_ptr) {
    const float   s      = scale_inv_ptr[0];
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int64_t tid0   = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if constexpr (VEC16) {
        const int64_t units = n / 8;
        dequant_pieces8<T, E5M2>(q, y, s, tid0, stride, units);
        const int64_t tail0 = units * 8;
        if (blockIdx.x == 0 && tail0 + threadIdx.x < n)
            y[tail0 + threadIdx.x] =
                HP<T>::from_f32(fp8_to_f32<E5M2>(q[tail0 + threadIdx.x], 0) * s);
    } else {
        for (int64_t i = tid0; i < n; i += stride)
            y[i] = HP<T>::from_f32(fp8_to_f32<E5M2>(q[i], 0) * s);
    }
}

template <typename T, bool E5M2>
static int launch_dequant_tensorwise(const void *q, int64_t n, const float *scale_inv, void *y,
                                     hipStream_t stream) {
    const bool    vec   = aligned_to(q, 16) && aligned_to(y, 16);
    const int64_t units = vec ? cdiv(n / 8, 4) : n; // work items of a thread: four 8-byte pieces, or one element
    const int     cus   = device_cu_count();
    int64_t       grid  = cdiv(units, 256);
    if (grid < 1)
        grid = 1;
    if (grid > 32L * cus)
        grid = 32L * cus;
    dim3 g(static_cast<unsigned>(grid)), b(256);
    if (vec)
        dequant_tensorwise_kernel<T, E5M2, true><<<g, b, 0, stream>>>(
            static_cast<const uint8_t *>(q), static_cast<T *>(y), n, scale_inv);
    else
        dequant_tensorwise_kernel<T, E5M2, false><<<g, b, 0, stream>>>(
            static_cast<const uint8_t *>(q), static_cast<T *>(y), n, scale_inv);
    return check_launch("dequant_tensorwise_kernel");
}

// ===========================================================================
// Rowwise (reduced axis contiguous): one workgroup per row, row kept in VGPRs
// ===========================================================================
// Rows up to ROW_HOLD_ELEMS elements are read from HBM once: each thread parks
// up to HOLD 8-element vectors. Longer rows re-read the remainder.
constexpr int RW_THREADS = 256;

template <typename T> struct Vec8 {
    static constexpr int DW = 8 * sizeof(T) / 4; // 4 or 8 dwords
    u32x4                v[DW / 4];
    // (streaming loads: a row is read once, or re-read only when it is longer than the registers hold)
    __device__ __forceinline__ void load(const T *p) {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i)
            v[i] = ld128_nt(reinterpret_cast<const char *>(p) + 16 * i);
    }
    __device__ __forceinline__ void keep_if(bool ok) {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i)
            v[i] = ok ? v[i] : u32x4{0u, 0u, 0u, 0u};
    }
    __device__ __forceinline__ void zero() {
#pragma unroll
        for (int i = 0; i < DW / 4; ++i)
            v[i] = u32x4{0, 0, 0, 0};
    }
    __device__ __forceinline__ void get(float (&f)[8]) const {
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                f[4 * i + 0] = __uint_as_float(v[i].x);
                f[4 * i + 1] = __uint_as_float(v[i].y);
                f[4 * i + 2] = __uint_as_float(v[i].z);
                f[4 * i + 3] = __uint_as_float(v[i].w);
            }
        } else {
            unpack2<T>(v[0].x, f[0], f[1]);
            unpack2<T>(v[0].y, f[2], f[3]);
            unpack2<T>(v[0].z, f[4], f[5]);
            unpack2<T>(v[0].w, f[6], f[7]);
        }
    }
    __device__ __forceinline__ float amax() const {
        float f[8];
        get(f);
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            m = fmaxf(m, fabsf(f[i]));
        return m;
    }
    template <bool E5M2> __device__ __forceinline__ u32x2 quant(float scale, float qmax) const {
        float f[8];
        get(f);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            f[i] = scale_clamp(f[i], scale, qmax);
        u32x2 o;
        o.x = cvt4_fp8<E5M2>(f[0], f[1], f[2], f[3]);
        o.y = cvt4_fp8<E5M2>(f[4], f[5], f[6], f[7]);
        return o;
    }
};

template <typename T, bool E5M2, bool VEC8, bool DYNAMIC, int HOLD>
__global__ __launch_bounds__(RW_THREADS) void quant_rowwise_inner_kernel(
    const T *__restrict__ x, uint8_t *__restrict__ q, const int64_t inner,
    const float *__restrict__ scale_in, float *__restrict__ scale_inv_out, const float qmax) {
    __shared__ float s_red[RW_THREADS / 64];
    const int64_t    row = blockIdx.x;
    const T         *xr  = x + row * inner;
    uint8_t         *qr  = q + row * inner;
    float            scale;
    if constexpr (VEC8) {
        const int64_t units = inner / 8; // inner % 8 == 0 on this path
        Vec8<T>       held[HOLD];
        if constexpr (DYNAMIC) {
            float amax = 0.f;
            // all pieces are requested before the first is used: a piece behind the row's end
            // re-reads the row's first piece and is zeroed (a branch between the loads would
            // make each wait for the one before)
#pragma unroll
            for (int it = 0; it < HOLD; ++it) {
                const int64_t u = threadIdx.x + it * RW_THREADS;
                held[it].load(xr + (u < units ? u : 0) * 8);
            }
#pragma unroll
            for (int it = 0; it < HOLD; ++it) {
                held[it].keep_if(threadIdx.x + it * RW_THREADS < units);
                amax = fmaxf(amax, held[it].amax());
            }
            for (int64_t u = threadIdx.x + HOLD * RW_THREADS; u < units; u += RW_THREADS) {
                Vec8<T> t;
                t.load(xr + u * 8);
                amax = fmaxf(amax, t.amax());
            }
            amax  = block_max(amax, s_red);
            scale = qmax / fmaxf(amax, 1e-12f);
            if (threadIdx.x == 0)
                scale_inv_out[row] = 1.0f / scale;
#pragma unroll
            for (int it = 0; it < HOLD; ++it) {
                const int64_t u = threadIdx.x + it * RW_THREADS;
                if (u < units)
                    st64_nt(qr + u * 8, held[it].template quant<E5M2>(scale, qmax));
            }
        } else {
            scale = scale_in[row];
            if (threadIdx.x == 0)
                scale_inv_out[row] = 1.0f / scale;
        }
        for (int64_t u = threadIdx.x + (DYNAMIC ? HOLD : 0) * RW_THREADS; u < units;
             u += RW_THREADS) {
            Vec8<T> t;
            t.load(xr + u * 8);
            st64_nt(qr + u * 8, t.template quant<E5M2>(scale, qmax));
        }
    } else {
        if constexpr (DYNAMIC) {
            float amax = 0.f;
            for (int64_t i = threadIdx.x; i < inner; i += RW_THREADS)
                amax = fmaxf(amax, fabsf(HP<T>::to_f32(xr[i])));
            amax  = block_max(amax, s_red);
            scale = qmax / fmaxf(amax, 1e-12f);
        } else {
            scale = scale_in[row];
        }
        if (threadIdx.x == 0)
            scale_inv_out[row] = 1.0f / scale;
        for (int64_t i = threadIdx.x; i < inner; i += RW_THREADS)
            qr[i] = quant1<E5M2>(HP<T>::to_f32(xr[i]), scale, qmax);
    }
}

// ===========================================================================
// Rowwise, reduced axis not contiguous: x viewed as [B, M, N], one scale per (b, n)
// ===========================================================================
// Pass 1: column abs-max. A workgroup owns a 64-column strip of one batch and a
// slab of rows; lanes of a wavefront read 64 consecutive columns (coalesced),
// the 4 wavefronts take different rows. Partial maxima meet through an integer
// atomic max on the fp32 bit pattern (amax >= 0), which is order independent.
constexpr int CM_ROWS_PER_BLOCK = 256;

template <typename T>
__global__ __launch_bounds__(256) void colmax_kernel(const T *__restrict__ x, uint32_t *amax_bits,
                                                     const int64_t M, const int64_t N) {
    const int     lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t b    = blockIdx.z;
    const int64_t n    = static_cast<int64_t>(blockIdx.x) * 64 + lane;
    const int64_t m0   = static_cast<int64_t>(blockIdx.y) * CM_ROWS_PER_BLOCK;
    const int64_t m1   = (m0 + CM_ROWS_PER_BLOCK < M) ? m0 + CM_ROWS_PER_BLOCK : M;
    __shared__ float s[4][64];
    float            a = 0.f;
    if (n < N) {
        const T *p = x + b * M * N + n;
        for (int64_t m = m0 + wave; m < m1; m += 4)
            a = fmaxf(a, fabsf(HP<T>::to_f32(p[m * N])));
    }
    s[wave][lane] = a;
    __syncthreads();
    if (wave == 0 && n < N) {
        a = fmaxf(fmaxf(s[0][lane], s[1][lane]), fmaxf(s[2][lane], s[3][lane]));
        __hip_atomic_fetch_max(&amax_bits[b * N + n], __float_as_uint(a), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Pass 2: turn the amax (held in scale_inv's storage as fp32 bits) into
// scale_inv and quantize. Each thread handles 4 consecutive columns of a row.
template <typename T, bool E5M2, bool DYNAMIC>
__global__ __launch_bounds__(256) void quant_rowwise_outer_kernel(
    const T *__restrict__ x, uint8_t *__restrict__ q, const float *__restrict__ amax_or_scale,
    const int64_t M, const int64_t N, const float qmax) {
    const int64_t b  = blockIdx.z;
    const int64_t n  = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const int64_t m0 = static_cast<int64_t>(blockIdx.y) * CM_ROWS_PER_BLOCK;
    const int64_t m1 = (m0 + CM_ROWS_PER_BLOCK < M) ? m0 + CM_ROWS_PER_BLOCK : M;
    if (n >= N)
        return;
    float scale;
    if constexpr (DYNAMIC)
        scale = qmax / fmaxf(amax_or_scale[b * N + n], 1e-12f);
    else
        scale = amax_or_scale[b * N + n];
    const T *p = x + b * M * N + n;
    uint8_t *o = q + b * M * N + n;
    for (int64_t m = m0; m < m1; ++m)
        o[m * N] = quant1<E5M2>(HP<T>::to_f32(p[m * N]), scale, qmax);
}

// amax (or given scale) -> scale_inv, in place or to a separate buffer
template <bool DYNAMIC>
__global__ void finish_scale_inv_kernel(const float *in, float *scale_inv, const int64_t n,
                                        const float qmax) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        float scale;
        if constexpr (DYNAMIC)
            scale = qmax / fmaxf(in[i], 1e-12f);
        else
            scale = in[i];
        scale_inv[i] = 1.0f / scale;
    }
}

__global__ void zero_u32_kernel(uint32_t *p, const int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n)
        p[i] = 0u;
}

template <typename T, bool E5M2>
static int launch_quant_rowwise(const void *x, int64_t B, int64_t M, int64_t N, void *q,
                                const float *scale_in, float *scale_inv, hipStream_t stream) {
    const float qmax = E5M2 ? 57344.0f : 448.0f;
    const T    *xp   = static_cast<const T *>(x);
    auto       *qp   = static_cast<uint8_t *>(q);
    if (B * M * N == 0)
        return PT_OK;
    if (N == 1) {
        // contiguous rows: B rows of M elements
        constexpr int HOLD = sizeof(T) == 4 ? 4 : 8;
        const bool    vec  = (M % 8 == 0) && aligned_to(x, 16) && aligned_to(q, 8);
        dim3          g(static_cast<unsigned>(B)), b(RW_THREADS);
        if (scale_in == nullptr) {
            if (vec)
                quant_rowwise_inner_kernel<T, E5M2, true, true, HOLD>
                    <<<g, b, 0, stream>>>(xp, qp, M, nullptr, scale_inv, qmax);
            else
                quant_rowwise_inner_kernel<T, E5M2, false, true, 1>
                    <<<g, b, 0, stream>>>(xp, qp, M, nullptr, scale_inv, qmax);
        } else {
            if (vec)
                quant_rowwise_inner_kernel<T, E5M2, true, false, 1>
                    <<<g, b, 0, stream>>>(xp, qp, M, scale_in, scale_inv, qmax);
            else
                quant_rowwise_inner_kernel<T, E5M2, false, false, 1>
                    <<<g, b, 0, stream>>>(xp, qp, M, scale_in, scale_inv, qmax);
        }
        return check_launch("quant_rowwise_inner_kernel");
    }
    const int64_t  nscale = B * N;
    const unsigned mslabs = static_cast<unsigned>(cdiv(M, CM_ROWS_PER_BLOCK));
    if (scale_in == nullptr) {
        // scale_inv's storage carries the amax bit patterns between the passes
        auto *bits = reinterpret_cast<uint32_t *>(scale_inv);
        zero_u32_kernel<<<static_cast<unsigned>(cdiv(nscale, 256)), 256, 0, stream>>>(bits, nscale);
        dim3 g1(static_cast<unsigned>(cdiv(N, 64)), mslabs, static_cast<unsigned>(B));
        colmax_kernel<T><<<g1, 256, 0, stream>>>(xp, bits, M, N);
        dim3 g2(static_cast<unsigned>(cdiv(N, 256)), mslabs, static_cast<unsigned>(B));
        quant_rowwise_outer_kernel<T, E5M2, true>
            <<<g2, 256, 0, stream>>>(xp, qp, scale_inv, M, N, qmax);
        finish_scale_inv_kernel<true><<<static_cast<unsigned>(cdiv(nscale, 256)), 256, 0, stream>>>(
            scale_inv, scale_inv, nscale, qmax);
    } else {
        dim3 g2(static_cast<unsigned>(cdiv(N, 256)), mslabs, static_cast<unsigned>(B));
        quant_rowwise_outer_kernel<T, E5M2, false>
            <<<g2, 256, 0, stream>>>(xp, qp, scale_in, M, N, qmax);
        finish_scale_inv_kernel<false><<<static_cast<unsigned>(cdiv(nscale, 256)), 256, 0, stream>>>(
            scale_in, scale_inv, nscale, qmax);
    }
    return check_launch("quant_rowwise_outer_kernel");
}

// ===========================================================================
// Rowwise dequantize: y[b, m, n] = T(float(q[b, m, n]) * scale_inv[b, n])   (N > 1)
//                     y[r, i]    = T(float(q[r, i]) * scale_inv[r])         (N == 1)
// ===========================================================================
template <typename T, bool E5M2>
__global__ __launch_bounds__(256) void dequant_rowwise_kernel(
    const uint8_t *__restrict__ q, T *__restrict__ y, const float *__restrict__ scale_inv,
    const int64_t B, const int64_t M, const int64_t N) {
    const int64_t total  = B * M * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += stride) {
        int64_t sidx;
        if (N == 1) {
            sidx = i / M;
        } else {
            const int64_t n = i % N;
            const int64_t b = i / (M * N);
            sidx            = b * N + n;
        }
        y[i] = HP<T>::from_f32(fp8_to_f32<E5M2>(q[i], 0) * scale_inv[sidx]);
    }
}

// 16 elements per thread when rows are contiguous and 16-aligned
template <typename T, bool E5M2>
__global__ __launch_bounds__(256) void dequant_rowwise_inner_vec_kernel(
    const uint8_t *__restrict__ q, T *__restrict__ y, const float *__restrict__ scale_inv,
    const int64_t inner) {
    const int64_t row   = blockIdx.x;
    const float   s     = scale_inv[row];
    dequant_pieces8<T, E5M2>(q + row * inner, y + row * inner, s, threadIdx.x, 256, inner / 8);
}

template <typename T, bool E5M2>
static int launch_dequant_rowwise(const void *q, int64_t B, int64_t M, int64_t N,
                                  const float *scale_inv, void *y, hipStream_t stream) {
    const int64_t total = B * M * N;
    if (total == 0)
        return PT_OK;
    if (N == 1 && M % 16 == 0 && aligned_to(q, 16) && aligned_to(y, 16)) {
        dequant_rowwise_inner_vec_kernel<T, E5M2><<<static_cast<unsigned>(B), 256, 0, stream>>>(
            static_cast<const uint8_t *>(q), static_cast<T *>(y), scale_inv, M);
        return check_launch("dequant_rowwise_inner_vec_kernel");
    }
    int64_t grid = cdiv(total, 256);
    if (grid > 65536)
        grid = 65536;
    dequant_rowwise_kernel<T, E5M2><<<static_cast<unsigned>(grid), 256, 0, stream>>>(
        static_cast<const uint8_t *>(q), static_cast<T *>(y), scale_inv, B, M, N);
    return check_launch("dequant_rowwise_kernel");
}

// ---------------------------------------------------------------------------
// Static scratch of pt_quantize_fp8_tensorwise_static: the exchange words live in the code
// object's own zero-initialised device memory, so that entry point needs no workspace and
// neither it nor its caller allocates anything. One slot set per stream that has used the
// entry point on the device (calls on one stream are ordered, calls on different streams
// must not share slots), PT_TENSORWISE_STATIC_MAX_STREAMS of them: 66 KB per GPU, held
// until the process ends. A slot set belongs to a stream HANDLE from its first call until
// pt_tensorwise_static_release(stream).
// ---------------------------------------------------------------------------
static __device__ __align__(256) uint64_t tw_scratch[PT_TENSORWISE_STATIC_MAX_STREAMS * WS_WORDS];

// Device address of tw_scratch on the current device (the array's name is only a host-side
// handle; every GPU holds its own copy at its own address) and the slot set of `stream`.
// release = true: give the stream's slot set back instead (out is not written).
static int static_scratch_for(hipStream_t stream, uint64_t **out, bool release = false) {
    constexpr int MAX_DEV = 64;
    struct PerDevice {
        uint64_t   *base = nullptr;
        bool        taken[PT_TENSORWISE_STATIC_MAX_STREAMS]   = {};
        hipStream_t streams[PT_TENSORWISE_STATIC_MAX_STREAMS] = {};
    };
    static PerDevice  table[MAX_DEV];
    static std::mutex mu;
    int               dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV)
        return fail(PT_ERR_LAUNCH, "pt_quantize_fp8_tensorwise_static: no current device");
    std::lock_guard<std::mutex> lock(mu);
    PerDevice                  &pd = table[dev];
    if (pd.base == nullptr) {
        void            *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(tw_scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(PT_ERR_LAUNCH, std::string("pt_quantize_fp8_tensorwise_static: "
                                                   "hipGetSymbolAddress failed: ") +
                                           hipGetErrorString(e));
        pd.base = static_cast<uint64_t *>(p);
    }
    int idx = -1, vacant = -1;
    for (int i = 0; i < PT_TENSORWISE_STATIC_MAX_STREAMS; ++i) {
        if (pd.taken[i] && pd.streams[i] == stream)
            idx = i;
        if (!pd.taken[i] && vacant < 0)
            vacant = i;
    }
    if (release) {
        if (idx >= 0)
            pd.taken[idx] = false; // the words stay as they are: generation tags need no clearing
        return PT_OK;
    }
    if (idx < 0) {
        if (vacant < 0)
            return fail(PT_ERR_WORKSPACE,
                        "pt_quantize_fp8_tensorwise_static: PT_TENSORWISE_STATIC_MAX_STREAMS stream handles "
                        "hold a slot set on this device; release one with pt_tensorwise_static_release, or "
                        "use pt_quantize_fp8_tensorwise with a workspace per stream");
        idx             = vacant;
        pd.taken[idx]   = true;
        pd.streams[idx] = stream;
    }
    *out = pd.base + static_cast<size_t>(idx) * WS_WORDS;
    return PT_OK;
}

// ---------------------------------------------------------------------------
// dtype dispatch
// ---------------------------------------------------------------------------
#define PT_DISPATCH_HP_FP8(hp, fp8, CALL)                                                          \
    do {                                                                                           \
        if (hp == PT_DTYPE_BF16 && fp8 == PT_DTYPE_E4M3) { CALL(bf16_t, false); }                  \
        else if (hp == PT_DTYPE_BF16 && fp8 == PT_DTYPE_E5M2) { CALL(bf16_t, true); }              \
        else if (hp == PT_DTYPE_F16 && fp8 == PT_DTYPE_E4M3) { CALL(f16_t, false); }               \
        else if (hp == PT_DTYPE_F16 && fp8 == PT_DTYPE_E5M2) { CALL(f16_t, true); }                \
        else if (hp == PT_DTYPE_F32 && fp8 == PT_DTYPE_E4M3) { CALL(float, false); }               \
        else { CALL(float, true); }                                                                \
    } while (0)

} // namespace pt

using namespace pt;

extern "C" {

size_t pt_quantize_fp8_tensorwise_workspace_bytes(void) {
    return WS_WORDS * sizeof(uint64_t);
}

static int quantize_fp8_tensorwise_common(const void *x, int x_dtype, int64_t numel, void *q,
                                          int q_dtype, const float *scale_in, float *scale_inv,
                                          uint64_t *ws, int32_t *status, uint32_t max_probes,
                                          int64_t phantom_blocks, hipStream_t st) {
#define CALL(T, E5)                                                                                \
    return launch_quant_tensorwise<T, E5>(x, numel, q, scale_in, scale_inv, ws, status,            \
                                          max_probes, phantom_blocks, st)
    PT_DISPATCH_HP_FP8(x_dtype, q_dtype, CALL);
#undef CALL
}

#define PT_TW_CHECK_ARGS()                                                                         \
    PT_REQUIRE(is_hp_dtype(x_dtype), "input must be bf16, fp16 or fp32");                          \
    PT_REQUIRE(is_fp8_dtype(q_dtype), "output must be e4m3 or e5m2");                              \
    PT_REQUIRE(numel >= 0, "numel must be non-negative");                                          \
    PT_REQUIRE(scale_inv != nullptr, "scale_inv must not be NULL");                                \
    PT_REQUIRE(numel == 0 || (x != nullptr && q != nullptr), "x and q must not be NULL")

int pt_quantize_fp8_tensorwise_ex(const void *x, int x_dtype, int64_t numel, void *q, int q_dtype,
                                  const float *scale_in, float *scale_inv, void *workspace,
                                  size_t workspace_bytes, int32_t *status, uint32_t max_probes,
                                  int64_t phantom_blocks, void *stream) {
    PT_TW_CHECK_ARGS();
    PT_REQUIRE(phantom_blocks >= 0, "phantom_blocks must be non-negative");
    if (scale_in == nullptr) {
        if (workspace == nullptr || workspace_bytes < pt_quantize_fp8_tensorwise_workspace_bytes() ||
            !aligned_to(workspace, 16))
            return fail(PT_ERR_WORKSPACE,
                        "pt_quantize_fp8_tensorwise: workspace missing, too small or misaligned");
    }
    return quantize_fp8_tensorwise_common(x, x_dtype, numel, q, q_dtype, scale_in, scale_inv,
                                          static_cast<uint64_t *>(workspace), status, max_probes,
                                          phantom_blocks, static_cast<hipStream_t>(stream));
}

int pt_quantize_fp8_tensorwise(const void *x, int x_dtype, int64_t numel, void *q, int q_dtype,
                               const float *scale_in, float *scale_inv, void *workspace,
                               size_t workspace_bytes, void *stream) {
    return pt_quantize_fp8_tensorwise_ex(x, x_dtype, numel, q, q_dtype, scale_in, scale_inv,
                                         workspace, workspace_bytes, nullptr, 0, 0, stream);
}

int pt_quantize_fp8_tensorwise_static(const void *x, int x_dtype, int64_t numel, void *q,
                                      int q_dtype, const float *scale_in, float *scale_inv,
                                      int32_t *status, void *stream) {
    PT_TW_CHECK_ARGS();
    PT_REQUIRE(numel <= PT_TENSORWISE_STATIC_MAX_NUMEL,
               "numel exceeds PT_TENSORWISE_STATIC_MAX_NUMEL; use pt_quantize_fp8_tensorwise with a workspace");
    uint64_t *ws = nullptr;
    if (scale_in == nullptr) {
        const int rc = static_scratch_for(static_cast<hipStream_t>(stream), &ws);
        if (rc != PT_OK)
            return rc;
    }
    return quantize_fp8_tensorwise_common(x, x_dtype, numel, q, q_dtype, scale_in, scale_inv, ws,
                                          status, 0, 0, static_cast<hipStream_t>(stream));
}

int pt_tensorwise_static_release(void *stream) {
    uint64_t *unused = nullptr;
    return static_scratch_for(static_cast<hipStream_t>(stream), &unused, true);
}

int pt_quantize_fp8_tensorwise_two_pass(const void *x, int x_dtype, int64_t numel, void *q, int q_dtype,
                                        float *scale_inv, void *workspace, size_t workspace_bytes,
                                        void *stream) {
    PT_TW_CHECK_ARGS();
    if (workspace == nullptr || workspace_bytes < pt_quantize_fp8_tensorwise_workspace_bytes() ||
        !aligned_to(workspace, 16))
        return fail(PT_ERR_WORKSPACE,
                    "pt_quantize_fp8_tensorwise_two_pass: workspace missing, too small or misaligned");
    auto st = static_cast<hipStream_t>(stream);
#define CALL(T, E5)                                                                                \
    return launch_quant_tensorwise_two_pass<T, E5>(x, numel, q, scale_inv,                         \
                                                   static_cast<float *>(workspace), st)
    PT_DISPATCH_HP_FP8(x_dtype, q_dtype, CALL);
#undef CALL
}

int pt_dequantize_fp8_tensorwise(const void *q, int q_dtype, int64_t numel, const float *scale_inv,
                                 void *y, int y_dtype, void *stream) {
    PT_REQUIRE(is_fp8_dtype(q_dtype), "input must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(y_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(numel >= 0, "numel must be non-negative");
    PT_REQUIRE(scale_inv != nullptr, "scale_inv must not be NULL");
    if (numel == 0)
        return PT_OK;
    PT_REQUIRE(q != nullptr && y != nullptr, "q and y must not be NULL");
    auto st = static_cast<hipStream_t>(stream);
#define CALL(T, E5) return launch_dequant_tensorwise<T, E5>(q, numel, scale_inv, y, st)
    PT_DISPATCH_HP_FP8(y_dtype, q_dtype, CALL);
#undef CALL
}

int pt_quantize_fp8_rowwise(const void *x, int x_dtype, int64_t B, int64_t M, int64_t N, void *q,
                            int q_dtype, const float *scale_in, float *scale_inv, void *stream) {
    PT_REQUIRE(is_hp_dtype(x_dtype), "input must be bf16, fp16 or fp32");
    PT_REQUIRE(is_fp8_dtype(q_dtype), "output must be e4m3 or e5m2");
    PT_REQUIRE(B >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    PT_REQUIRE(B * M * N == 0 || (x && q && scale_inv), "NULL tensor pointer");
    PT_REQUIRE(N == 1 ? B < (1LL << 31) : (B < 65536 && cdiv(M, 256) < 65536),
               "grid dimension out of range");
    auto st = static_cast<hipStream_t>(stream);
#define CALL(T, E5) return launch_quant_rowwise<T, E5>(x, B, M, N, q, scale_in, scale_inv, st)
    PT_DISPATCH_HP_FP8(x_dtype, q_dtype, CALL);
#undef CALL
}

int pt_dequantize_fp8_rowwise(const void *q, int q_dtype, int64_t B, int64_t M, int64_t N,
                              const float *scale_inv, void *y, int y_dtype, void *stream) {
    PT_REQUIRE(is_fp8_dtype(q_dtype), "input must be e4m3 or e5m2");
    PT_REQUIRE(is_hp_dtype(y_dtype), "output must be bf16, fp16 or fp32");
    PT_REQUIRE(B >= 0 && M >= 0 && N >= 0, "dimensions must be non-negative");
    PT_REQUIRE(B * M * N == 0 || (q && y && scale_inv), "NULL tensor pointer");
    PT_REQUIRE(N != 1 || B < (1LL << 31), "grid dimension out of range");
    auto st = static_cast<hipStream_t>(stream);
#define CALL(T, E5) return launch_dequant_rowwise<T, E5>(q, B, M, N, scale_inv, y, st)
    PT_DISPATCH_HP_FP8(y_dtype, q_dtype, CALL);
#undef CALL
}

} // extern "C"
