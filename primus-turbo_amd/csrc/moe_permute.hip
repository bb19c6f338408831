// MoE token permute / unpermute: gathers the rows of `tokens` into expert-major order (every
// expert's rows padded with zero rows to a multiple of `pad_multiple`), carries per-token FP8 scale
// factors and router probabilities along, and adds the experts' outputs back per token.
// Semantics and the row_id_map format follow Primus-Turbo's kernels
// (csrc/kernels/moe_permute/moe_permute.cu:84-330 preprocessing, :425-510 permute, :553-620
// unpermute; host side csrc/pytorch/moe_permute/moe_permute.cpp:42-282):
//
//   row_id_map [T + pad_multiple, 2 E + 1] int32. Row of token t: entry [2 E] = n, the number of
//   local experts the token is routed to; entries [0, n) = 1-based destination rows in the permuted
//   tensor, ascending expert order; entries [E, E + n) = the expert id of each, or with top-k
//   aligned probabilities the slot k with topk_idx[t, k] == expert. Rows T + i (i < pad_multiple)
//   list, as negative 1-based rows, the i-th zero row of every expert that has one.
//   A destination beyond num_permuted_tokens (> 0) is dropped and raises overflow_flag.
//
// The reference finds each token's rank with a single-pass decoupled look-back scan whose blocks
// spin on each other's tile states. Here the scan is three short launches (per-block counts,
// one-block prefix, row map) without any inter-block waiting: the maps are a few MB against the
// GBs the permute moves, and no launch can hang on another block's progress.
// Differences: rows of `tokens` are real for every t < T (the reference treats rows at and after
// the number of routed tokens as padding, which agrees when every token is routed, the case its
// tests cover), and unpermute writes zeros for tokens routed nowhere instead of leaving them unwritten.
#include "pt_common.h"

namespace pt {

constexpr int TOK    = 256; // tokens per workgroup in the preprocessing kernels
constexpr int MAX_E  = 240; // TOK * E flag bytes + wave counts fit 64 KB of LDS

// s_flag[e * TOK + t] = 1 when token tok0 + t is routed to local expert e
template <typename MapT>
__device__ __forceinline__ void fill_flags(uint8_t *s_flag, const MapT *__restrict__ map, int64_t tok0, int64_t T, int E,
                                           int K) {
    const int tid = threadIdx.x;
    if constexpr (sizeof(MapT) == 1) {
        for (int i = tid; i < TOK * E; i += 256) {
            const int     t = i / E, e = i - t * E;
            const int64_t gt = tok0 + t;
            s_flag[e * TOK + t] = (gt < T && map[gt * E + e] != 0) ? 1 : 0;
        }
    } else {
        for (int i = tid; i < TOK * E; i += 256)
            s_flag[i] = 0;
        __syncthreads();
        for (int i = tid; i < TOK * K; i += 256) {
            const int     t = i / K, k = i - t * K;
            const int64_t gt = tok0 + t;
            if (gt >= T)
                continue;
            const int64_t e = static_cast<int64_t>(map[gt * K + k]);
            if (e >= 0 && e < E)
                s_flag[e * TOK + t] = 1;
        }
    }
    __syncthreads();
}

// s_wcnt[e * 4 + w] = routed tokens of wavefront w for expert e; s_wcnt[E * 4 + w] = tokens routed anywhere
__device__ __forceinline__ void wave_counts(const uint8_t *s_flag, int *s_wcnt, int E) {
    const int t = threadIdx.x, w = t >> 6;
    int       any = 0;
    for (int e = 0; e < E; ++e) {
        const int f = s_flag[e * TOK + t];
        any |= f;
        const int c = __popcll(__ballot(f));
        if ((t & 63) == 0)
            s_wcnt[e * 4 + w] = c;
    }
    const int c = __popcll(__ballot(any));
    if ((t & 63) == 0)
        s_wcnt[E * 4 + w] = c;
    __syncthreads();
}

template <typename MapT>
__global__ __launch_bounds__(256) void moe_count_kernel(const MapT *__restrict__ map, int64_t T, int E, int K,
                                                        int *__restrict__ counts) {
    extern __shared__ uint8_t lds[];
    uint8_t *s_flag = lds;
    int     *s_wcnt = reinterpret_cast<int *>(lds + TOK * E);
    fill_flags(s_flag, map, blockIdx.x * static_cast<int64_t>(TOK), T, E, K);
    wave_counts(s_flag, s_wcnt, E);
    for (int e = threadIdx.x; e <= E; e += 256)
        counts[blockIdx.x * static_cast<int64_t>(E + 1) + e] =
            (s_wcnt[e * 4] + s_wcnt[e * 4 + 1]) + (s_wcnt[e * 4 + 2] + s_wcnt[e * 4 + 3]);
}

// one workgroup: per-expert exclusive prefix over the blocks (in place), expert totals, padded
// expert offsets, tokens_per_expert, the padding rows of the map
__global__ __launch_bounds__(256) void moe_scan_kernel(int *__restrict__ counts, int nb, int E, int64_t T,
                                                       int pad_multiple, int64_t npt, int *__restrict__ pref,
                                                       int64_t *__restrict__ tokens_per_expert,
                                                       int *__restrict__ row_id_map, int *__restrict__ overflow_flag,
                                                       int *__restrict__ num_dispatched) {
    __shared__ int s_tot[MAX_E + 1], s_pref[MAX_E + 1], s_npad[MAX_E + 1];
    for (int e = threadIdx.x; e <= E; e += 256) {
        int run = 0;
        for (int b = 0; b < nb; ++b) {
            const int64_t i = b * static_cast<int64_t>(E + 1) + e;
            const int     c = counts[i];
            counts[i]       = run;
            run += c;
        }
        s_tot[e] = run;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int64_t prefix = 0;
        for (int e = 0; e < E; ++e) {
            const int v      = s_tot[e];
            const int padded = pad_multiple > 0 ? (v + pad_multiple - 1) / pad_multiple * pad_multiple : v;
            s_pref[e]        = static_cast<int>(prefix);
            s_npad[e]        = padded - v;
            pref[e]          = static_cast<int>(prefix);
            const int64_t over   = padded + prefix - npt;
            tokens_per_expert[e] = over < 0 ? padded : (padded - over > 0 ? padded - over : 0);
            prefix += padded;
        }
        *overflow_flag  = prefix > npt ? 1 : 0;
        *num_dispatched = s_tot[E];
    }
    __syncthreads();
    const int stride = 2 * E + 1;
    for (int i = threadIdx.x; i < pad_multiple; i += 256) {
        int *row = row_id_map + (T + i) * stride;
        int  n   = 0;
        for (int e = 0; e < E; ++e) {
            if (i >= s_npad[e])
                continue;
            const int64_t off = static_cast<int64_t>(s_tot[e]) + s_pref[e] + i + 1;
            if (off > npt)
                continue;
            row[n]     = -static_cast<int>(off);
            row[E + n] = e;
            ++n;
        }
        row[2 * E] = n;
    }
}

template <typename MapT>
__global__ __launch_bounds__(256) void moe_rowmap_kernel(const MapT *__restrict__ map, int64_t T, int E, int K,
                                                         const int *__restrict__ counts_excl,
                                                         const int *__restrict__ pref, int64_t npt, int topk_aligned,
                                                         int *__restrict__ row_id_map) {
    extern __shared__ uint8_t lds[];
    uint8_t *s_flag = lds;
    int     *s_wcnt = reinterpret_cast<int *>(lds + TOK * E);
    const int64_t tok0 = blockIdx.x * static_cast<int64_t>(TOK);
    fill_flags(s_flag, map, tok0, T, E, K);
    // first destination row of this block's tokens per expert, fetched once instead of per iteration
    __shared__ int s_base[MAX_E];
    for (int e = threadIdx.x; e < E; e += 256)
        s_base[e] = counts_excl[blockIdx.x * static_cast<int64_t>(E + 1) + e] + pref[e];
    wave_counts(s_flag, s_wcnt, E);
    const int     t = threadIdx.x, w = t >> 6, lane = t & 63;
    const int64_t gt  = tok0 + t;
    int          *row = row_id_map + (gt < T ? gt : 0) * (2 * E + 1);
    int           n   = 0;
    for (int e = 0; e < E; ++e) {
        const int      f    = s_flag[e * TOK + t];
        const uint64_t mask = __ballot(f);
        if (!f)
            continue;
        int before = __popcll(mask & ((1ull << lane) - 1ull));
        for (int w2 = 0; w2 < w; ++w2)
            before += s_wcnt[e * 4 + w2];
        const int64_t dest = static_cast<int64_t>(s_base[e]) + before + 1;
        if (dest > npt)
            continue;
        int aux = e;
        if constexpr (sizeof(MapT) != 1) {
            if (topk_aligned)
                for (int k = 0; k < K; ++k)
                    if (static_cast<int64_t>(map[gt * K + k]) == e) {
                        aux = k;
                        break;
                    }
        }
        row[n]     = static_cast<int>(dest);
        row[E + n] = aux;
        ++n;
    }
    if (gt < T)
        row[2 * E] = n;
}

// one workgroup per source row (tokens, then the pad_multiple rows of zeros)
__global__ __launch_bounds__(256) void moe_permute_kernel(const uint8_t *__restrict__ tokens, uint8_t *__restrict__ out,
                                                          int64_t hidden_bytes, const uint8_t *__restrict__ sf,
                                                          uint8_t *__restrict__ out_sf, int64_t sf_bytes,
                                                          const uint8_t *__restrict__ probs,
                                                          uint8_t *__restrict__ out_probs, int prob_bytes,
                                                          int64_t probs_stride, const int *__restrict__ row_id_map,
                                                          int E, int64_t T, int64_t out_rows) {
    const int64_t token  = blockIdx.x;
    const bool    is_pad = token >= T;
    const int    *row    = row_id_map + token * (2 * E + 1);
    const int     n      = row[2 * E];
    if (n == 0)
        return;
    const u32x4 zero{0u, 0u, 0u, 0u};
    // four 16-byte pieces per thread and round, all requested before the first is stored (a piece
    // behind the row's end re-reads the thread's first piece: no branch between the loads)
    for (int64_t j0 = threadIdx.x * 16L; j0 < hidden_bytes; j0 += 4 * 256 * 16L) {
        u32x4 v[4] = {zero, zero, zero, zero};
        if (!is_pad) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t j = j0 + q * 256 * 16L;
                v[q]            = ld128(tokens + token * hidden_bytes + (j < hidden_bytes ? j : j0));
            }
        }
        for (int i = 0; i < n; ++i) {
            const int     d = row[i];
            const int64_t r = d > 0 ? d - 1 : -static_cast<int64_t>(d) - 1;
            if (d != 0 && r < out_rows) { // a map made for a larger output never writes past this one
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int64_t j = j0 + q * 256 * 16L;
                    if (j < hidden_bytes)
                        st128_nt(out + r * hidden_bytes + j, d > 0 ? v[q] : zero);
                }
            }
        }
    }
    if (sf != nullptr)
        for (int64_t j = threadIdx.x; j < sf_bytes; j += 256) {
            const uint8_t v = is_pad ? 0 : sf[token * sf_bytes + j];
            for (int i = 0; i < n; ++i) {
                const int     d = row[i];
                const int64_t r = d > 0 ? d - 1 : -static_cast<int64_t>(d) - 1;
                if (d != 0 && r < out_rows)
                    out_sf[r * sf_bytes + j] = d > 0 ? v : 0;
            }
        }
    if (probs != nullptr)
        for (int i = threadIdx.x; i < n * prob_bytes; i += 256) {
            const int     idx = i / prob_bytes, byte = i - idx * prob_bytes;
            const int     d   = row[idx];
            const int64_t r   = d > 0 ? d - 1 : -static_cast<int64_t>(d) - 1;
            if (d == 0 || r >= out_rows)
                continue;
            const uint8_t v =
                (is_pad || d <= 0) ? 0 : probs[(token * probs_stride + row[E + idx]) * prob_bytes + byte];
            out_probs[r * prob_bytes + byte] = v;
        }
}

// one workgroup per token: sum of its experts' rows in fp32, in map order
template <typename T>
__global__ __launch_bounds__(256) void moe_unpermute_kernel(const T *__restrict__ permuted, T *__restrict__ out,
                                                            int64_t H, const uint8_t *__restrict__ permuted_probs,
                                                            uint8_t *__restrict__ probs, int prob_bytes,
                                                            int64_t probs_stride, const int *__restrict__ row_id_map,
                                                            int E, int64_t in_rows) {
    const int64_t token = blockIdx.x;
    const int    *row   = row_id_map + token * (2 * E + 1);
    const int     n     = row[2 * E];
    for (int64_t c = threadIdx.x * 8L; c < H; c += 256 * 8L) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        // the copies of four map entries are requested together, then added in the map's order
        // (an entry that names no row reads this thread's own output piece and is not added)
        for (int i0 = 0; i0 < n; i0 += 4) {
            u32x4 w[4];
            bool  ok[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int s = i0 + q < n ? row[i0 + q] : 0;
                ok[q]       = s > 0 && s <= in_rows;
                w[q]        = ld128(ok[q] ? permuted + (s - 1) * H + c : out + token * H + c);
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (ok[q]) {
                    float f0, f1;
                    unpack2<T>(w[q].x, f0, f1); acc[0] += f0; acc[1] += f1;
                    unpack2<T>(w[q].y, f0, f1); acc[2] += f0; acc[3] += f1;
                    unpack2<T>(w[q].z, f0, f1); acc[4] += f0; acc[5] += f1;
                    unpack2<T>(w[q].w, f0, f1); acc[6] += f0; acc[7] += f1;
                }
        }
        st128_nt(out + token * H + c, u32x4{pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3]), pack2<T>(acc[4], acc[5]),
                                           pack2<T>(acc[6], acc[7])});
    }
    if (probs != nullptr) {
        uint8_t *prow = probs + token * probs_stride * prob_bytes;
        for (int64_t j = threadIdx.x; j < probs_stride * prob_bytes; j += 256)
            prow[j] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < n * prob_bytes; i += 256) {
            const int idx = i / prob_bytes, byte = i - idx * prob_bytes;
            const int s   = row[idx];
            if (s > 0 && s <= in_rows)
                prow[row[E + idx] * prob_bytes + byte] = permuted_probs[(s - 1) * static_cast<int64_t>(prob_bytes) + byte];
        }
    }
}

static size_t preprocess_lds(int E) {
    return static_cast<size_t>(TOK) * E + static_cast<size_t>(E + 1) * 4 * sizeof(int);
}

} // namespace pt

using namespace pt;

extern "C" {

size_t pt_moe_permute_workspace_bytes(int64_t num_tokens, int64_t num_local_experts) {
    if (num_tokens < 0 || num_local_experts < 0)
        return 0;
    return static_cast<size_t>(cdiv(num_tokens, TOK) * (num_local_experts + 1) + num_local_experts) * sizeof(int);
}

int pt_moe_permute_preprocess(const void *expert_map, int map_kind, int64_t num_tokens, int64_t num_local_experts,
                              int64_t num_topk, int64_t pad_multiple, int64_t num_permuted_tokens, int topk_aligned_probs,
                              int *row_id_map, int64_t *tokens_per_expert, int *overflow_flag, int *num_dispatched_tokens,
                              void *workspace, size_t workspace_bytes, void *stream) {
    PT_REQUIRE(map_kind >= 0 && map_kind <= 2, "map_kind must be 0 (bool), 1 (int32) or 2 (int64)");
    PT_REQUIRE(num_tokens > 0 && num_tokens <= INT32_MAX / 2, "num_tokens must be positive (and fit the int32 row map)");
    PT_REQUIRE(num_local_experts >= 1 && num_local_experts <= MAX_E,
               "num_local_experts must be in [1, " + std::to_string(MAX_E) + "]");
    PT_REQUIRE(map_kind == 0 || num_topk >= 1, "index expert_map needs num_topk >= 1");
    PT_REQUIRE(map_kind != 0 || !topk_aligned_probs, "top-k aligned probs need the topk_idx form of expert_map");
    PT_REQUIRE(pad_multiple >= 0, "pad_multiple must be >= 0");
    PT_REQUIRE(expert_map && row_id_map && tokens_per_expert && overflow_flag && num_dispatched_tokens && workspace,
               "NULL tensor pointer");
    PT_REQUIRE(workspace_bytes >= pt_moe_permute_workspace_bytes(num_tokens, num_local_experts), "workspace too small");
    const int     E = static_cast<int>(num_local_experts), K = static_cast<int>(num_topk);
    const int     nb     = static_cast<int>(cdiv(num_tokens, TOK));
    const int64_t npt    = num_permuted_tokens <= 0 ? INT32_MAX : num_permuted_tokens;
    int          *counts = static_cast<int *>(workspace);
    int          *pref   = counts + static_cast<int64_t>(nb) * (E + 1);
    auto          st     = static_cast<hipStream_t>(stream);
    const size_t  lds    = preprocess_lds(E);
#define PT_MOE_MAP(KERNEL, ...)                                                                                           \
    do {                                                                                                                  \
        if (map_kind == 0)                                                                                                \
            KERNEL<uint8_t><<<nb, 256, lds, st>>>(static_cast<const uint8_t *>(expert_map), __VA_ARGS__);                 \
        else if (map_kind == 1)                                                                                           \
            KERNEL<int32_t><<<nb, 256, lds, st>>>(static_cast<const int32_t *>(expert_map), __VA_ARGS__);                 \
        else                                                                                                              \
            KERNEL<int64_t><<<nb, 256, lds, st>>>(static_cast<const int64_t *>(expert_map), __VA_ARGS__);                 \
    } while (0)
    PT_MOE_MAP(moe_count_kernel, num_tokens, E, K, counts);
    moe_scan_kernel<<<1, 256, 0, st>>>(counts, nb, E, num_tokens, static_cast<int>(pad_multiple), npt, pref,
                                       tokens_per_expert, row_id_map, overflow_flag, num_dispatched_tokens);
    PT_MOE_MAP(moe_rowmap_kernel, num_tokens, E, K, counts, pref, npt, topk_aligned_probs, row_id_map);
#undef PT_MOE_MAP
    return check_launch("moe_permute_preprocess");
}

int pt_moe_permute(const void *tokens, void *permuted_tokens, int64_t hidden_bytes, const void *scaling_factor,
                   void *permuted_scaling_factor, int64_t scale_bytes_per_token, const void *probs, void *permuted_probs,
                   int prob_bytes, int64_t probs_stride, const int *row_id_map, int64_t num_tokens, int64_t pad_multiple,
                   int64_t num_local_experts, int64_t num_permuted_rows, void *stream) {
    PT_REQUIRE(num_tokens >= 0 && pad_multiple >= 0 && hidden_bytes >= 0 && num_permuted_rows >= 0,
               "dimensions must be non-negative");
    PT_REQUIRE(num_local_experts >= 1 && num_local_experts <= MAX_E, "num_local_experts out of range");
    if (num_tokens + pad_multiple == 0 || num_permuted_rows == 0)
        return PT_OK;
    PT_REQUIRE(row_id_map && permuted_tokens && (tokens || num_tokens == 0), "NULL tensor pointer");
    PT_REQUIRE(hidden_bytes % 16 == 0 && aligned_to(tokens, 16) && aligned_to(permuted_tokens, 16),
               "token rows must be whole 16-byte vectors");
    PT_REQUIRE((scaling_factor == nullptr) == (permuted_scaling_factor == nullptr), "scaling factors come in pairs");
    PT_REQUIRE((probs == nullptr) == (permuted_probs == nullptr), "probs come in pairs");
    PT_REQUIRE(probs == nullptr || ((prob_bytes == 2 || prob_bytes == 4) && probs_stride >= 1),
               "probs must be 2- or 4-byte elements with a positive row stride");
    PT_REQUIRE(num_tokens + pad_multiple <= INT32_MAX, "too many rows");
    moe_permute_kernel<<<static_cast<unsigned>(num_tokens + pad_multiple), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t *>(tokens), static_cast<uint8_t *>(permuted_tokens), hidden_bytes,
        static_cast<const uint8_t *>(scaling_factor), static_cast<uint8_t *>(permuted_scaling_factor),
        scale_bytes_per_token, static_cast<const uint8_t *>(probs), static_cast<uint8_t *>(permuted_probs), prob_bytes,
        probs_stride, row_id_map, static_cast<int>(num_local_experts), num_tokens, num_permuted_rows);
    return check_launch("moe_permute_kernel");
}

int pt_moe_unpermute(const void *permuted_tokens, void *tokens, int dtype, int64_t hidden, const void *permuted_probs,
                     void *probs, int prob_bytes, int64_t probs_stride, const int *row_id_map, int64_t num_tokens,
                     int64_t num_local_experts, int64_t num_permuted_rows, void *stream) {
    PT_REQUIRE(dtype == PT_DTYPE_BF16 || dtype == PT_DTYPE_F16, "tokens must be bf16 or fp16");
    PT_REQUIRE(num_tokens >= 0 && hidden >= 0, "dimensions must be non-negative");
    PT_REQUIRE(num_local_experts >= 1 && num_local_experts <= MAX_E, "num_local_experts out of range");
    if (num_tokens == 0)
        return PT_OK;
    PT_REQUIRE(row_id_map && tokens && permuted_tokens, "NULL tensor pointer");
    PT_REQUIRE(hidden % 8 == 0 && aligned_to(tokens, 16) && aligned_to(permuted_tokens, 16),
               "token rows must be whole 16-byte vectors");
    PT_REQUIRE((probs == nullptr) == (permuted_probs == nullptr), "probs come in pairs");
    PT_REQUIRE(probs == nullptr || ((prob_bytes == 2 || prob_bytes == 4) && probs_stride >= 1),
               "probs must be 2- or 4-byte elements with a positive row stride");
    PT_REQUIRE(num_tokens <= INT32_MAX, "too many rows");
    auto           st   = static_cast<hipStream_t>(stream);
    const unsigned grid = static_cast<unsigned>(num_tokens);
    const int      E    = static_cast<int>(num_local_experts);
    if (dtype == PT_DTYPE_BF16)
        moe_unpermute_kernel<bf16_t><<<grid, 256, 0, st>>>(
            static_cast<const bf16_t *>(permuted_tokens), static_cast<bf16_t *>(tokens), hidden,
            static_cast<const uint8_t *>(permuted_probs), static_cast<uint8_t *>(probs), prob_bytes, probs_stride,
            row_id_map, E, num_permuted_rows);
    else
        moe_unpermute_kernel<f16_t><<<grid, 256, 0, st>>>(
            static_cast<const f16_t *>(permuted_tokens), static_cast<f16_t *>(tokens), hidden,
            static_cast<const uint8_t *>(permuted_probs), static_cast<uint8_t *>(probs), prob_bytes, probs_stride,
            row_id_map, E, num_permuted_rows);
    return check_launch("moe_unpermute_kernel");
}

} // extern "C"
