// Paged attention for gfx950, compiled once per head size (-DSOC_HEAD_DIM=D, D a
// multiple of 16 up to 256).
//
// paged_attn_token_kernel: one workgroup per (token, kv head, query-head chunk, key
// split). A query token at position p of cache row r attends to the keys lo..p of that
// row (lo = 0, or p - window + 1 with a window), read through the row's block table.
// It serves single decoded tokens and tokens of prompt portions alike, in float32 and
// bfloat16. The reference's decode kernel (model/kernels/csrc/paged_attention.cu:65-274)
// has the same task for one token per row; this one is laid out for 64-wide waves:
// 16 lanes share one key (each owns D/16 consecutive elements, so D = 128 in bfloat16
// is one 16-byte load per lane and a wave load covers four keys), a workgroup of 256
// threads walks 16 keys at a time, four keys per lane group are in flight, and softmax
// is kept online per lane group so that no score buffer bounds the context length.
// Scores, softmax and the weighted sum are float32; the output is rounded once.
//
// paged_attn_reduce_kernel merges the key splits of a token
// (model/kernels/csrc/paged_attention.cu:278-297).
#include "common.h"

#ifndef SOC_HEAD_DIM
#error "compile with -DSOC_HEAD_DIM=<head size>"
#endif
static_assert(SOC_HEAD_DIM % 16 == 0 && SOC_HEAD_DIM >= 16 && SOC_HEAD_DIM <= 256, "head size");

constexpr int D = SOC_HEAD_DIM;
constexpr int EPL = D / 16;          // elements per lane
constexpr int KEYS_IN_FLIGHT = 4;

template <typename T> __device__ __forceinline__ float soc_exp(float x);
template <> __device__ __forceinline__ float soc_exp<float>(float x) { return expf(x); }
template <> __device__ __forceinline__ float soc_exp<bf16>(float x) { return __expf(x); }

__device__ __forceinline__ float group16_sum(float v) {
    v += __shfl_xor(v, 8, SOC_WAVE);
    v += __shfl_xor(v, 4, SOC_WAVE);
    v += __shfl_xor(v, 2, SOC_WAVE);
    v += __shfl_xor(v, 1, SOC_WAVE);
    return v;
}

// Merge another partial (m2, l2, a2) into (m, l, a): the usual rescaling of online softmax.
template <typename T>
__device__ __forceinline__ void merge_partial(float& m, float& l, float (&a)[EPL], float m2, float l2,
                                              const float (&a2)[EPL]) {
    const float mn = fmaxf(m, m2);
    if (mn == -INFINITY) return;                      // both empty
    const float s1 = soc_exp<T>(m - mn), s2 = soc_exp<T>(m2 - mn);
    l = l * s1 + l2 * s2;
#pragma unroll
    for (int e = 0; e < EPL; ++e) a[e] = a[e] * s1 + a2[e] * s2;
    m = mn;
}

template <typename T, int GC>
__global__ void __launch_bounds__(256)
paged_attn_token_kernel(const T* __restrict__ q, const T* __restrict__ k_pool,
                        const T* __restrict__ v_pool, const int* __restrict__ block_table,
                        int table_width, const int* __restrict__ token_rows,
                        const int* __restrict__ positions, T* __restrict__ out,
                        float* __restrict__ part_o, float* __restrict__ part_ml, int Hq, int Hkv,
                        int BS, float scale, int window, int split_len, int n_splits) {
    const int G = Hq / Hkv;
    const int chunks = (G + GC - 1) / GC;
    const int kvh = blockIdx.x / chunks, g0 = (blockIdx.x % chunks) * GC;
    const int n = blockIdx.y, split = blockIdx.z;
    const int p = positions[n];
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int start = lo + split * split_len;
    const int end = min(p + 1, start + split_len);
    if (start >= end) return;                          // this split holds no key of the token

    const int tid = threadIdx.x;
    const int kg = tid / 16, l16 = tid % 16;           // key group 0..15, lane in the group
    const int* table = block_table + (size_t)token_rows[n] * table_width;

    // The group's queries, scaled, in registers: GC heads x EPL elements.
    float qr[GC][EPL];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        if (g0 + g < G) {
            VecLoad<T, EPL>::load(q + ((size_t)n * Hq + (size_t)kvh * G + g0 + g) * D + l16 * EPL, qr[g]);
#pragma unroll
            for (int e = 0; e < EPL; ++e) qr[g][e] *= scale;
        } else {
#pragma unroll
            for (int e = 0; e < EPL; ++e) qr[g][e] = 0.f;
        }
    }

    float m[GC], l[GC], acc[GC][EPL];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        m[g] = -INFINITY; l[g] = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[g][e] = 0.f;
    }

    const size_t head_off = (size_t)kvh * BS * D + (size_t)l16 * EPL;
    for (int base = start + kg; base < end; base += 16 * KEYS_IN_FLIGHT) {
        float kx[KEYS_IN_FLIGHT][EPL], vx[KEYS_IN_FLIGHT][EPL];
#pragma unroll
        for (int u = 0; u < KEYS_IN_FLIGHT; ++u) {
            const int key = base + 16 * u;
            if (key < end) {
                const int page = table[key / BS];
                const size_t off = ((size_t)page * Hkv * BS + (size_t)(key % BS)) * D + head_off;
                VecLoad<T, EPL>::load(k_pool + off, kx[u]);
                VecLoad<T, EPL>::load(v_pool + off, vx[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < KEYS_IN_FLIGHT; ++u) {
            if (base + 16 * u < end) {                 // uniform within the 16-lane group
#pragma unroll
                for (int g = 0; g < GC; ++g) {
                    float s = 0.f;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) s = fmaf(qr[g][e], kx[u][e], s);
                    s = group16_sum(s);
                    const float mn = fmaxf(m[g], s);
                    const float alpha = soc_exp<T>(m[g] - mn);      // 0 on the first key (m = -inf)
                    const float w = soc_exp<T>(s - mn);
                    l[g] = l[g] * alpha + w;
#pragma unroll
                    for (int e = 0; e < EPL; ++e) acc[g][e] = fmaf(acc[g][e], alpha, w * vx[u][e]);
                    m[g] = mn;
                }
            }
        }
    }

    // Merge the four key groups of a wave by shuffles, then the four waves through LDS.
#pragma unroll
    for (int g = 0; g < GC; ++g) {
#pragma unroll
        for (int mask = 16; mask <= 32; mask <<= 1) {
            const float m2 = __shfl_xor(m[g], mask, SOC_WAVE), l2 = __shfl_xor(l[g], mask, SOC_WAVE);
            float a2[EPL];
#pragma unroll
            for (int e = 0; e < EPL; ++e) a2[e] = __shfl_xor(acc[g][e], mask, SOC_WAVE);
            merge_partial<T>(m[g], l[g], acc[g], m2, l2, a2);
        }
    }
    __shared__ float sm_acc[4][GC][D];
    __shared__ float sm_ml[4][GC][2];
    const int wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
    if (lane < 16) {
#pragma unroll
        for (int g = 0; g < GC; ++g) {
#pragma unroll
            for (int e = 0; e < EPL; ++e) sm_acc[wave][g][l16 * EPL + e] = acc[g][e];
            if (l16 == 0) { sm_ml[wave][g][0] = m[g]; sm_ml[wave][g][1] = l[g]; }
        }
    }
    __syncthreads();
    for (int i = tid; i < GC * D; i += 256) {
        const int g = i / D, e = i % D;
        if (g0 + g >= G) continue;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) M = fmaxf(M, sm_ml[w][g][0]);
        float L = 0.f, A = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float mw = sm_ml[w][g][0];
            if (mw == -INFINITY) continue;
            const float s = soc_exp<T>(mw - M);
            L += sm_ml[w][g][1] * s;
            A += sm_acc[w][g][e] * s;
        }
        const int h = kvh * G + g0 + g;
        if (n_splits == 1) {
            out[((size_t)n * Hq + h) * D + e] = from_float<T>(A / L);
        } else {
            const size_t pi = ((size_t)n * Hq + h) * n_splits + split;
            part_o[pi * D + e] = A;
            if (e == 0) { part_ml[pi * 2] = M; part_ml[pi * 2 + 1] = L; }
        }
    }
}

template <typename T>
__global__ void paged_attn_reduce_kernel(const float* __restrict__ part_o,
                                         const float* __restrict__ part_ml,
                                         const int* __restrict__ positions, T* __restrict__ out,
                                         int Hq, int window, int split_len, int n_splits) {
    const int h = blockIdx.x, n = blockIdx.y;
    const int p = positions[n];
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int np = min(n_splits, (p + 1 - lo + split_len - 1) / split_len);
    const size_t base = ((size_t)n * Hq + h) * n_splits;
    float M = -INFINITY;
    for (int s = 0; s < np; ++s) M = fmaxf(M, part_ml[(base + s) * 2]);
    float L = 0.f;
    for (int s = 0; s < np; ++s) L += part_ml[(base + s) * 2 + 1] * soc_exp<T>(part_ml[(base + s) * 2] - M);
    for (int e = threadIdx.x; e < D; e += blockDim.x) {
        float A = 0.f;
        for (int s = 0; s < np; ++s)
            A += part_o[(base + s) * D + e] * soc_exp<T>(part_ml[(base + s) * 2] - M);
        out[((size_t)n * Hq + h) * D + e] = from_float<T>(A / L);
    }
}

template <typename T, int GC>
static int launch_token(const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                        int table_width, const int* token_rows, const int* positions, void* out,
                        float* part_o, float* part_ml, int N, int Hq, int Hkv, int BS, float scale,
                        int window, int split_len, int n_splits, hipStream_t stream) {
    const int G = Hq / Hkv, chunks = (G + GC - 1) / GC;
    hipLaunchKernelGGL((paged_attn_token_kernel<T, GC>), dim3(Hkv * chunks, N, n_splits), dim3(256), 0,
                       stream, (const T*)q, (const T*)k_pool, (const T*)v_pool, block_table,
                       table_width, token_rows, positions, (T*)out, part_o, part_ml, Hq, Hkv, BS,
                       scale, window, split_len, n_splits);
    int err = soc_last_error();
    if (err || n_splits == 1) return err;
    hipLaunchKernelGGL(paged_attn_reduce_kernel<T>, dim3(Hq, N), dim3(64), 0, stream, part_o, part_ml,
                       positions, (T*)out, Hq, window, split_len, n_splits);
    return soc_last_error();
}

template <typename T>
static int dispatch_token(int G, const void* q, const void* k_pool, const void* v_pool,
                          const int* block_table, int table_width, const int* token_rows,
                          const int* positions, void* out, float* part_o, float* part_ml, int N,
                          int Hq, int Hkv, int BS, float scale, int window, int split_len,
                          int n_splits, hipStream_t stream) {
#define SOC_ARGS q, k_pool, v_pool, block_table, table_width, token_rows, positions, out, part_o, \
                 part_ml, N, Hq, Hkv, BS, scale, window, split_len, n_splits, stream
    if (G == 1) return launch_token<T, 1>(SOC_ARGS);
    if (G == 2) return launch_token<T, 2>(SOC_ARGS);
    if (G <= 4) return launch_token<T, 4>(SOC_ARGS);
    if (D <= 128) return launch_token<T, 8>(SOC_ARGS);
    return launch_token<T, 4>(SOC_ARGS);
#undef SOC_ARGS
}

// q [N, Hq, D]; pools [pages, Hkv, BS, D]; out [N, Hq, D]. window <= 0: no window.
// n_splits > 1 needs part_o [N, Hq, n_splits, D] and part_ml [N, Hq, n_splits, 2] (float32);
// split s covers keys lo + s * split_len .. of each token.
SOC_EXPORT int soc_paged_attention_tokens(const void* q, const void* k_pool, const void* v_pool,
                                          const int* block_table, int table_width,
                                          const int* token_rows, const int* positions, void* out,
                                          float* part_o, float* part_ml, int N, int Hq, int Hkv,
                                          int BS, float scale, int window, int split_len,
                                          int n_splits, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (Hkv < 1 || Hq % Hkv || BS < 1 || n_splits < 1 || split_len < 1) return (int)hipErrorInvalidValue;
    if (n_splits > 1 && (!part_o || !part_ml)) return (int)hipErrorInvalidValue;
    if (N > 65535 || n_splits > 65535) return (int)hipErrorInvalidValue;
    const int G = Hq / Hkv;
    if (dtype == 0)
        return dispatch_token<float>(G, q, k_pool, v_pool, block_table, table_width, token_rows,
                                     positions, out, part_o, part_ml, N, Hq, Hkv, BS, scale, window,
                                     split_len, n_splits, stream);
    return dispatch_token<bf16>(G, q, k_pool, v_pool, block_table, table_width, token_rows, positions,
                                out, part_o, part_ml, N, Hq, Hkv, BS, scale, window, split_len,
                                n_splits, stream);
}

SOC_EXPORT int soc_attention_head_dim() { return D; }
