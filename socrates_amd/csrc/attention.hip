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
#include <type_traits>

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

// Terms that an architecture may add to plain softmax attention (none of them in the reference's
// model; all three are off when the fields are zero / null). They are computed by this kernel
// only: the MFMA kernels below take plain scores, and their callers send a layer with such a
// term here.
//   slopes   [Hq] float32: slopes[h] * (key position - query position) is added to the scaled
//            score of head h (a bias by distance)
//   softcap  > 0: the score becomes softcap * tanh(score / softcap) (after the bias)
//   sinks    [Hq] float32: one more logit per head that takes its share of the softmax and
//            contributes no value: the sum of weights gains exp(sinks[h] - max)
struct ScoreTerms {
    float softcap;
    const float* sinks;
    const float* slopes;
};

template <typename T, int GC>
__global__ void __launch_bounds__(256)
paged_attn_token_kernel(const T* __restrict__ q, const T* __restrict__ k_pool,
                        const T* __restrict__ v_pool, const int* __restrict__ block_table,
                        int table_width, const int* __restrict__ token_rows,
                        const int* __restrict__ positions, T* __restrict__ out,
                        float* __restrict__ part_o, float* __restrict__ part_ml, int Hq, int Hkv,
                        int BS, float scale, int window, int split_len, int n_splits, ScoreTerms st) {
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

    float m[GC], l[GC], acc[GC][EPL], slope[GC];
#pragma unroll
    for (int g = 0; g < GC; ++g) {
        m[g] = -INFINITY; l[g] = 0.f;
        slope[g] = st.slopes && g0 + g < G ? st.slopes[kvh * G + g0 + g] : 0.f;
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
                    if (st.slopes) s += slope[g] * (float)(base + 16 * u - p);
                    if (st.softcap > 0.f) s = st.softcap * tanhf(s / st.softcap);
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
            if (st.sinks) {                                  // the sink's share of the weights, no value
                const float sk = st.sinks[h], M2 = fmaxf(M, sk), sc = soc_exp<T>(M - M2);
                L = L * sc + soc_exp<T>(sk - M2);
                A *= sc;
            }
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
                                         int Hq, int window, int split_len, int n_splits, ScoreTerms st) {
    const int h = blockIdx.x, n = blockIdx.y;
    const int p = positions[n];
    const int lo = window > 0 ? max(0, p - window + 1) : 0;
    const int np = min(n_splits, (p + 1 - lo + split_len - 1) / split_len);
    const size_t base = ((size_t)n * Hq + h) * n_splits;
    float M = st.sinks ? st.sinks[h] : -INFINITY;
    for (int s = 0; s < np; ++s) M = fmaxf(M, part_ml[(base + s) * 2]);
    float L = st.sinks ? soc_exp<T>(st.sinks[h] - M) : 0.f;
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
                        int window, int split_len, int n_splits, ScoreTerms st, hipStream_t stream) {
    const int G = Hq / Hkv, chunks = (G + GC - 1) / GC;
    hipLaunchKernelGGL((paged_attn_token_kernel<T, GC>), dim3(Hkv * chunks, N, n_splits), dim3(256), 0,
                       stream, (const T*)q, (const T*)k_pool, (const T*)v_pool, block_table,
                       table_width, token_rows, positions, (T*)out, part_o, part_ml, Hq, Hkv, BS,
                       scale, window, split_len, n_splits, st);
    int err = soc_last_error();
    if (err || n_splits == 1) return err;
    hipLaunchKernelGGL(paged_attn_reduce_kernel<T>, dim3(Hq, N), dim3(64), 0, stream, part_o, part_ml,
                       positions, (T*)out, Hq, window, split_len, n_splits, st);
    return soc_last_error();
}

template <typename T>
static int dispatch_token(int G, const void* q, const void* k_pool, const void* v_pool,
                          const int* block_table, int table_width, const int* token_rows,
                          const int* positions, void* out, float* part_o, float* part_ml, int N,
                          int Hq, int Hkv, int BS, float scale, int window, int split_len,
                          int n_splits, ScoreTerms st, hipStream_t stream) {
#define SOC_ARGS q, k_pool, v_pool, block_table, table_width, token_rows, positions, out, part_o, \
                 part_ml, N, Hq, Hkv, BS, scale, window, split_len, n_splits, st, stream
    if (G == 1) return launch_token<T, 1>(SOC_ARGS);
    if (G == 2) return launch_token<T, 2>(SOC_ARGS);
    if (G <= 4) return launch_token<T, 4>(SOC_ARGS);
    if (D <= 128) return launch_token<T, 8>(SOC_ARGS);
    return launch_token<T, 4>(SOC_ARGS);
#undef SOC_ARGS
}

// q [N, Hq, D]; pools [pages, Hkv, BS, D]; out [N, Hq, D]. window <= 0: no window.
// n_splits > 1 needs part_o [N, Hq, n_splits, D] and part_ml [N, Hq, n_splits, 2] (float32);
// split s covers keys lo + s * split_len .. of each token. softcap (0: none), sinks and slopes
// ([Hq] float32 each, or null): see ScoreTerms. Any scale, also none or a negative one.
SOC_EXPORT int soc_paged_attention_tokens(const void* q, const void* k_pool, const void* v_pool,
                                          const int* block_table, int table_width,
                                          const int* token_rows, const int* positions, void* out,
                                          float* part_o, float* part_ml, int N, int Hq, int Hkv,
                                          int BS, float scale, int window, int split_len,
                                          int n_splits, int dtype, float softcap, const float* sinks,
                                          const float* slopes, hipStream_t stream) {
    if (N <= 0) return 0;
    if (Hkv < 1 || Hq % Hkv || BS < 1 || n_splits < 1 || split_len < 1 || softcap < 0.f) return (int)hipErrorInvalidValue;
    const ScoreTerms st{softcap, sinks, slopes};
    if (n_splits > 1 && (!part_o || !part_ml)) return (int)hipErrorInvalidValue;
    if (N > 65535 || n_splits > 65535) return (int)hipErrorInvalidValue;
    const int G = Hq / Hkv;
    if (dtype == 0)
        return dispatch_token<float>(G, q, k_pool, v_pool, block_table, table_width, token_rows,
                                     positions, out, part_o, part_ml, N, Hq, Hkv, BS, scale, window,
                                     split_len, n_splits, st, stream);
    return dispatch_token<bf16>(G, q, k_pool, v_pool, block_table, table_width, token_rows, positions,
                                out, part_o, part_ml, N, Hq, Hkv, BS, scale, window, split_len,
                                n_splits, st, stream);
}


// =============================================================================================
// MFMA path (bfloat16). One wave owns a block of rows that share a cache row and a kv head:
// rows are (token, query head of the group) pairs, 16 per row tile, RT row tiles per wave.
// A single decoded token fills G of the 16 rows; a prompt portion fills all of them with
// consecutive tokens. The wave walks the keys of its split 16 at a time:
//   S^T[key, row]  = K_tile [16 x D] * Q^T [D x 16]        (A = keys, B = rows)
//   online softmax per row: a row is an MFMA column, so its running maximum, its scale and
//   its sum live in the lanes of that column; the maximum over the 16 keys of a tile
//   needs two cross-lane steps
//   O^T[d, row]   += V_tile^T [16 d x 16 keys] * P^T [16 keys x 16 rows]
// S^T comes out of the first product in exactly the lane layout the second one wants for
// its B operand, so P never leaves registers. V pages are row-major [slot][d]; the V tile
// is staged through LDS (wave-private) to read it transposed. Scores, softmax and both
// accumulators are float32; P is rounded to bfloat16 for the second product, as V is.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr bool QK_K32 = (D % 32 == 0);
constexpr int QK_STEPS = QK_K32 ? D / 32 : D / 16;
constexpr int DV = D / 16;                   // 16-wide blocks of the head dimension
constexpr int V_STRIDE = D + 4;              // LDS row stride (elements): conflict-free transposed reads
constexpr int V_CHUNKS = 16 * D / 8;         // 16-byte chunks in a 16-key V tile
constexpr int V_PER_LANE = (V_CHUNKS + 63) / 64;

struct KFrag { uint4 v[QK_STEPS]; };         // K32: 16 bytes per step; K16: the low 8 bytes

__device__ __forceinline__ f32x4_t qk_mfma(const uint4& a, const uint4& b, f32x4_t c) {
    if constexpr (QK_K32) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8_t*>(&a),
                                                       *reinterpret_cast<const bf16x8_t*>(&b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const s16x4_t*>(&a),
                                                         *reinterpret_cast<const s16x4_t*>(&b), c, 0, 0, 0);
    }
}

// The slice of a K (or Q) row that this lane feeds to QK step `kk`.
__device__ __forceinline__ uint4 load_qk_slice(const bf16* row, int kk, int kb) {
    if constexpr (QK_K32) {
        return *reinterpret_cast<const uint4*>(row + kk * 32 + kb * 8);
    } else {
        const uint2 t = *reinterpret_cast<const uint2*>(row + kk * 16 + kb * 4);
        return make_uint4(t.x, t.y, 0u, 0u);
    }
}

// TP: pages hold a multiple of 16 keys (and a power of two of them), so a tile lies in one page.
constexpr float LAZY_MAX = 8.f;        // log2 of the largest softmax weight before a row's reference moves

// The rare tile that moves a reference rescales the accumulators where they are, one register
// at a time, each multiply written so that the compiler cannot regroup it: a product that
// defines a whole accumulator anew gives it a new home, and then every tile copies all
// accumulators at the join behind the branch, rescaled or not.
__device__ __forceinline__ void scale_in_place(float& v, float by) {
    asm volatile("v_mul_f32 %0, %0, %1" : "+v"(v) : "v"(by));
}
// The compiler does not look into these multiplies when it places the wait states that a
// matrix instruction needs after (or before) a vector instruction on the same registers; a
// rescaling is rare, so it is simply fenced with more idle cycles than any such rule asks for.
__device__ __forceinline__ void scale_fence() { asm volatile("s_nop 15\n\ts_nop 7" ::: "memory"); }
template <int RT_, int DV_>
__device__ __forceinline__ void rescale_in_place(f32x4_t (&o)[RT_][DV_], const float (&alpha)[RT_]) {
    scale_fence();
#pragma unroll
    for (int rt = 0; rt < RT_; ++rt)
#pragma unroll
        for (int j = 0; j < DV_; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = o[rt][j][e];
                scale_in_place(v, alpha[rt]);
                o[rt][j][e] = v;
            }
    scale_fence();
}

// FUSED (decode steps: every token alone; one row tile; head sizes in steps of 32, and of 64
// with a rotation, which is over the whole head): q is not given. The kernel reads the token's raw
// [q heads | k heads | v heads] row as the QKV product left it, and does what
// qk_norm_rope_kernel does on its way: per-head RMSNorm of q and k (if gains are given), the
// rotation at the token's position, all in float32 with one rounding to bfloat16. A lane's
// slices of a head hold both partners of every rotated pair, so nothing crosses lanes but the
// sum of squares. The token's own key and value do not go through the cache: the wave whose
// split holds the token's position adds them as one more tile from registers, and (for one
// chunk of heads) stores them to the page for the steps to come. The work hides behind the
// start of the walk (position -> table -> first keys), which it does not depend on.
struct FusedQkv {
    const bf16* qkv;            // [N, row_heads, D]: q heads, then (if the step writes the slot) k and v heads
    int row_heads;
    const float* q_gain;        // [D] each, or null: no norm
    const float* k_gain;
    const float* rope_table;    // [positions][2][D / 2] cosines and sines (soc_rope_table), or null: no rotation
    float eps;
    int write_kv;               // the step writes this cache slot (else it only reads it: queries only)
    bf16* k_pool_w;             // the pools again, to write to
    bf16* v_pool_w;
};

template <int RT, bool TP, bool FUSED = false>
__global__ void __launch_bounds__(256)
paged_attn_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pool,
                       const bf16* __restrict__ v_pool, const int* __restrict__ block_table,
                       int table_width, const int* __restrict__ token_rows,
                       const int* __restrict__ positions, const int* __restrict__ row_blocks,
                       int n_row_blocks, bf16* __restrict__ out, float* __restrict__ part_o,
                       float* __restrict__ part_ml, int* __restrict__ arrivals, int Hq, int Hkv, int BS,
                       int bs_shift, float scale, int window, int split_len_arg, int n_splits,
                       int group_pad_log2, FusedQkv fz, int out_tiled) {
    static_assert(!FUSED || (RT == 1 && QK_K32), "the fused form: one row tile, head sizes in steps of 32");
    // One piece of LDS: the waves' V tiles while the keys are walked; afterwards, with key
    // splits, what the four waves of the workgroup have gathered, to be combined.
    constexpr int V_BYTES = 4 * 16 * V_STRIDE * 2, C_BYTES = 4 * RT * DV * 64 * 16;
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[V_BYTES > C_BYTES ? V_BYTES : C_BYTES];
    __shared__ float c_ml[4][RT][16][2];
    __shared__ int came_last;
    uint16_t (*v_lds)[16 * V_STRIDE] = reinterpret_cast<uint16_t (*)[16 * V_STRIDE]>(lds_raw);
    // the wave index is the same in all lanes: say so, and what depends on it (the task, its
    // token, position and table row) is computed and loaded on the scalar side
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / SOC_WAVE), lane = threadIdx.x % SOC_WAVE;
    const int G = Hq / Hkv;
    const int Gp = 1 << group_pad_log2;                 // rows per token in a row block
    const int chunks = (G + 15) / 16;                   // head chunks when G > 16
    // Without key splits the four waves of a workgroup take four tasks. With splits
    // (a multiple of four) they take four consecutive splits of one task, combine what they
    // find through LDS, and the workgroups of a task (n_splits / 4 of them) meet in memory.
    const bool by_split = n_splits > 1;
    const int task = by_split ? (int)blockIdx.x : (int)blockIdx.x * 4 + wave;
    if (task >= n_row_blocks * Hkv * chunks) return;
    const int blk = task / (Hkv * chunks);
    const int kvh = (task / chunks) % Hkv, chunk = task % chunks;
    const int split = by_split ? (int)blockIdx.y * 4 + wave : 0;
    // no list of row blocks: every token alone (a decode step), one dependent load fewer
    const int tok0 = row_blocks ? row_blocks[2 * blk] : blk, ntok = row_blocks ? row_blocks[2 * blk + 1] : 1;
    const int pos0 = positions[tok0];
    const int* table = block_table + (size_t)token_rows[tok0] * table_width;

    // keys this wave walks: its split, cut to what its rows can see
    // split_len_arg 0: the keys this block's rows can see are shared out evenly among the
    // n_splits waves of the task (whole tiles of 16), whatever length the launch was planned
    // for: no wave of a short row walks far, none of a long row is idle
    int split_len = split_len_arg, first_key = 0;
    if (split_len_arg <= 0) {
        first_key = window > 0 ? max(0, pos0 - window + 1) & ~15 : 0;
        split_len = max(16, ((pos0 + ntok - first_key + n_splits - 1) / n_splits + 15) & ~15);
    }
    const int split_lo = first_key + split * split_len;     // the split's first key
    int klo = split_lo;
    // FUSED and writing: the token's own key is not read from the cache (it is not there yet)
    const bool own_key = FUSED && fz.write_kv;
    const bool covers = pos0 >= klo && pos0 < klo + split_len;      // this wave's split holds the token's position
    int khi = min(klo + split_len, own_key ? pos0 : pos0 + ntok);
    if (window > 0) klo = max(klo, pos0 - window + 1);
    const int kmin = klo;                                // first key any row of the block can see
    klo = klo & ~15;                                     // tiles are aligned to 16 keys
    const int li = lane % 16, kb = lane / 16;
    uint16_t* vl = v_lds[wave];

    // rows of this lane's column, per row tile
    int row_pos[RT];                                     // position of the row's token, -1: no row
    size_t row_q[RT];                                    // offset of the row's query / output
    uint4 qf[RT][QK_STEPS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int rho = rt * 16 + li;
        const int tt = rho >> group_pad_log2, g = chunk * 16 + (rho & (Gp - 1));
        const bool ok = tt < ntok && g < G;
        row_pos[rt] = ok ? pos0 + tt : -1;
        row_q[rt] = ((size_t)(tok0 + (ok ? tt : 0)) * Hq + (size_t)kvh * G + (ok ? g : 0)) * D;
        if constexpr (!FUSED) {
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk)
                qf[rt][kk] = ok ? load_qk_slice(q + row_q[rt], kk, kb) : make_uint4(0u, 0u, 0u, 0u);
        }
    }
    __shared__ float rope_cs[FUSED ? 4 : 1][FUSED ? D : 1];          // cos [0, D / 2), sin [D / 2, D) of the wave's token
    __shared__ uint4 new_kv[FUSED ? 4 : 1][FUSED ? 2 * (D / 8) : 1]; // the token's key (normed, rotated) and value, by 16-byte part
    if constexpr (FUSED) {
        const bf16* row_in = fz.qkv + (size_t)tok0 * fz.row_heads * D;
        const int g = chunk * 16 + (li & (Gp - 1));
        const bool ok = row_pos[0] >= 0;
        // raw slices first: the row's query head, the kv head's key, one part of its value
        // (every wave loads; without k and v heads in the row, a query head stands in and is
        // not used)
        const size_t q_at = ((size_t)kvh * G + (ok ? g : 0)) * D;
        const size_t k_at = own_key ? (size_t)(Hq + kvh) * D : q_at, v_at = own_key ? (size_t)(Hq + Hkv + kvh) * D : q_at;
        uint4 qraw[QK_STEPS], kraw[QK_STEPS];
#pragma unroll
        for (int kk = 0; kk < QK_STEPS; ++kk) {
            qraw[kk] = load_qk_slice(row_in + q_at, kk, kb);
            kraw[kk] = load_qk_slice(row_in + k_at, kk, kb);
        }
        const uint4 vraw = *reinterpret_cast<const uint4*>(row_in + v_at + (lane % (D / 8)) * 8);
        // the token's cosines and sines, from the table (an accurate sincosf in each of a
        // launch's thousands of waves would cost more vector time than the walk itself)
        if (fz.rope_table) {
            const float* cs_row = fz.rope_table + (size_t)pos0 * D;
            for (int j = lane; j < D; j += SOC_WAVE) rope_cs[wave][j] = cs_row[j];
            __builtin_amdgcn_wave_barrier();
        }
        // norm and rotation of this lane's slices of one head: elements 32 kk + 8 kb + t; the
        // partner of an element of the first half lies QK_STEPS / 2 slices on, in the same lane
        auto norm_rope = [&](const uint4 (&raw)[QK_STEPS], const float* gain, uint4 (&res)[QK_STEPS]) {
            float x[QK_STEPS][8];
            float ss = 0.f;
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk) {
                const uint32_t w4[4] = {raw[kk].x, raw[kk].y, raw[kk].z, raw[kk].w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    x[kk][2 * t] = __uint_as_float(w4[t] << 16);
                    x[kk][2 * t + 1] = __uint_as_float(w4[t] & 0xffff0000u);
                    ss += x[kk][2 * t] * x[kk][2 * t] + x[kk][2 * t + 1] * x[kk][2 * t + 1];
                }
            }
            if (gain) {
                ss = sum_xor32(sum_xor16(ss));
                const float inv = 1.0f / sqrtf(ss / (float)D + fz.eps);
#pragma unroll
                for (int kk = 0; kk < QK_STEPS; ++kk) {
                    float gn[8];
                    VecLoad<float, 8>::load(gain + kk * 32 + kb * 8, gn);
#pragma unroll
                    for (int t = 0; t < 8; ++t) x[kk][t] = x[kk][t] * inv * gn[t];
                }
            }
            if (fz.rope_table) {
                constexpr int HK = QK_STEPS / 2;
#pragma unroll
                for (int kk = 0; kk < HK; ++kk)
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const float cs = rope_cs[wave][kk * 32 + kb * 8 + t], sn = rope_cs[wave][D / 2 + kk * 32 + kb * 8 + t];
                        const float a = x[kk][t], b = x[kk + HK][t];
                        x[kk][t] = a * cs - b * sn;
                        x[kk + HK][t] = b * cs + a * sn;
                    }
            }
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk)
                res[kk] = make_uint4(pack_bf16x2(x[kk][0], x[kk][1]), pack_bf16x2(x[kk][2], x[kk][3]),
                                     pack_bf16x2(x[kk][4], x[kk][5]), pack_bf16x2(x[kk][6], x[kk][7]));
        };
        uint4 qn[QK_STEPS];
        norm_rope(qraw, fz.q_gain, qn);
#pragma unroll
        for (int kk = 0; kk < QK_STEPS; ++kk) qf[0][kk] = ok ? qn[kk] : make_uint4(0u, 0u, 0u, 0u);
        if (own_key && covers) {                              // uniform over the wave
            uint4 kn[QK_STEPS];
            norm_rope(kraw, fz.k_gain, kn);
            if (li == 0) {
#pragma unroll
                for (int kk = 0; kk < QK_STEPS; ++kk) new_kv[wave][kk * 4 + kb] = kn[kk];
            }
            if (lane < D / 8) new_kv[wave][D / 8 + lane] = vraw;
            if (chunk == 0) {
                // to the page, for the steps to come (nothing of this launch reads it there)
                const int page_i = bs_shift >= 0 ? pos0 >> bs_shift : pos0 / BS;
                const size_t off = (size_t)table[page_i] * Hkv * BS * D + (size_t)kvh * BS * D +
                                   (size_t)(pos0 - page_i * BS) * D;
                if (li == 0) {
#pragma unroll
                    for (int kk = 0; kk < QK_STEPS; ++kk)
                        *reinterpret_cast<uint4*>(fz.k_pool_w + off + kk * 32 + kb * 8) = kn[kk];
                }
                if (lane < D / 8) *reinterpret_cast<uint4*>(fz.v_pool_w + off + lane * 8) = vraw;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }

    // Where four outputs of a row go: element `at` = (token * Hq + head) * D + d of out
    // [N, Hq * D], or (out_tiled = R > 0: at most R tokens) the same element of out [Hq * D / 32, R, 32],
    // the layout in which the product that follows reads 64 bytes of every row side by side.
    auto out_at = [&](size_t at) -> bf16* {
        if (!out_tiled) return out + at;
        const size_t width = (size_t)Hq * D, tok = at / width;
        const int col = (int)(at - tok * width);
        return out + ((size_t)(col / 32) * out_tiled + tok) * 32 + col % 32;
    };
    f32x4_t o[RT][DV];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY; l[rt] = 0.f;
#pragma unroll
        for (int j = 0; j < DV; ++j) o[rt][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    }

    const float c2 = scale * 1.44269504088896340736f;   // scores to base 2
    const size_t page_stride = (size_t)Hkv * BS * D;
    const bf16* k_base = k_pool + (size_t)kvh * BS * D;
    const bf16* v_base = v_pool + (size_t)kvh * BS * D;
    // Pages of a multiple of 16 keys: a tile lies in one page, so its page is one value for
    // the whole wave, read on the scalar side, and no lane needs another's.
    constexpr bool tile_in_page = TP;
    // Loads must stay in flight until their tile is computed, so nothing touches what they
    // bring before that: no branch around a load (the two sides would have to be reconciled
    // in registers behind it), no select on its result. A key that must not be read (outside
    // what the block's rows can see) is redirected to the first entry of the row's table (a
    // page of the pool whatever it holds), and its data are replaced by zeros when the tile
    // is computed, so that what lies in stale slots (inf, NaN) never meets a product.
    // lookup: the page of the tile (TP: one value for the wave) or of this lane's key (lanes
    // 0..15 of every lane group hold keys 0..15).
    auto lookup = [&](int key0) -> int {
        if constexpr (tile_in_page) {
            const bool any = key0 < khi && key0 + 16 > kmin;
            return table[__builtin_amdgcn_readfirstlane(any ? key0 >> bs_shift : 0)];
        } else {
            const int key = key0 + li;
            const bool ok = key >= kmin && key < khi;
            return table[ok ? key / BS : 0];
        }
    };
    // Global loads of one tile: this lane's K slices and its share of the V tile.
    auto fetch = [&](int key0, int page, KFrag& kf, uint4 (&vr)[V_PER_LANE]) {
        if constexpr (tile_in_page) {
            const size_t tile_off = (size_t)page * page_stride + (size_t)((key0 & (BS - 1)) * D);
            const bf16* krow = k_base + tile_off + li * D;
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk) kf.v[kk] = load_qk_slice(krow, kk, kb);
#pragma unroll
            for (int j = 0; j < V_PER_LANE; ++j) {
                const int c = (lane + 64 * j) % V_CHUNKS;        // lanes past the tile's chunks reload one of them
                const int vk = c / (D / 8), part = c % (D / 8);
                vr[j] = *reinterpret_cast<const uint4*>(v_base + tile_off + vk * D + part * 8);
            }
        } else {
            const int key = key0 + li;
            const bf16* krow = k_base + (size_t)page * page_stride + (size_t)(key % BS) * D;
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk) kf.v[kk] = load_qk_slice(krow, kk, kb);
#pragma unroll
            for (int j = 0; j < V_PER_LANE; ++j) {
                const int c = (lane + 64 * j) % V_CHUNKS;
                const int vk = c / (D / 8), part = c % (D / 8);
                const int vpage = __shfl(page, vk, SOC_WAVE);                  // from the lane that owns key vk
                vr[j] = *reinterpret_cast<const uint4*>(
                    v_base + (size_t)vpage * page_stride + (size_t)((key0 + vk) % BS) * D + part * 8);
            }
        }
    };

    // One tile: V to LDS, scores, online softmax, weighted values. MASKED: some key of the
    // tile is hidden from some row of the block (or lies outside the split).
    // A tile in two halves. The first (MASKED or not): the V tile to LDS, scores and softmax
    // weights, packed as operand B of the second product. The second half is one piece of code
    // behind both variants, so that the accumulators have one home (with the products inside
    // the variants the compiler copies accumulators at every join).
    // MASKED: keys outside [lo, hi) are not there (their data become zeros), and a row sees
    // the keys from lo_seen on, up to its own position, inside its window.
    auto scores = [&](int key0, const KFrag& kf, const uint4 (&vr)[V_PER_LANE], auto masked_tag,
                      s16x4_t (&pf)[RT], float (&alpha)[RT], bool& any_rescale, int lo, int hi, int lo_seen) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // V tile -> LDS, row-major with a padded stride (two 8-byte stores per chunk); keys
        // that were not to be read become zeros here, now that their loads have landed
#pragma unroll
        for (int j = 0; j < V_PER_LANE; ++j) {
            const int c = lane + 64 * j;
            if (V_CHUNKS % 64 == 0 || c < V_CHUNKS) {
                const int vk = c / (D / 8), part = c % (D / 8);
                uint4 t = vr[j];
                if constexpr (MASKED) {
                    const int vkey = key0 + vk;
                    if (vkey < lo || vkey >= hi) t = make_uint4(0u, 0u, 0u, 0u);
                }
                uint2* dst = reinterpret_cast<uint2*>(&vl[vk * V_STRIDE + part * 8]);
                dst[0] = make_uint2(t.x, t.y);
                dst[1] = make_uint2(t.z, t.w);
            }
        }
        __builtin_amdgcn_wave_barrier();
        const bool k_ok = !MASKED || (key0 + li >= lo && key0 + li < hi);
        any_rescale = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            f32x4_t s = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk)
                s = qk_mfma(k_ok ? kf.v[kk] : make_uint4(0u, 0u, 0u, 0u), qf[rt][kk], s);
            float sv[4];
            float mx = -INFINITY;                           // of the raw scores: the scale is positive
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sv[r] = s[r];
                if constexpr (MASKED) {
                    const int key = key0 + 4 * kb + r;
                    bool seen = key <= row_pos[rt] && key < hi && key >= lo_seen;
                    if (window > 0) seen = seen && key > row_pos[rt] - window;
                    sv[r] = seen ? sv[r] : -INFINITY;
                }
                mx = fmaxf(mx, sv[r]);
            }
            mx = max_xor32(max_xor16(mx)) * c2;
            // m is the row's reference for the exponentials, not its maximum: it moves only
            // when a tile's maximum lies more than LAZY_MAX above it, so the accumulators are
            // rescaled a few times per row instead of in most tiles (weights stay below 2^8);
            // the merge of splits works with any reference
            const bool move = mx > m[rt] + LAZY_MAX;
            const float mn = move ? mx : m[rt];
            const float ms = mn == -INFINITY ? 0.f : mn;
            alpha[rt] = move ? __builtin_amdgcn_exp2f(m[rt] - ms) : 1.f;
            float p[4];
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], c2, -ms));
                psum += p[r];
            }
            l[rt] = l[rt] * alpha[rt] + psum;
            any_rescale = any_rescale || move;
            m[rt] = mn;
            const uint32_t p01 = pack_bf16x2(p[0], p[1]), p23 = pack_bf16x2(p[2], p[3]);
            pf[rt] = (s16x4_t){(short)(p01 & 0xffffu), (short)(p01 >> 16), (short)(p23 & 0xffffu), (short)(p23 >> 16)};
        }
    };
    auto weighted = [&](const s16x4_t (&pf)[RT], const float (&alpha)[RT], bool any_rescale) {
        if (__any(any_rescale)) rescale_in_place(o, alpha);
        // O^T += V^T P^T, one 16-wide block of d at a time; the V^T slice is shared by the row tiles
#pragma unroll
        for (int j = 0; j < DV; ++j) {
            const uint16_t* src = &vl[(4 * kb) * V_STRIDE + j * 16 + li];
            const s16x4_t vt = (s16x4_t){(short)src[0], (short)src[V_STRIDE], (short)src[2 * V_STRIDE],
                                         (short)src[3 * V_STRIDE]};
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                o[rt][j] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vt, pf[rt], o[rt][j], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
    };
    // whole: every key of the tile lies in the split, at or before the block's first position
    // and inside the window of its last one, so no score needs a mask
    const int last_pos = pos0 + ntok - 1;
    auto tile = [&](int key0, const KFrag& kf, const uint4 (&vr)[V_PER_LANE]) {
        const bool whole = key0 >= split_lo && key0 + 15 < khi && key0 + 15 <= pos0 &&
                           (window <= 0 || key0 > last_pos - window);
        s16x4_t pf[RT];
        float alpha[RT];
        bool any_rescale;
        if constexpr (D > 128) {
            scores(key0, kf, vr, std::true_type{}, pf, alpha, any_rescale, kmin, khi, split_lo);     // one variant: registers are short at these sizes
        } else {
            if (whole) scores(key0, kf, vr, std::false_type{}, pf, alpha, any_rescale, kmin, khi, split_lo);
            else scores(key0, kf, vr, std::true_type{}, pf, alpha, any_rescale, kmin, khi, split_lo);
        }
        weighted(pf, alpha, any_rescale);
    };

    // Three tiles are in flight per wave (48 keys). Buffer b holds tiles b, b + 3, b + 6, ...
    // of the wave's range; the page of a tile is looked up three tiles before its loads are
    // issued.
    KFrag kf0, kf1, kf2;
    uint4 vr0[V_PER_LANE], vr1[V_PER_LANE], vr2[V_PER_LANE];
    // Lookups first, then the tile loads: a wait for a lookup then leaves the loads in flight.
    // Lookups may run past the end of the range (redirected); tile loads do not: the rounds
    // of the main loop are those in which all three buffers have a tile to load, and what
    // remains (at most five tiles, two of them still to load) follows without a loop.
    int pa = lookup(klo), pb = lookup(klo + 16), pc = lookup(klo + 32);
    int pg0 = lookup(klo + 48), pg1 = lookup(klo + 64), pg2 = lookup(klo + 80);
    fetch(klo, pa, kf0, vr0);
    if (klo + 16 < khi) fetch(klo + 16, pb, kf1, vr1);
    if (klo + 32 < khi) fetch(klo + 32, pc, kf2, vr2);
    int key0 = klo;
    for (; key0 + 80 < khi; key0 += 48) {
        tile(key0, kf0, vr0);
        fetch(key0 + 48, pg0, kf0, vr0);
        pg0 = lookup(key0 + 96);
        tile(key0 + 16, kf1, vr1);
        fetch(key0 + 64, pg1, kf1, vr1);
        pg1 = lookup(key0 + 112);
        tile(key0 + 32, kf2, vr2);
        fetch(key0 + 80, pg2, kf2, vr2);
        pg2 = lookup(key0 + 128);
    }
    for (; key0 < khi; key0 += 48) {                         // at most two rounds: five tiles
        tile(key0, kf0, vr0);
        if (key0 + 48 < khi) fetch(key0 + 48, pg0, kf0, vr0);
        if (key0 + 16 >= khi) break;
        tile(key0 + 16, kf1, vr1);
        if (key0 + 64 < khi) fetch(key0 + 64, pg1, kf1, vr1);
        if (key0 + 32 >= khi) break;
        tile(key0 + 32, kf2, vr2);
    }

    if constexpr (FUSED) {
        if (own_key && covers) {
            // the token's own key and value, from where the prologue left them: one more tile
            // whose first key is the only one there
            KFrag kfn;
            uint4 vrn[V_PER_LANE];
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk) kfn.v[kk] = new_kv[wave][kk * 4 + kb];
#pragma unroll
            for (int j = 0; j < V_PER_LANE; ++j) vrn[j] = new_kv[wave][D / 8 + (lane + 64 * j) % (D / 8)];
            s16x4_t pf[RT];
            float alpha[RT];
            bool any_rescale;
            scores(pos0, kfn, vrn, std::true_type{}, pf, alpha, any_rescale, pos0, pos0 + 1, pos0);
            weighted(pf, alpha, any_rescale);
        }
    }
    // finish: the row sum is spread over the four lanes of the row's column
    float L[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) L[rt] = sum_xor32(sum_xor16(l[rt]));
    if (!by_split) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            if (row_pos[rt] < 0) continue;
            const float inv = L[rt] > 0.f ? 1.0f / L[rt] : 0.f;
#pragma unroll
            for (int j = 0; j < DV; ++j) {
                uint2 pk;
                pk.x = pack_bf16x2(o[rt][j][0] * inv, o[rt][j][1] * inv);
                pk.y = pack_bf16x2(o[rt][j][2] * inv, o[rt][j][3] * inv);
                *reinterpret_cast<uint2*>(out_at(row_q[rt] + j * 16 + 4 * kb)) = pk;
            }
        }
        return;
    }
    // Four splits, one per wave, through LDS: every wave leaves its sums and its references,
    // then takes every fourth 16-wide block of the head dimension and adds the four shares of
    // it under a common reference (any reference serves, see the lazy maximum above).
    float4 (*c_o)[RT * DV][64] = reinterpret_cast<float4 (*)[RT * DV][64]>(lds_raw);
    __syncthreads();                                        // every wave is done with its V tiles
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int j = 0; j < DV; ++j)
            c_o[wave][rt * DV + j][lane] = make_float4(o[rt][j][0], o[rt][j][1], o[rt][j][2], o[rt][j][3]);
        if (kb == 0) { c_ml[wave][rt][li][0] = m[rt]; c_ml[wave][rt][li][1] = L[rt]; }
    }
    __syncthreads();
    const int outer = n_splits / 4;                         // workgroups of this task
    // partials lie by (row block, token in it), not by token: a call may cover some of the
    // tokens only
    const long shift = row_blocks ? (long)blk * ((16 * RT) >> group_pad_log2) - tok0 : 0;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float wgt[4], M4 = -INFINITY, L4 = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) M4 = fmaxf(M4, c_ml[w][rt][li][0]);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float mw = c_ml[w][rt][li][0];
            wgt[w] = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M4);
            L4 += wgt[w] * c_ml[w][rt][li][1];
        }
        if (row_pos[rt] < 0) continue;
        const size_t pi = (size_t)((long)(row_q[rt] / D) + shift * Hq) * outer + blockIdx.y;
        const float inv = L4 > 0.f ? 1.0f / L4 : 0.f;
        for (int j = wave; j < DV; j += 4) {
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const float4 t = c_o[w][rt * DV + j][lane];
                a.x += t.x * wgt[w]; a.y += t.y * wgt[w]; a.z += t.z * wgt[w]; a.w += t.w * wgt[w];
            }
            if (outer == 1) {
                uint2 pk;
                pk.x = pack_bf16x2(a.x * inv, a.y * inv);
                pk.y = pack_bf16x2(a.z * inv, a.w * inv);
                *reinterpret_cast<uint2*>(out_at(row_q[rt] + j * 16 + 4 * kb)) = pk;
            } else {
                // written through the caches (agent scope): another workgroup reads it below
                float* dst = part_o + pi * D + j * 16 + 4 * kb;
                __hip_atomic_store(dst, a.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + 1, a.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + 2, a.z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + 3, a.w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (outer > 1 && wave == 0 && kb == 0) {
            __hip_atomic_store(part_ml + pi * 2, M4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(part_ml + pi * 2 + 1, L4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (outer == 1) return;
    // The workgroups of a task meet in memory without a fence (a fence writes back and
    // invalidates the chip's whole L2): the partial results above went through the caches, a
    // wait for their acknowledgement orders them before the arrival count, and the workgroup
    // counted last reads all of them past the caches and writes the rows. The count is left
    // at zero for the next launch.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const int before = __hip_atomic_fetch_add(arrivals + task, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        came_last = before == outer - 1;
        if (came_last) __hip_atomic_store(arrivals + task, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!came_last) return;
    // The rows of the task go round the four waves. For a row, the splits' references and sums
    // lie across the lanes (at most 64 workgroups per task); a lane owns four elements of the
    // head dimension, every D / 4 lanes form a group, and group g adds the splits g, g + NG, ...
    // in that order; the groups are added in order. All loads of a round are issued before the
    // first is needed: one trip to memory for a row.
    constexpr int LPG = D / 4, NG = SOC_WAVE / LPG, ROUND = 8;
    float4* red = reinterpret_cast<float4*>(lds_raw) + wave * SOC_WAVE;
    const int sg = lane / LPG, e4 = lane % LPG;
    for (int rho = wave; rho < 16 * RT; rho += 4) {
        const int tt = rho >> group_pad_log2, g = chunk * 16 + ((rho % 16) & (Gp - 1));
        if (tt >= ntok || g >= G) continue;
        const size_t row = (size_t)(tok0 + tt) * Hq + (size_t)kvh * G + g;       // (token, head)
        const size_t p0 = (size_t)((long)row + shift * Hq) * outer;
        const int mine = lane < outer ? lane : 0;
        const float ms_ = __hip_atomic_load(part_ml + (p0 + mine) * 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const float ls_ = __hip_atomic_load(part_ml + (p0 + mine) * 2 + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        float M = 0.f, Lt = 0.f, wl = 0.f;
        for (int s0 = 0; s0 < outer; s0 += ROUND * NG) {
            float4 v[ROUND];
#pragma unroll
            for (int j = 0; j < ROUND; ++j) {
                const int sp = s0 + sg + j * NG;
                const float* src = part_o + (p0 + (sg < NG && sp < outer ? sp : 0)) * D + e4 * 4;
                v[j].x = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v[j].y = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v[j].z = __hip_atomic_load(src + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                v[j].w = __hip_atomic_load(src + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (s0 == 0) {
                const float ms = lane < outer ? ms_ : -INFINITY;
                M = wave_max(ms);
                wl = ms == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ms - M);      // the references are in base 2
                Lt = wave_sum(wl * (lane < outer ? ls_ : 0.f));
            }
#pragma unroll
            for (int j = 0; j < ROUND; ++j) {
                const int sp = s0 + sg + j * NG;
                const float wj = __shfl(wl, sp < SOC_WAVE ? sp : 0, SOC_WAVE);
                if (sg < NG && sp < outer && wj != 0.f) {
                    acc.x += v[j].x * wj; acc.y += v[j].y * wj; acc.z += v[j].z * wj; acc.w += v[j].w * wj;
                }
            }
        }
        if constexpr (NG > 1) {
            red[lane] = acc;
            __builtin_amdgcn_wave_barrier();
            if (lane < LPG)
                for (int gi = 1; gi < NG; ++gi) {
                    const float4 t = red[gi * LPG + lane];
                    acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
                }
            __builtin_amdgcn_wave_barrier();
        }
        if (lane < LPG) {
            const float inv = Lt > 0.f ? 1.0f / Lt : 0.f;
            uint2 pk;
            pk.x = pack_bf16x2(acc.x * inv, acc.y * inv);
            pk.y = pack_bf16x2(acc.z * inv, acc.w * inv);
            *reinterpret_cast<uint2*>(out_at(row * D + e4 * 4)) = pk;
        }
    }
}

// bfloat16 only. row_blocks [n_row_blocks, 2] = (first token, tokens) of each block of at most
// (16 * row_tiles) >> group_pad_log2 tokens of one sequence, or null: every token is a block
// of its own (n_row_blocks = N); 2^group_pad_log2 >= min(G, 16).
// Splits are over absolute key indices: split s covers keys [s * split_len, (s + 1) * split_len),
// split_len a multiple of 16; or split_len 0: every row block's visible keys are shared out
// evenly among its n_splits splits (whole tiles of 16). n_splits > 1 must be a multiple of 4 (four splits share a
// workgroup), at most 256, and needs part_o [R, Hq, n_splits / 4, D] and part_ml
// [R, Hq, n_splits / 4, 2] if n_splits > 4, with R = N without row blocks, else n_row_blocks *
// tokens per block (the blocks may cover some of the N tokens only; the others' outputs are
// not touched), and `arrivals`, one int per task (row block x kv head x chunk of 16 heads),
// zero before the call and zero again after it; calls that may run at the same time need
// arrival counts of their own. out_tiled = R (0: no; N <= R <= 64, Hq * D a multiple of 32): out is
// written [Hq * D / 32, R, 32] instead of [N, Hq * D], for a product that reads its x by tile.
SOC_EXPORT int soc_paged_attention_mfma(const void* q, const void* k_pool, const void* v_pool,
                                        const int* block_table, int table_width, const int* token_rows,
                                        const int* positions, const int* row_blocks, int n_row_blocks,
                                        void* out, float* part_o, float* part_ml, int* arrivals, int N,
                                        int Hq, int Hkv, int BS, float scale, int window, int split_len,
                                        int n_splits, int row_tiles, int group_pad_log2, int out_tiled,
                                        hipStream_t stream) {
    if (N <= 0 || n_row_blocks <= 0) return 0;
    if (out_tiled && (out_tiled < 0 || N > out_tiled || out_tiled > 64 || (Hq * D) % 32)) return (int)hipErrorInvalidValue;
    if (Hkv < 1 || Hq % Hkv || BS < 1 || n_splits < 1 || (split_len != 0 && split_len < 16) || split_len % 16)
        return (int)hipErrorInvalidValue;
    if (!row_blocks && n_row_blocks != N) return (int)hipErrorInvalidValue;
    if (n_splits > 1 && n_splits % 4) return (int)hipErrorInvalidValue;
    if (n_splits > 4 && (!part_o || !part_ml || !arrivals)) return (int)hipErrorInvalidValue;
    const int G = Hq / Hkv;
    if ((1 << group_pad_log2) < (G < 16 ? G : 16) || group_pad_log2 > 4) return (int)hipErrorInvalidValue;
    if (n_splits > 256) return (int)hipErrorInvalidValue;
    if (!(scale > 0.f)) return (int)hipErrorInvalidValue;        // the maximum is taken of the raw scores
    const long tasks = (long)n_row_blocks * Hkv * ((G + 15) / 16);
    if (tasks > 0x7fffffffL) return (int)hipErrorInvalidValue;
    const FusedQkv fz{};
    const dim3 grid = n_splits > 1 ? dim3((unsigned)tasks, n_splits / 4) : dim3((unsigned)((tasks + 3) / 4), 1);
    int bs_shift = -1;                                           // log2 of the page size if it is a power of two
    if ((BS & (BS - 1)) == 0)
        for (bs_shift = 0; (1 << bs_shift) < BS; ++bs_shift) {}
#define SOC_MFMA_ARGS (const bf16*)q, (const bf16*)k_pool, (const bf16*)v_pool, block_table, table_width, \
        token_rows, positions, row_blocks, n_row_blocks, (bf16*)out, part_o, part_ml, arrivals, Hq, Hkv, BS, bs_shift, \
        scale, window, split_len, n_splits, group_pad_log2, fz, out_tiled
    // Row tiles beyond what the registers hold at this head size are refused: two up to head
    // size 128, four up to 64.
    const bool tp = bs_shift >= 4;
#define SOC_MFMA_LAUNCH(RT_)                                                                          \
    do {                                                                                              \
        if (tp) hipLaunchKernelGGL((paged_attn_mfma_kernel<RT_, true>), grid, dim3(256), 0, stream, SOC_MFMA_ARGS); \
        else hipLaunchKernelGGL((paged_attn_mfma_kernel<RT_, false>), grid, dim3(256), 0, stream, SOC_MFMA_ARGS);   \
    } while (0)
    if (row_tiles == 1) {
        SOC_MFMA_LAUNCH(1);
    } else if (row_tiles == 2) {
        if constexpr (D <= 128) SOC_MFMA_LAUNCH(2);
        else return (int)hipErrorInvalidValue;
    } else if (row_tiles == 4) {
        if constexpr (D <= 64) SOC_MFMA_LAUNCH(4);
        else return (int)hipErrorInvalidValue;
    } else {
        return (int)hipErrorInvalidValue;
    }
#undef SOC_MFMA_LAUNCH
#undef SOC_MFMA_ARGS
    return soc_last_error();
}


// A decode step's attention from the QKV product's raw rows (the FUSED form of the kernel
// above): qkv [N, row_heads, D] with row_heads = Hq + 2 Hkv if write_kv, else at least Hq;
// q_gain, k_gain [D] float32 or both null; rope_table [rope_positions][2][D / 2] float32
// (soc_rope_table; every position of the step lies below rope_positions, which the caller
// checks) or null (no rotation; else it is over the whole head); every token alone. With write_kv the token's key and value
// are stored at its position in the pools. Head sizes in steps of 32, with a rotation in
// steps of 64 (returns hipErrorNotSupported otherwise: the caller then runs the kernels one
// after the other).
SOC_EXPORT int soc_paged_attention_decode_fused(const void* qkv, int row_heads, void* k_pool, void* v_pool,
                                                const int* block_table, int table_width,
                                                const int* token_rows, const int* positions, void* out,
                                                float* part_o, float* part_ml, int* arrivals, int N, int Hq,
                                                int Hkv, int BS, float scale, int window, int split_len,
                                                int n_splits, int group_pad_log2, const float* q_gain,
                                                const float* k_gain, const float* rope_table, float eps,
                                                int write_kv, int out_tiled, hipStream_t stream) {
    if constexpr (!QK_K32) {
        return (int)hipErrorNotSupported;
    } else {
        if (N <= 0) return 0;
        if (out_tiled && (out_tiled < 0 || N > out_tiled || out_tiled > 64 || (Hq * D) % 32)) return (int)hipErrorInvalidValue;
        if (Hkv < 1 || Hq % Hkv || BS < 1 || n_splits < 1 || (split_len != 0 && split_len < 16) || split_len % 16)
            return (int)hipErrorInvalidValue;
        if (n_splits > 1 && n_splits % 4) return (int)hipErrorInvalidValue;
        if (n_splits > 4 && (!part_o || !part_ml || !arrivals)) return (int)hipErrorInvalidValue;
        if (n_splits > 256 || !(scale > 0.f)) return (int)hipErrorInvalidValue;
        if ((q_gain == nullptr) != (k_gain == nullptr)) return (int)hipErrorInvalidValue;
        if (rope_table && D % 64) return (int)hipErrorNotSupported;    // partners of a pair in one lane
        if (row_heads < (write_kv ? Hq + 2 * Hkv : Hq)) return (int)hipErrorInvalidValue;
        const int G = Hq / Hkv;
        if ((1 << group_pad_log2) < (G < 16 ? G : 16) || group_pad_log2 > 4) return (int)hipErrorInvalidValue;
        const long tasks = (long)N * Hkv * ((G + 15) / 16);
        if (tasks > 0x7fffffffL) return (int)hipErrorInvalidValue;
        FusedQkv fz{};
        fz.qkv = (const bf16*)qkv; fz.row_heads = row_heads; fz.q_gain = q_gain; fz.k_gain = k_gain;
        fz.rope_table = rope_table; fz.eps = eps; fz.write_kv = write_kv ? 1 : 0;
        fz.k_pool_w = (bf16*)k_pool; fz.v_pool_w = (bf16*)v_pool;
        const dim3 grid = n_splits > 1 ? dim3((unsigned)tasks, n_splits / 4) : dim3((unsigned)((tasks + 3) / 4), 1);
        int bs_shift = -1;
        if ((BS & (BS - 1)) == 0)
            for (bs_shift = 0; (1 << bs_shift) < BS; ++bs_shift) {}
#define SOC_FUSED_ARGS (const bf16*)nullptr, (const bf16*)k_pool, (const bf16*)v_pool, block_table, table_width, \
        token_rows, positions, (const int*)nullptr, N, (bf16*)out, part_o, part_ml, arrivals, Hq, Hkv, BS, bs_shift, \
        scale, window, split_len, n_splits, group_pad_log2, fz, out_tiled
        if (bs_shift >= 4)
            hipLaunchKernelGGL((paged_attn_mfma_kernel<1, true, true>), grid, dim3(256), 0, stream, SOC_FUSED_ARGS);
        else
            hipLaunchKernelGGL((paged_attn_mfma_kernel<1, false, true>), grid, dim3(256), 0, stream, SOC_FUSED_ARGS);
#undef SOC_FUSED_ARGS
        return soc_last_error();
    }
}


// =============================================================================================
// Prompt portions (bfloat16): a workgroup of four waves owns 4 * RT * 16 rows of one sequence
// and kv head (consecutive tokens x the heads of the group) and walks the keys 32 at a time.
// The four waves load each K and V tile once, together, into LDS, which cuts the traffic from
// L2 by four against one wave per row block. Tiles are double-buffered in LDS; the global
// loads of the next tile are issued before the products of the current one, and the pages of
// the tile after that are looked up at the same time, so no wave waits for a lookup.
//
// Layouts. A lane owns eight consecutive keys of a tile (8 * (lane / 16) ..): K rows are
// stored in LDS in the order in which the two 16-key products want them (row 16 * sub + i
// holds key 8 * (i / 4) + 4 * sub + i % 4), so that the scores of a lane, from both products,
// are those eight keys, which is what the 32-key second product wants as operand B. V is
// stored transposed ([d][key], two keys packed per word on the way in), so that a lane's
// slice of V^T is 16 contiguous bytes. Softmax runs in base 2 (scores times scale * log2 e)
// in float32. Tiles that every row of a wave sees whole take a path without masks.
constexpr int PF_KEYS = 32;
constexpr int PF_K_STRIDE = D + 8;                  // K tile [32][D + 8]
constexpr int PF_V_STRIDE = PF_KEYS + 4;            // V^T tile [D][32 + 4]
constexpr int PF_K_ELEMS = PF_KEYS * PF_K_STRIDE, PF_V_ELEMS = D * PF_V_STRIDE;
constexpr int PF_PARTS = D / 8;                     // 16-byte chunks of one key

__device__ __forceinline__ int pf_k_row(int k) {    // LDS row of key k of a tile
    return 16 * ((k >> 2) & 1) + 4 * (k >> 3) + (k & 3);
}

// LDS row of key k of a tile for the 32-row products: bits 2 and 3 of k change places, so that
// the 16 scores a lane gets from one 32 x 32 product are two runs of eight neighbouring keys,
// which is what the second product wants from it as operand B.
__device__ __forceinline__ int pf_k_row32(int k) { return (k & ~12) | ((k & 4) << 1) | ((k & 8) >> 1); }

typedef __attribute__((ext_vector_type(16))) float f32x16_t;

// PAIR: pages hold an even, power-of-two number of keys, so a thread's two keys share a page.
// M32: a wave owns 32 rows and multiplies with the 32 x 32 x 16 instruction (RT = 1; head
// sizes that are multiples of 32): per row, half the loads, LDS reads, stores and barriers
// of RT = 1, as RT = 2 has with the 16 x 16 products; the two are equally fast.
// KS = 2 (with M32): eight waves; waves 0-3 walk the first half of the block's key tiles and
// waves 4-7, with the same rows, the second half, each four with tiles of their own in LDS;
// at the end the two partial results are combined through LDS. Twice the waves for the same
// number of workgroups: for launches whose workgroups are too few, or too uneven (a prompt
// from its start: the last block sees all keys, the first none), to fill the GPU otherwise.
template <int RT, bool PAIR, bool M32, int KS>
__global__ void __launch_bounds__(256 * KS)
paged_attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_pool,
                          const bf16* __restrict__ v_pool, const int* __restrict__ block_table,
                          int table_width, const int* __restrict__ token_rows,
                          const int* __restrict__ positions, const int* __restrict__ row_blocks,
                          bf16* __restrict__ out, int Hq, int Hkv, int BS, int bs_shift, float scale,
                          int window, int group_pad_log2) {
    static_assert(D <= 128, "one key pair per thread");
    static_assert(KS == 1 || (KS == 2 && M32), "key halves come with the 32-row products");
    constexpr int PF_TILE_ELEMS = PF_K_ELEMS + PF_V_ELEMS;          // one K tile and one V^T tile
    __shared__ __attribute__((aligned(16))) uint16_t tiles_lds[KS * 2 * PF_TILE_ELEMS];
    const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x / SOC_WAVE), lane = threadIdx.x % SOC_WAVE;
    const int half = wave_all / 4, wave = wave_all % 4;             // which keys, which rows
    const int tid = threadIdx.x % 256;                              // among the four waves that share tiles
    uint16_t* const k_lds[2] = {tiles_lds + (half * 2) * PF_TILE_ELEMS, tiles_lds + (half * 2 + 1) * PF_TILE_ELEMS};
    uint16_t* const v_lds[2] = {k_lds[0] + PF_K_ELEMS, k_lds[1] + PF_K_ELEMS};
    const int li = lane % 16, kb = lane / 16;
    const int G = Hq / Hkv, Gp = 1 << group_pad_log2;
    const int chunks = (G + 15) / 16;
    // late row blocks see the most keys: they go first, so that the short ones fill the end
    const int blk = (int)(gridDim.x / (Hkv * chunks)) - 1 - (int)(blockIdx.x / (Hkv * chunks));
    const int kvh = (blockIdx.x / chunks) % Hkv, chunk = blockIdx.x % chunks;
    const int tok0 = row_blocks ? row_blocks[2 * blk] : blk, ntok = row_blocks ? row_blocks[2 * blk + 1] : 1;
    const int pos0 = positions[tok0];
    const int* table = block_table + (size_t)token_rows[tok0] * table_width;
    const int tokens_per_wave = ((M32 ? 32 : 16 * RT)) >> group_pad_log2;

    const int khi = pos0 + ntok;                                    // keys any row of the block sees
    const int kmin = window > 0 ? max(0, pos0 - window + 1) : 0;
    int klo = kmin & ~(PF_KEYS - 1);
    // kend: where this half's walk over the tiles ends. Both halves take the same number of
    // steps (they share the barriers); the second may run past khi, where keys are stand-ins
    // that no row sees.
    int kend = khi;
    if constexpr (KS == 2) {
        const int per_half = ((khi - klo + PF_KEYS - 1) / PF_KEYS + 1) / 2 * PF_KEYS;
        klo += half * per_half;
        kend = klo + per_half;
    }
    // this wave's rows
    const int wtok0 = wave * tokens_per_wave;                       // first token of the wave in the block
    const int wave_lo_pos = pos0 + wtok0;                           // its first and last positions
    const int wave_hi_pos = min(khi, wave_lo_pos + tokens_per_wave) - 1;
    const bool wave_has_rows = wtok0 < ntok;
    const float c2 = scale * 1.44269504088896340736f;               // to base 2

    int row_pos[RT];
    size_t row_q[RT];
    uint4 qf[RT][QK_STEPS];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int rho = rt * 16 + li;
        const int tt = wtok0 + (rho >> group_pad_log2), g = chunk * 16 + (rho & (Gp - 1));
        const bool ok = tt < ntok && g < G;
        row_pos[rt] = ok ? pos0 + tt : -1;
        row_q[rt] = ((size_t)(tok0 + (ok ? tt : 0)) * Hq + (size_t)kvh * G + (ok ? g : 0)) * D;
#pragma unroll
        for (int kk = 0; kk < QK_STEPS; ++kk)
            qf[rt][kk] = ok ? load_qk_slice(q + row_q[rt], kk, kb) : make_uint4(0u, 0u, 0u, 0u);
    }
    f32x4_t o[RT][DV];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        m[rt] = -INFINITY; l[rt] = 0.f;
#pragma unroll
        for (int j = 0; j < DV; ++j) o[rt][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    }
    // 32-row products: the lane's row is lane % 32, its half of every 16-wide k step lane / 32
    constexpr int DQ32 = D / 16, DB32 = D / 32;
    const int c32 = lane % 32, g32 = lane / 32;
    int row_pos32 = -1;
    size_t row_q32 = 0;
    uint4 qf32[M32 ? DQ32 : 1];                           // the lane's slices of its query row
    f32x16_t o32[M32 ? DB32 : 1];
    float m32 = -INFINITY, l32 = 0.f;
    if constexpr (M32) {
        const int tt = wtok0 + (c32 >> group_pad_log2), gh = chunk * 16 + (c32 & (Gp - 1));
        const bool ok = tt < ntok && gh < G;
        row_pos32 = ok ? pos0 + tt : -1;
        row_q32 = ((size_t)(tok0 + (ok ? tt : 0)) * Hq + (size_t)kvh * G + (ok ? gh : 0)) * D;
#pragma unroll
        for (int t = 0; t < DQ32; ++t)
            qf32[t] = ok ? *reinterpret_cast<const uint4*>(q + row_q32 + 16 * t + 8 * g32) : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int b = 0; b < DB32; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) o32[b][i] = 0.f;
    }

    // Cooperative tile loads: a thread owns two neighbouring keys (2 kp, 2 kp + 1) and one
    // 16-byte part of them, of K and of V. Keys that no row of the block sees are never read;
    // zeros stand in for them.
    // Loads must stay in flight until their tile is moved to LDS, so nothing touches what
    // they bring before that: no branch around a load, no select on its result. A key that
    // must not be read is redirected to the first entry of the row's table (a page of the
    // pool whatever it holds) and becomes zeros when the tile is stored to LDS. Threads past
    // the parts of a key (head sizes under 128) load a part again and store nothing.
    const int kp = tid % 16, part = tid / 16;
    const bool loader = part < PF_PARTS;
    const int part_ld = PF_PARTS == 16 ? part : part % PF_PARTS;
    const size_t page_stride = (size_t)Hkv * BS * D;
    const bf16* k_base = k_pool + (size_t)kvh * BS * D + part_ld * 8;
    const bf16* v_base = v_pool + (size_t)kvh * BS * D + part_ld * 8;
    auto lookup = [&](int key0, int (&pg)[2]) {
        if constexpr (PAIR) {
            const int key = key0 + 2 * kp;
            const bool ok = key + 1 >= kmin && key < khi;
            pg[0] = pg[1] = table[ok ? key >> bs_shift : 0];
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int key = key0 + 2 * kp + h;
                const bool ok = key >= kmin && key < khi;
                pg[h] = table[ok ? (bs_shift >= 0 ? key >> bs_shift : key / BS) : 0];
            }
        }
    };
    auto fetch = [&](int key0, const int (&pg)[2], uint4 (&kr)[2], uint4 (&vr)[2]) {
        if constexpr (PAIR) {
            const size_t off = (size_t)pg[0] * page_stride + (size_t)(((key0 + 2 * kp) & (BS - 1)) * D);
            kr[0] = *reinterpret_cast<const uint4*>(k_base + off);
            kr[1] = *reinterpret_cast<const uint4*>(k_base + off + D);
            vr[0] = *reinterpret_cast<const uint4*>(v_base + off);
            vr[1] = *reinterpret_cast<const uint4*>(v_base + off + D);
        } else {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int key = key0 + 2 * kp + h;
                const int in_page = bs_shift >= 0 ? key & (BS - 1) : key % BS;
                const size_t off = (size_t)pg[h] * page_stride + (size_t)(in_page * D);
                kr[h] = *reinterpret_cast<const uint4*>(k_base + off);
                vr[h] = *reinterpret_cast<const uint4*>(v_base + off);
            }
        }
    };
    auto stash = [&](int buf, int key0, const uint4 (&kr)[2], const uint4 (&vr)[2]) {
        if (!loader) return;
        uint4 k0 = kr[0], k1 = kr[1], v0 = vr[0], v1 = vr[1];
        if (key0 < kmin || key0 + PF_KEYS > khi) {           // uniform: a tile at an edge of the range
            const int key = key0 + 2 * kp;
            if (key < kmin || key >= khi) { k0 = make_uint4(0u, 0u, 0u, 0u); v0 = k0; }
            if (key + 1 < kmin || key + 1 >= khi) { k1 = make_uint4(0u, 0u, 0u, 0u); v1 = k1; }
        }
        const int r0 = M32 ? pf_k_row32(2 * kp) : pf_k_row(2 * kp), r1 = M32 ? pf_k_row32(2 * kp + 1) : pf_k_row(2 * kp + 1);
        *reinterpret_cast<uint4*>(&k_lds[buf][r0 * PF_K_STRIDE + part * 8]) = k0;
        *reinterpret_cast<uint4*>(&k_lds[buf][r1 * PF_K_STRIDE + part * 8]) = k1;
        const uint32_t a[4] = {v0.x, v0.y, v0.z, v0.w};
        const uint32_t b[4] = {v1.x, v1.y, v1.z, v1.w};
        uint32_t* vt = reinterpret_cast<uint32_t*>(&v_lds[buf][(part * 8) * PF_V_STRIDE + 2 * kp]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            // element 2e and 2e+1 of both keys: (key 2kp in the low half, key 2kp+1 in the high)
            vt[(2 * e) * (PF_V_STRIDE / 2)] = __builtin_amdgcn_perm(b[e], a[e], 0x05040100u);
            vt[(2 * e + 1) * (PF_V_STRIDE / 2)] = __builtin_amdgcn_perm(b[e], a[e], 0x07060302u);
        }
    };

    // One tile for this wave's rows, in two halves. The first: scores and softmax weights
    // (packed as operand B of the second product); MASKED: some key of the tile is hidden from
    // some row. The second half is one piece of code behind both variants, so that the
    // accumulators have one home: with the products inside the variants the compiler copied
    // all accumulators at every join.
    auto scores = [&](int key0, int buf, auto masked_tag, uint4 (&pf)[RT], float (&alpha)[RT], bool& any_rescale) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const uint16_t* kt = k_lds[buf];
        uint4 ka[QK_STEPS], kc[QK_STEPS];
#pragma unroll
        for (int kk = 0; kk < QK_STEPS; ++kk) {
            ka[kk] = load_qk_slice(reinterpret_cast<const bf16*>(kt + li * PF_K_STRIDE), kk, kb);
            kc[kk] = load_qk_slice(reinterpret_cast<const bf16*>(kt + (16 + li) * PF_K_STRIDE), kk, kb);
        }
        any_rescale = false;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            f32x4_t s0 = (f32x4_t){0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
            for (int kk = 0; kk < QK_STEPS; ++kk) {
                s0 = qk_mfma(ka[kk], qf[rt][kk], s0);
                s1 = qk_mfma(kc[kk], qf[rt][kk], s1);
            }
            float t[8];
            float mx = -INFINITY;                           // of the raw scores: the scale is positive
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                t[r] = r < 4 ? s0[r & 3] : s1[r & 3];
                if constexpr (MASKED) {
                    const int key = key0 + 8 * kb + r;
                    bool seen = key <= row_pos[rt];
                    if (window > 0) seen = seen && key > row_pos[rt] - window;
                    t[r] = seen ? t[r] : -INFINITY;
                }
                mx = fmaxf(mx, t[r]);
            }
            mx = max_xor32(max_xor16(mx)) * c2;
            // m is the row's reference for the exponentials, moved only when a tile's maximum
            // lies more than LAZY_MAX above it (see the 32-row form)
            const bool move = mx > m[rt] + LAZY_MAX;
            const float mn = move ? mx : m[rt];
            const float ms = mn == -INFINITY ? 0.f : mn;
            alpha[rt] = move ? __builtin_amdgcn_exp2f(m[rt] - ms) : 1.f;
            float p[8];
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(t[r], c2, -ms));
                psum += p[r];
            }
            l[rt] = l[rt] * alpha[rt] + psum;
            any_rescale = any_rescale || move;
            m[rt] = mn;
            pf[rt] = make_uint4(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]),
                                pack_bf16x2(p[4], p[5]), pack_bf16x2(p[6], p[7]));
        }
    };
    auto weighted = [&](int buf, const uint4 (&pf)[RT], const float (&alpha)[RT], bool any_rescale) {
        const uint16_t* vt = v_lds[buf];
        if (__any(any_rescale)) rescale_in_place(o, alpha);
        // O^T += V^T P^T over the 32 keys, one 16-wide block of d at a time
        uint4 va[DV];
#pragma unroll
        for (int j = 0; j < DV; ++j) {
            const uint2* src = reinterpret_cast<const uint2*>(vt + (j * 16 + li) * PF_V_STRIDE + 8 * kb);
            const uint2 lo = src[0], hi = src[1];
            va[j] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
#pragma unroll
        for (int j = 0; j < DV; ++j)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                o[rt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    *reinterpret_cast<const bf16x8_t*>(&va[j]), *reinterpret_cast<const bf16x8_t*>(&pf[rt]),
                    o[rt][j], 0, 0, 0);
    };

    // The same with 32 rows per wave: S^T [32 keys x 32 rows] from D / 16 products, a row's
    // scores in two lanes (16 each), O^T [32 d x 32 rows] per 32-wide block of d.
    auto scores32 = [&](int key0, int buf, auto masked_tag, uint4 (&pf)[2], float& alpha, bool& rescale) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const uint16_t* kt = k_lds[buf];
        f32x16_t sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
#pragma unroll
        for (int t = 0; t < DQ32; ++t) {
            const uint4 ka = *reinterpret_cast<const uint4*>(kt + c32 * PF_K_STRIDE + 16 * t + 8 * g32);
            sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8_t*>(&ka),
                                                         *reinterpret_cast<const bf16x8_t*>(&qf32[t]), sc, 0, 0, 0);
        }
        float mx = -INFINITY;                               // of the raw scores: the scale is positive
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if constexpr (MASKED) {
                const int key = key0 + 16 * (i / 8) + 8 * g32 + i % 8;
                bool seen = key <= row_pos32;
                if (window > 0) seen = seen && key > row_pos32 - window;
                sc[i] = seen ? sc[i] : -INFINITY;
            }
            mx = fmaxf(mx, sc[i]);
        }
        mx = max_xor32(mx) * c2;
        // m32 is the row's reference for the exponentials, not its maximum: it moves only when
        // a tile's maximum lies more than LAZY_MAX above it, so the accumulators are rescaled a
        // few times per row instead of in most tiles; weights stay below 2^LAZY_MAX
        rescale = mx > m32 + LAZY_MAX;
        const float mn = rescale ? mx : m32;
        const float ms = mn == -INFINITY ? 0.f : mn;
        alpha = rescale ? __builtin_amdgcn_exp2f(m32 - ms) : 1.f;
        float p[16];
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            p[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], c2, -ms));
            psum += p[i];
        }
        l32 = l32 * alpha + psum;
        m32 = mn;
#pragma unroll
        for (int h = 0; h < 2; ++h)
            pf[h] = make_uint4(pack_bf16x2(p[8 * h], p[8 * h + 1]), pack_bf16x2(p[8 * h + 2], p[8 * h + 3]),
                               pack_bf16x2(p[8 * h + 4], p[8 * h + 5]), pack_bf16x2(p[8 * h + 6], p[8 * h + 7]));
    };
    auto weighted32 = [&](int buf, const uint4 (&pf)[2], float alpha, bool rescale) {
        const uint16_t* vt = v_lds[buf];
        if (__any(rescale)) {                               // rare; in place (see scale_in_place)
            scale_fence();
#pragma unroll
            for (int b = 0; b < DB32; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float v = o32[b][i];
                    scale_in_place(v, alpha);
                    o32[b][i] = v;
                }
            scale_fence();
        }
#pragma unroll
        for (int b = 0; b < DB32; ++b) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint2* src = reinterpret_cast<const uint2*>(vt + (32 * b + c32) * PF_V_STRIDE + 16 * h + 8 * g32);
                const uint2 lo = src[0], hi = src[1];
                const uint4 va = make_uint4(lo.x, lo.y, hi.x, hi.y);
                o32[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8_t*>(&va),
                                                                  *reinterpret_cast<const bf16x8_t*>(&pf[h]), o32[b], 0, 0, 0);
            }
        }
    };

    // Two tiles of global loads are in flight while one is computed: at the top of the
    // iteration of tile t, tile t sits in LDS buffer t % 2, the loads of tile t + 1 are on
    // their way into one pair of staging registers, and the pages of tile t + 2 were asked
    // for. The iteration issues the lookup of tile t + 3 and the loads of tile t + 2, computes,
    // and then moves tile t + 1 from its registers to the other LDS buffer, which nobody has
    // read since the barrier that ended the previous iteration. Loads return in order, so a
    // lookup is issued before the tile loads of its iteration: waiting for it then leaves
    // those in flight. Lookups may run past the end of the range (redirected); tile loads do
    // not: the main loop takes the rounds in which both buffers have a tile to load, and
    // the last tiles (at most three) follow without a loop.
    auto tile = [&](int key0, int buf) {
        if (wave_has_rows && key0 <= wave_hi_pos) {
            // whole: every key of the tile is at or before the wave's first position and inside
            // the window of its last one
            const bool whole = key0 + PF_KEYS - 1 <= wave_lo_pos &&
                               (window <= 0 || key0 > wave_hi_pos - window);
            if constexpr (M32) {
                uint4 pf[2];
                float alpha;
                bool rescale;
                if (whole) scores32(key0, buf, std::false_type{}, pf, alpha, rescale);
                else scores32(key0, buf, std::true_type{}, pf, alpha, rescale);
                weighted32(buf, pf, alpha, rescale);
            } else {
                uint4 pf[RT];
                float alpha[RT];
                bool any_rescale;
                if (whole) scores(key0, buf, std::false_type{}, pf, alpha, any_rescale);
                else scores(key0, buf, std::true_type{}, pf, alpha, any_rescale);
                weighted(buf, pf, alpha, any_rescale);
            }
        }
    };
    int pg0[2], pg1[2];
    uint4 kr0[2], vr0[2], kr1[2], vr1[2];
    lookup(klo, pg0);
    lookup(klo + PF_KEYS, pg1);
    fetch(klo, pg0, kr0, vr0);
    lookup(klo + 2 * PF_KEYS, pg0);
    if (klo + PF_KEYS < kend) fetch(klo + PF_KEYS, pg1, kr1, vr1);
    stash(0, klo, kr0, vr0);
    __syncthreads();
    int key0 = klo;
    for (; key0 + 3 * PF_KEYS < kend; key0 += 2 * PF_KEYS) {
        lookup(key0 + 3 * PF_KEYS, pg1);
        fetch(key0 + 2 * PF_KEYS, pg0, kr0, vr0);
        tile(key0, 0);
        stash(1, key0 + PF_KEYS, kr1, vr1);
        __syncthreads();
        lookup(key0 + 4 * PF_KEYS, pg0);
        fetch(key0 + 3 * PF_KEYS, pg1, kr1, vr1);
        tile(key0 + PF_KEYS, 1);
        stash(0, key0 + 2 * PF_KEYS, kr0, vr0);
        __syncthreads();
    }
    const bool has1 = key0 + PF_KEYS < kend, has2 = key0 + 2 * PF_KEYS < kend;    // the same in all threads
    if (has2) fetch(key0 + 2 * PF_KEYS, pg0, kr0, vr0);
    tile(key0, 0);
    if (has1) {
        stash(1, key0 + PF_KEYS, kr1, vr1);
        __syncthreads();
        tile(key0 + PF_KEYS, 1);
        if (has2) {
            stash(0, key0 + 2 * PF_KEYS, kr0, vr0);
            __syncthreads();
            tile(key0 + 2 * PF_KEYS, 0);
        }
    }

    if constexpr (M32) {
        float L = sum_xor32(l32);
        if constexpr (KS == 2) {
            // the second half hands its result over: [wave][value][lane] floats where the tiles were
            static_assert(KS * 2 * PF_TILE_ELEMS * 2 >= 4 * 64 * (16 * DB32 + 2) * 4, "the tiles' space holds the exchange");
            float* xch = reinterpret_cast<float*>(tiles_lds) + (size_t)wave * (16 * DB32 + 2) * 64 + lane;
            __syncthreads();                                 // every wave is done with the tiles
            if (half == 1) {
#pragma unroll
                for (int b = 0; b < DB32; ++b)
#pragma unroll
                    for (int i = 0; i < 16; ++i) xch[(16 * b + i) * 64] = o32[b][i];
                xch[(16 * DB32) * 64] = m32;
                xch[(16 * DB32 + 1) * 64] = L;
            }
            __syncthreads();
            if (half == 1) return;
            const float m_b = xch[(16 * DB32) * 64], l_b = xch[(16 * DB32 + 1) * 64];
            const float mn = fmaxf(m32, m_b);
            const float ms = mn == -INFINITY ? 0.f : mn;
            const float wa = __builtin_amdgcn_exp2f(m32 - ms), wb = __builtin_amdgcn_exp2f(m_b - ms);
            L = L * wa + l_b * wb;
#pragma unroll
            for (int b = 0; b < DB32; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) o32[b][i] = o32[b][i] * wa + xch[(16 * b + i) * 64] * wb;
        }
        if (row_pos32 >= 0) {
            const float inv = L > 0.f ? 1.0f / L : 0.f;
#pragma unroll
            for (int b = 0; b < DB32; ++b)
#pragma unroll
                for (int a = 0; a < 4; ++a) {                 // o32[b][4a + j] is d = 32 b + 8 a + 4 g32 + j
                    uint2 pk;
                    pk.x = pack_bf16x2(o32[b][4 * a] * inv, o32[b][4 * a + 1] * inv);
                    pk.y = pack_bf16x2(o32[b][4 * a + 2] * inv, o32[b][4 * a + 3] * inv);
                    *reinterpret_cast<uint2*>(out + row_q32 + 32 * b + 8 * a + 4 * g32) = pk;
                }
        }
        return;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float L = l[rt];
        L = sum_xor32(sum_xor16(L));
        if (row_pos[rt] < 0) continue;
        const float inv = L > 0.f ? 1.0f / L : 0.f;
#pragma unroll
        for (int j = 0; j < DV; ++j) {
            uint2 pk;
            pk.x = pack_bf16x2(o[rt][j][0] * inv, o[rt][j][1] * inv);
            pk.y = pack_bf16x2(o[rt][j][2] * inv, o[rt][j][3] * inv);
            *reinterpret_cast<uint2*>(out + row_q[rt] + j * 16 + 4 * kb) = pk;
        }
    }
}

// bfloat16 only, head sizes up to 128, no key splits. row_blocks [n_row_blocks, 2] = (first
// token, tokens) of each block of at most 4 * ((16 * row_tiles) >> group_pad_log2) tokens of
// one sequence, or null: every token is a block of its own. row_tiles 32: a wave owns 32 rows
// (blocks of at most 4 * (32 >> group_pad_log2) tokens), head sizes that are multiples of 32;
// row_tiles 64: the same with eight waves, four for each half of a block's keys.
SOC_EXPORT int soc_paged_attention_prefill(const void* q, const void* k_pool, const void* v_pool,
                                           const int* block_table, int table_width, const int* token_rows,
                                           const int* positions, const int* row_blocks, int n_row_blocks,
                                           void* out, int N, int Hq, int Hkv, int BS, float scale,
                                           int window, int row_tiles, int group_pad_log2,
                                           hipStream_t stream) {
    if (N <= 0 || n_row_blocks <= 0) return 0;
    if (Hkv < 1 || Hq % Hkv || BS < 1) return (int)hipErrorInvalidValue;
    if (!(scale > 0.f)) return (int)hipErrorInvalidValue;        // the maximum is taken of the raw scores
    if (!row_blocks && n_row_blocks != N) return (int)hipErrorInvalidValue;
    const int G = Hq / Hkv;
    if ((1 << group_pad_log2) < (G < 16 ? G : 16) || group_pad_log2 > 4) return (int)hipErrorInvalidValue;
    const long groups = (long)n_row_blocks * Hkv * ((G + 15) / 16);
    if (groups > 0x7fffffffL) return (int)hipErrorInvalidValue;
    int bs_shift = -1;
    if ((BS & (BS - 1)) == 0)
        for (bs_shift = 0; (1 << bs_shift) < BS; ++bs_shift) {}
    if constexpr (D <= 128) {
#define SOC_PF_ARGS (const bf16*)q, (const bf16*)k_pool, (const bf16*)v_pool, block_table, table_width, \
        token_rows, positions, row_blocks, (bf16*)out, Hq, Hkv, BS, bs_shift, scale, window, group_pad_log2
        const bool pair = bs_shift >= 1;
#define SOC_PF_LAUNCH(RT_, M32_, KS_)                                                                            \
    do {                                                                                                    \
        if (pair) hipLaunchKernelGGL((paged_attn_prefill_kernel<RT_, true, M32_, KS_>), dim3((unsigned)groups), dim3(256 * KS_), 0, stream, SOC_PF_ARGS); \
        else hipLaunchKernelGGL((paged_attn_prefill_kernel<RT_, false, M32_, KS_>), dim3((unsigned)groups), dim3(256 * KS_), 0, stream, SOC_PF_ARGS);     \
    } while (0)
        if (row_tiles == 1) SOC_PF_LAUNCH(1, false, 1);
        else if (row_tiles == 2) SOC_PF_LAUNCH(2, false, 1);
        else if (row_tiles == 32 || row_tiles == 64) {       // 32 rows per wave through the 32 x 32 products
            if constexpr (D % 32 == 0) {
                if (row_tiles == 32) SOC_PF_LAUNCH(1, true, 1);
                else SOC_PF_LAUNCH(1, true, 2);              // and the keys of a block in two halves
            } else return (int)hipErrorInvalidValue;
        } else return (int)hipErrorInvalidValue;
#undef SOC_PF_LAUNCH
#undef SOC_PF_ARGS
        return soc_last_error();
    } else {
        return (int)hipErrorInvalidValue;
    }
}

SOC_EXPORT int soc_attention_head_dim() { return D; }
