// Memory-bound kernels between the matrix products: embedding gather, RMSNorm with
// the residual sum fused in, per-head QK-norm + rotary encoding + cache-page write,
// SwiGLU. Statistics, angles and sums are float32; a result is rounded once when it
// is stored in bfloat16. The residual stream is float32.
//
// Formulas: model/qwen/qwen_kv_cont.py:45-77, 250-266 and
// model/qwen/qwen_kv_paged.py:111-127, 147-156 of the reference.
#include "common.h"

// ---------------------------------------------------------------------------------------------
// out[n, :] = table[ids[n], :] as float32 (start of the residual stream)
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int d, int V) {
    const int n = blockIdx.x;
    int id = ids[n];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);          // the host checks ids; never read outside
    const T* row = table + (size_t)id * d;
    float* o = out + (size_t)n * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) o[i] = to_float(row[i]);
}

SOC_EXPORT int soc_embedding(const int* ids, const void* table, float* out, int N, int d, int V,
                             int table_dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (table_dtype == 0)
        hipLaunchKernelGGL(embedding_kernel<float>, dim3(N), dim3(256), 0, stream, ids,
                           (const float*)table, out, d, V);
    else
        hipLaunchKernelGGL(embedding_kernel<bf16>, dim3(N), dim3(256), 0, stream, ids,
                           (const bf16*)table, out, d, V);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// In place: r = residual[n] + delta[n]; residual[n] = r; out[n] = r / sqrt(mean(r^2) + eps) * w.
// With `rows`: n = rows[i], nothing is written back, out has one row per index.
// delta is either one tensor [N, d] of the compute type, or n_partials float32 tensors
// [n_partials, N, d] (split-K partial sums of a matrix product) that are added in order.
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                   const float* __restrict__ partials, int n_partials,
                                   size_t partial_stride, const float* __restrict__ w,
                                   T* __restrict__ out, const int* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int n = rows ? rows[i] : i;
    float* r = residual + (size_t)n * d;
    const T* dl = delta ? delta + (size_t)n * d : nullptr;
    const float* dp = partials ? partials + (size_t)n * d : nullptr;
    T* o = out + (size_t)i * d;
    const bool adds = dl || dp;
    auto summed = [&](int j) {
        float v = r[j];
        if (dl) v += to_float(dl[j]);
        if (dp) for (int s = 0; s < n_partials; ++s) v += dp[s * partial_stride + j];
        return v;
    };
    float ss = 0.f;
    for (int j = threadIdx.x; j < d; j += blockDim.x) {
        const float v = summed(j);
        if (!rows && adds) r[j] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    for (int j = threadIdx.x; j < d; j += blockDim.x) {
        const float v = (rows && adds) ? summed(j) : r[j];
        o[j] = from_float<T>(v * inv * w[j]);
    }
}

// The same in one pass for rows of at most VPT * blockDim elements: a thread keeps its
// elements in registers between the sum of squares and the scaling.
template <typename T, int VPT>
__global__ void add_rmsnorm_regs_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                        const float* __restrict__ partials, int n_partials,
                                        size_t partial_stride, const float* __restrict__ w,
                                        T* __restrict__ out, const int* __restrict__ rows, int d, float eps) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int n = rows ? rows[i] : i;
    float* r = residual + (size_t)n * d;
    const T* dl = delta ? delta + (size_t)n * d : nullptr;
    const float* dp = partials ? partials + (size_t)n * d : nullptr;
    float v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
        const int j = threadIdx.x + u * blockDim.x;
        v[u] = 0.f;
        if (j < d) {
            v[u] = r[j];
            if (dl) v[u] += to_float(dl[j]);
            if (dp) for (int s = 0; s < n_partials; ++s) v[u] += dp[s * partial_stride + j];
            if (!rows && (dl || dp)) r[j] = v[u];
        }
        ss += v[u] * v[u];
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    T* o = out + (size_t)i * d;
#pragma unroll
    for (int u = 0; u < VPT; ++u) {
        const int j = threadIdx.x + u * blockDim.x;
        if (j < d) o[j] = from_float<T>(v[u] * inv * w[j]);
    }
}

// The same with eight consecutive elements per thread and 16-byte accesses, for rows of a
// multiple of eight elements up to 8 * 1024: fewer, wider loads, all issued before the first
// is needed. blockDim = d / 8 rounded up to whole waves.
template <typename T>
__global__ void __launch_bounds__(1024)
add_rmsnorm_vec8_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                        const float* __restrict__ partials, int n_partials, size_t partial_stride,
                        const float* __restrict__ w, T* __restrict__ out, const int* __restrict__ rows,
                        int d, float eps, int tile_rows) {
    __shared__ float scratch[16];
    const int i = blockIdx.x;
    const int n = rows ? rows[i] : i;
    const int j = threadIdx.x * 8;
    const bool in = j < d;
    float v[8], g[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = g[e] = 0.f;
    if (in) {
        float* r = residual + (size_t)n * d + j;
        VecLoad<float, 8>::load(r, v);
        VecLoad<float, 8>::load(w + j, g);
        if (delta) {
            float t[8];
            VecLoad<T, 8>::load(delta + (size_t)n * d + j, t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += t[e];
        }
        if (partials) {
            const float* dp = partials + (size_t)n * d + j;
            for (int s = 0; s < n_partials; ++s) {
                float t[8];
                VecLoad<float, 8>::load(dp + s * partial_stride, t);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += t[e];
            }
        }
        if (!rows && (delta || partials)) {
            *reinterpret_cast<float4*>(r) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4*>(r + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    if (!in) return;
    // tile_rows R > 0 (d a multiple of 32): out is laid out [d / 32][R][32] for a product that
    // reads 64 bytes of each of its rows side by side
    T* o = tile_rows > 0 ? out + ((size_t)(j / 32) * tile_rows + i) * 32 + j % 32 : out + (size_t)i * d + j;
    if constexpr (sizeof(T) == 2) {
        uint4 pk;
        pk.x = pack_bf16x2(v[0] * inv * g[0], v[1] * inv * g[1]);
        pk.y = pack_bf16x2(v[2] * inv * g[2], v[3] * inv * g[3]);
        pk.z = pack_bf16x2(v[4] * inv * g[4], v[5] * inv * g[5]);
        pk.w = pack_bf16x2(v[6] * inv * g[6], v[7] * inv * g[7]);
        *reinterpret_cast<uint4*>(o) = pk;
    } else {
        float* of = reinterpret_cast<float*>(o);
        *reinterpret_cast<float4*>(of) = make_float4(v[0] * inv * g[0], v[1] * inv * g[1], v[2] * inv * g[2], v[3] * inv * g[3]);
        *reinterpret_cast<float4*>(of + 4) = make_float4(v[4] * inv * g[4], v[5] * inv * g[5], v[6] * inv * g[6], v[7] * inv * g[7]);
    }
}

template <typename T>
static int launch_add_rmsnorm(float* residual, const void* delta, const float* partials, int n_partials,
                              size_t partial_stride, const float* w, void* out, const int* rows, int n_out,
                              int d, float eps, int tile_rows, hipStream_t stream) {
    constexpr int VPT = 8;
    const int threads = d <= 1024 ? 128 : (d <= 2048 ? 256 : (d <= 4096 ? 512 : 1024));
    const bool aligned = d % 8 == 0 && partial_stride % 4 == 0 &&
                         ((uintptr_t)residual | (uintptr_t)delta | (uintptr_t)partials | (uintptr_t)w | (uintptr_t)out) % 16 == 0;
    if (tile_rows > 0 && !(aligned && d <= 8 * 1024 && d % 32 == 0 && n_out <= tile_rows))
        return (int)hipErrorInvalidValue;                // only the 16-byte form lays its output out by tile
    if (aligned && d <= 8 * 1024)
        hipLaunchKernelGGL(add_rmsnorm_vec8_kernel<T>, dim3(n_out), dim3((d / 8 + 63) / 64 * 64), 0, stream, residual,
                           (const T*)delta, partials, n_partials, partial_stride, w, (T*)out, rows, d, eps, tile_rows);
    else if (d <= VPT * threads)
        hipLaunchKernelGGL((add_rmsnorm_regs_kernel<T, VPT>), dim3(n_out), dim3(threads), 0, stream, residual,
                           (const T*)delta, partials, n_partials, partial_stride, w, (T*)out, rows, d, eps);
    else
        hipLaunchKernelGGL(add_rmsnorm_kernel<T>, dim3(n_out), dim3(1024), 0, stream, residual, (const T*)delta,
                           partials, n_partials, partial_stride, w, (T*)out, rows, d, eps);
    return 0;
}

// tile_rows R > 0: out is written [d / 32][R][32] (R >= n_out; d a multiple of 32, at most 8,192,
// 16-byte aligned operands) instead of [n_out][d].
SOC_EXPORT int soc_add_rmsnorm(float* residual, const void* delta, const float* partials, int n_partials,
                               long long partial_stride, const float* w, void* out, const int* rows,
                               int n_out, int d, float eps, int dtype, int tile_rows, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (delta && partials) return (int)hipErrorInvalidValue;
    const int refused = dtype == 0
        ? launch_add_rmsnorm<float>(residual, delta, partials, n_partials, (size_t)partial_stride, w, out, rows,
                                    n_out, d, eps, tile_rows, stream)
        : launch_add_rmsnorm<bf16>(residual, delta, partials, n_partials, (size_t)partial_stride, w, out, rows,
                                   n_out, d, eps, tile_rows, stream);
    return refused ? refused : soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Plain RMSNorm over rows of `dim` elements, one wave per row.
template <typename T>
__global__ void rmsnorm_rows_kernel(const T* __restrict__ x, const float* __restrict__ w,
                                    T* __restrict__ out, int R, int dim, float eps) {
    const int row = blockIdx.x * (blockDim.x / SOC_WAVE) + threadIdx.x / SOC_WAVE;
    const int lane = threadIdx.x % SOC_WAVE;
    if (row >= R) return;
    const T* xr = x + (size_t)row * dim;
    T* o = out + (size_t)row * dim;
    float ss = 0.f;
    for (int j = lane; j < dim; j += SOC_WAVE) { float v = to_float(xr[j]); ss += v * v; }
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
    for (int j = lane; j < dim; j += SOC_WAVE) o[j] = from_float<T>(to_float(xr[j]) * inv * w[j]);
}

SOC_EXPORT int soc_rmsnorm(const void* x, const float* w, void* out, int R, int dim, float eps,
                           int dtype, hipStream_t stream) {
    if (R <= 0) return 0;
    const int grid = (R + 3) / 4;
    if (dtype == 0)
        hipLaunchKernelGGL(rmsnorm_rows_kernel<float>, dim3(grid), dim3(256), 0, stream,
                           (const float*)x, w, (float*)out, R, dim, eps);
    else
        hipLaunchKernelGGL(rmsnorm_rows_kernel<bf16>, dim3(grid), dim3(256), 0, stream,
                           (const bf16*)x, w, (bf16*)out, R, dim, eps);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// out[n, j] = silu(gate[n, j]) * up[n, j],  silu(z) = z / (1 + exp(-z)). gate_up holds
// [gate | up] halves (interleave 0), or gate and up columns alternating in blocks of
// `interleave` (the layout of a fused weight whose rows alternate that way).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, size_t total, int ff,
                              int interleave) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < total; i += stride) {
        const size_t n = i / ff, j = i % ff;
        size_t gi, ui;
        if (interleave > 0) {
            gi = (j / interleave) * 2 * interleave + j % interleave;
            ui = gi + interleave;
        } else {
            gi = j; ui = ff + j;
        }
        const float g = to_float(gate_up[n * 2 * ff + gi]);
        const float u = to_float(gate_up[n * 2 * ff + ui]);
        out[i] = from_float<T>(u * (g / (1.0f + expf(-g))));
    }
}

// Eight columns per thread with 16-byte loads (bfloat16) when the layout allows: ff and the
// interleave block are multiples of 8, so eight consecutive outputs share one gate run and
// one up run.
__global__ void swiglu_bf16x8_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, size_t groups,
                                     int ff, int interleave) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const int per_row = ff / 8;
    for (; i < groups; i += stride) {
        const size_t n = i / per_row;
        const int j = (int)(i % per_row) * 8;
        size_t gi, ui;
        if (interleave > 0) { gi = (size_t)(j / interleave) * 2 * interleave + j % interleave; ui = gi + interleave; }
        else { gi = j; ui = (size_t)ff + j; }
        float g[8], u[8];
        VecLoad<bf16, 8>::load(gate_up + n * 2 * ff + gi, g);
        VecLoad<bf16, 8>::load(gate_up + n * 2 * ff + ui, u);
        uint32_t pk[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = u[2 * e] * (g[2 * e] / (1.0f + expf(-g[2 * e])));
            const float b = u[2 * e + 1] * (g[2 * e + 1] / (1.0f + expf(-g[2 * e + 1])));
            pk[e] = (uint32_t)f32_to_bf16_bits(a) | ((uint32_t)f32_to_bf16_bits(b) << 16);
        }
        *reinterpret_cast<uint4*>(out + n * ff + j) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    }
}

// x = scale * x, then (cap > 0) x = cap * tanh(x / cap), in place on float32: what an
// architecture may ask for behind the embedding (a multiplier) and on the logits (a
// multiplier, a soft cap). The reference's model has neither.
__global__ void scale_softcap_kernel(float* __restrict__ x, size_t n, float scale, float cap) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        float v = x[i] * scale;
        if (cap > 0.f) v = cap * tanhf(v / cap);
        x[i] = v;
    }
}

SOC_EXPORT int soc_scale_softcap(float* x, long long n, float scale, float cap, hipStream_t stream) {
    if (n <= 0) return 0;
    if (cap < 0.f) return (int)hipErrorInvalidValue;
    size_t blocks = ((size_t)n + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, x, (size_t)n, scale, cap);
    return soc_last_error();
}

// Rows that are owed their norm's factor, settled: out[m][c] = x[m][c] / sqrt(sum_t ssq[m][t] /
// dim + eps), bfloat16 in and out, for a product that cannot apply the factor to its sums (a
// weight kept in float32, a float32 result). One workgroup per row; every thread adds the row's
// partial sums in the same order.
__global__ void settle_owed_kernel(const bf16* __restrict__ x, const float* __restrict__ ssq, int tiles,
                                   int ssq_stride, bf16* __restrict__ out, int dim, float eps) {
    const int m = blockIdx.x;
    float sum = 0.f;
    for (int t = 0; t < tiles; ++t) sum += ssq[(size_t)m * ssq_stride + t];
    const float factor = rsqrtf(sum / (float)dim + eps);
    for (int c = threadIdx.x; c < dim; c += blockDim.x)
        out[(size_t)m * dim + c] = from_float<bf16>(to_float(x[(size_t)m * dim + c]) * factor);
}

SOC_EXPORT int soc_settle_owed(const void* x, const float* ssq, int tiles, int ssq_stride, void* out, int M,
                               int dim, float eps, hipStream_t stream) {
    if (M <= 0 || dim <= 0) return 0;
    if (tiles < 1 || ssq_stride < tiles) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(settle_owed_kernel, dim3((unsigned)M), dim3(256), 0, stream, (const bf16*)x, ssq, tiles,
                       ssq_stride, (bf16*)out, dim, eps);
    return soc_last_error();
}

SOC_EXPORT int soc_swiglu(const void* gate_up, void* out, int N, int ff, int interleave, int dtype,
                          hipStream_t stream) {
    const size_t total = (size_t)N * ff;
    if (total == 0) return 0;
    if (interleave < 0 || (interleave > 0 && ff % interleave)) return (int)hipErrorInvalidValue;
    if (dtype == 1 && ff % 8 == 0 && interleave % 8 == 0) {
        const size_t groups = total / 8;
        size_t vblocks = (groups + 255) / 256;
        if (vblocks > 65536) vblocks = 65536;
        hipLaunchKernelGGL(swiglu_bf16x8_kernel, dim3((unsigned)vblocks), dim3(256), 0, stream,
                           (const bf16*)gate_up, (bf16*)out, groups, ff, interleave);
        return soc_last_error();
    }
    size_t blocks = (total + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (dtype == 0)
        hipLaunchKernelGGL(swiglu_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           (const float*)gate_up, (float*)out, total, ff, interleave);
    else
        hipLaunchKernelGGL(swiglu_kernel<bf16>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           (const bf16*)gate_up, (bf16*)out, total, ff, interleave);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Per token and head of a packed [q heads | k heads | v heads] row: RMSNorm over the head
// (q and k only, if gains are given), rotate-half rotation at the token's position (q and k
// only, if inv_freq is given), then store: q to q_out; k and v into the cache pages of the
// token's row at its position, or to k_out / v_out when no pools are given.
// One wave per head. A workgroup of four waves takes 4 * heads_per_wave heads of one token:
// one head per wave for a decode step (few tokens: many small workgroups, one short pass),
// all heads of the token for prompt portions (fewer, fatter workgroups). A lane owns VE
// consecutive elements of the head (VE = 2 at head size 128: one 4-byte access).
#define SOC_MAX_HEAD 256

template <typename T, int VE>
__global__ void __launch_bounds__(256)
qk_norm_rope_kernel(const T* __restrict__ qkv, T* __restrict__ q_out,
                                    T* __restrict__ k_out, T* __restrict__ v_out,
                                    T* __restrict__ k_pool, T* __restrict__ v_pool,
                                    const int* __restrict__ block_table, int table_width,
                                    const int* __restrict__ token_rows,
                                    const int* __restrict__ positions,
                                    const float* __restrict__ q_gain, const float* __restrict__ k_gain,
                                    const float* __restrict__ inv_freq, int Hq, int Hkv, int D,
                                    int rotary_dim, int BS, float eps, int heads_per_wave) {
    __shared__ float cos_t[SOC_MAX_HEAD / 2], sin_t[SOC_MAX_HEAD / 2];
    const int n = blockIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / SOC_WAVE), lane = threadIdx.x % SOC_WAVE;
    const int heads = Hq + 2 * Hkv;
    const int half = rotary_dim / 2;
    const int e0 = lane * VE;                          // this lane's elements e0 .. e0 + VE - 1
    const bool lane_on = e0 < D;                       // D is a multiple of VE
    // A wave takes head after head (the same trip count for all waves); the next head's
    // load is issued before the current one is worked on, and the first before anything
    // that depends on the token's position.
    // (No branch around the load and nothing done to its result here, or the wave would wait
    // for it on the spot: a head or a lane outside reads a valid address and is dropped later.)
    auto load_head = [&](int it, float (&dst)[VE]) {
        const int h = min((blockIdx.y * heads_per_wave + it) * 4 + wave, heads - 1);
        VecLoad<T, VE>::load(qkv + ((size_t)n * heads + h) * D + (lane_on ? e0 : 0), dst);
    };
    float v[VE], nxt[VE];
    load_head(0, v);
    const int pos = positions ? positions[n] : 0;
    if (inv_freq) {
        // the token's angles once per workgroup (float32, accurate range reduction:
        // positions reach thousands of radians)
        if ((int)threadIdx.x < half) sincosf((float)pos * inv_freq[threadIdx.x], &sin_t[threadIdx.x], &cos_t[threadIdx.x]);
        __syncthreads();
    }
    size_t page_base = 0;
    if (k_pool) {
        const int page = block_table[(size_t)token_rows[n] * table_width + pos / BS];
        page_base = ((size_t)page * Hkv * BS + (size_t)(pos % BS)) * D;
    }
    for (int it = 0; it < heads_per_wave; ++it) {
        load_head(it + 1, nxt);
        const int h = (blockIdx.y * heads_per_wave + it) * 4 + wave;
        const bool active = h < heads;
        const bool is_q = h < Hq, is_k = !is_q && h < Hq + Hkv;
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < VE; ++i) {
            if (!lane_on) v[i] = 0.f;                       // lanes past the head size add nothing
            ss += v[i] * v[i];
        }
        const float* gain = is_q ? q_gain : (is_k ? k_gain : nullptr);
        if (gain && active) {
            ss = wave_sum(ss);
            const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
            for (int i = 0; i < VE; ++i) if (lane_on) v[i] = v[i] * inv * gain[e0 + i];
        }
        if (inv_freq) {                                 // uniform over the wave
            // the partner of element e is e +- half: the same slot of the lane half / VE away
            // (half is a multiple of VE, checked by the launcher)
            const int shift = half / VE;
            const int src = e0 < half ? lane + shift : lane - shift;
#pragma unroll
            for (int i = 0; i < VE; ++i) {
                const float partner = __shfl(v[i], src & (SOC_WAVE - 1), SOC_WAVE);
                const int e = e0 + i;
                if (active && (is_q || is_k) && lane_on && e < rotary_dim) {
                    const int j = e < half ? e : e - half;
                    const float sn = sin_t[j], cs = cos_t[j];
                    v[i] = e < half ? v[i] * cs - partner * sn : v[i] * cs + partner * sn;
                }
            }
        }
        if (active && lane_on) {
            T* dst;
            if (is_q) dst = q_out + ((size_t)n * Hq + h) * D;
            else {
                const int kvh = is_k ? h - Hq : h - Hq - Hkv;
                if (k_pool) dst = (is_k ? k_pool : v_pool) + page_base + (size_t)kvh * BS * D;
                else dst = (is_k ? k_out : v_out) + ((size_t)n * Hkv + kvh) * D;
            }
            if constexpr (VE == 1) {
                dst[e0] = from_float<T>(v[0]);
            } else if constexpr (sizeof(T) == 2) {
                uint32_t pk[VE / 2];
#pragma unroll
                for (int i = 0; i < VE / 2; ++i) pk[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
                if constexpr (VE == 2) *reinterpret_cast<uint32_t*>(dst + e0) = pk[0];
                else *reinterpret_cast<uint2*>(dst + e0) = make_uint2(pk[0], pk[1]);
            } else {
#pragma unroll
                for (int i = 0; i < VE; ++i) dst[e0 + i] = from_float<T>(v[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < VE; ++i) v[i] = nxt[i];
    }
}

// The same for many tokens, bfloat16, head sizes 64 and 128 and a rotation over the whole
// head (or none): a lane owns eight consecutive elements (16-byte accesses), LPH = D / 8
// lanes form a head and a wave works on 64 / LPH heads at once, which cuts the instructions
// per head by that factor (the one-head-per-wave kernel is bound by them on long prompts).
// Gains and the token's sines and cosines sit in registers; the sums cross lanes through DPP.
// WPT: a wave owns a token (the setup, gains, angles and page, is paid once per token, not by
// four waves) and walks all its heads; else the four waves of a workgroup share a token's
// heads, which gives short launches four times the waves.
template <int LPH, bool WPT>
__global__ void __launch_bounds__(256)
qk_norm_rope_wide_kernel(const bf16* __restrict__ qkv, bf16* __restrict__ q_out, bf16* __restrict__ k_out,
                         bf16* __restrict__ v_out, bf16* __restrict__ k_pool, bf16* __restrict__ v_pool,
                         const int* __restrict__ block_table, int table_width,
                         const int* __restrict__ token_rows, const int* __restrict__ positions,
                         const float* __restrict__ q_gain, const float* __restrict__ k_gain,
                         const float* __restrict__ inv_freq, int Hq, int Hkv, int BS, float eps,
                         int n_tokens, int groups) {
    constexpr int D = LPH * 8, HPW = SOC_WAVE / LPH, half = D / 2;
    __shared__ float cos_t[WPT ? 4 : 1][half], sin_t[WPT ? 4 : 1][half];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / SOC_WAVE), lane = threadIdx.x % SOC_WAVE;
    // a wave past the end redoes the last token and stores nothing
    const bool live = !WPT || (int)blockIdx.x * 4 + wave < n_tokens;
    const int n = !WPT ? (int)blockIdx.x : (live ? (int)blockIdx.x * 4 + wave : n_tokens - 1);
    const int heads = Hq + 2 * Hkv;
    const int sub = lane / LPH, e0 = (lane % LPH) * 8;
    const int tw = WPT ? wave : 0;                          // whose angles
    auto head_of = [&](int it) { return WPT ? it * HPW + sub : (it * 4 + wave) * HPW + sub; };
    auto load_head = [&](int it) {                         // unconditional: a head outside reads the last one
        return *reinterpret_cast<const uint4*>(qkv + ((size_t)n * heads + min(head_of(it), heads - 1)) * D + e0);
    };
    // Heads go in rounds of RD: all loads of a round are issued before the first is used, and
    // the next round's before this round's work, so a wave of 12 groups of heads pays for two
    // trips to memory, not for six.
    constexpr int RD = 6;
    uint4 cur[RD], nxt[RD];
    auto load_round = [&](uint4 (&r)[RD], int it0) {
#pragma unroll
        for (int j = 0; j < RD; ++j) r[j] = load_head(min(it0 + j, groups - 1));
    };
    load_round(cur, 0);
    const int pos = positions ? positions[n] : 0;
    float gq[8], gk[8], cs[8], sn[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { gq[i] = q_gain ? q_gain[e0 + i] : 1.f; gk[i] = k_gain ? k_gain[e0 + i] : 1.f; }
    if (inv_freq) {
        const int fi = WPT ? lane : (int)threadIdx.x;
        if (fi < half) sincosf((float)pos * inv_freq[fi], &sin_t[tw][fi], &cos_t[tw][fi]);
        __syncthreads();
        const int j0 = e0 < half ? e0 : e0 - half;
#pragma unroll
        for (int i = 0; i < 8; ++i) { cs[i] = cos_t[tw][j0 + i]; sn[i] = sin_t[tw][j0 + i]; }
    }
    size_t page_base = 0;
    if (k_pool) {
        const int page = block_table[(size_t)token_rows[n] * table_width + pos / BS];
        page_base = ((size_t)page * Hkv * BS + (size_t)(pos % BS)) * D;
    }
    auto work = [&](const uint4& raw, int it) {
        const int h = head_of(it);
        const bool is_q = h < Hq, is_k = !is_q && h < Hq + Hkv;
        float v[8];
        {
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
        }
        if ((is_q && q_gain) || (is_k && k_gain)) {         // the same for all lanes of a head
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
            ss += soc_dpp<SOC_DPP_XOR1>(ss);
            ss += soc_dpp<SOC_DPP_XOR2>(ss);
            ss += soc_dpp<SOC_DPP_HALF_MIRROR>(ss);
            if constexpr (LPH == 16) ss += soc_dpp<SOC_DPP_ROW_MIRROR>(ss);
            const float inv = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = v[i] * inv * (is_q ? gq[i] : gk[i]);
        }
        if (inv_freq) {
            // the partner of element e is e +- D / 2: the same slot of the lane LPH / 2 away in the head
            float partner[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                if constexpr (LPH == 16) partner[i] = soc_dpp<0x128>(v[i]);          // rotate the row of 16 by 8
                else partner[i] = __shfl_xor(v[i], LPH / 2, SOC_WAVE);
            }
            if (is_q || is_k) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    v[i] = e0 < half ? v[i] * cs[i] - partner[i] * sn[i] : v[i] * cs[i] + partner[i] * sn[i];
            }
        }
        if (h < heads && live) {
            bf16* dst;
            if (is_q) dst = q_out + ((size_t)n * Hq + h) * D;
            else {
                const int kvh = is_k ? h - Hq : h - Hq - Hkv;
                if (k_pool) dst = (is_k ? k_pool : v_pool) + page_base + (size_t)kvh * BS * D;
                else dst = (is_k ? k_out : v_out) + ((size_t)n * Hkv + kvh) * D;
            }
            *reinterpret_cast<uint4*>(dst + e0) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                             pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
        }
    };
    for (int it0 = 0; it0 < groups; it0 += RD) {
        const bool more = it0 + RD < groups;                // the same for the whole wave
        if (more) load_round(nxt, it0 + RD);
#pragma unroll
        for (int j = 0; j < RD; ++j)
            if (it0 + j < groups) work(cur[j], it0 + j);
        if (more) {
#pragma unroll
            for (int j = 0; j < RD; ++j) cur[j] = nxt[j];
        }
    }
}

template <typename T>
static void launch_qk_norm_rope(const void* qkv, void* q_out, void* k_out, void* v_out, void* k_pool,
                                void* v_pool, const int* block_table, int table_width,
                                const int* token_rows, const int* positions, const float* q_gain,
                                const float* k_gain, const float* inv_freq, int N, int Hq, int Hkv, int D,
                                int rotary_dim, int BS, float eps, hipStream_t stream) {
    const int heads = Hq + 2 * Hkv;
    if constexpr (sizeof(T) == 2) {
        // many tokens, a head size and a rotation the wide kernel takes: several heads per wave
        if (N >= 256 && (D == 64 || D == 128) && (!inv_freq || rotary_dim == D)) {
            const int hpw_wide = D == 128 ? 4 : 8;
            const int groups = (heads + hpw_wide - 1) / hpw_wide;
            // from 1,024 tokens on a wave per token (measured at 48 heads of 128: 2,048 tokens
            // 17 us against 23 us, 512 tokens 11 us against 9 us)
            const bool wpt = N >= 1024;
            const dim3 grid_wide(wpt ? (N + 3) / 4 : N, 1);
            const int its = wpt ? groups : (groups + 3) / 4;
#define SOC_QKW_ARGS (const bf16*)qkv, (bf16*)q_out, (bf16*)k_out, (bf16*)v_out, (bf16*)k_pool, (bf16*)v_pool, \
        block_table, table_width, token_rows, positions, q_gain, k_gain, inv_freq, Hq, Hkv, BS, eps, N, its
            if (D == 128 && wpt) hipLaunchKernelGGL((qk_norm_rope_wide_kernel<16, true>), grid_wide, dim3(256), 0, stream, SOC_QKW_ARGS);
            else if (D == 128) hipLaunchKernelGGL((qk_norm_rope_wide_kernel<16, false>), grid_wide, dim3(256), 0, stream, SOC_QKW_ARGS);
            else if (wpt) hipLaunchKernelGGL((qk_norm_rope_wide_kernel<8, true>), grid_wide, dim3(256), 0, stream, SOC_QKW_ARGS);
            else hipLaunchKernelGGL((qk_norm_rope_wide_kernel<8, false>), grid_wide, dim3(256), 0, stream, SOC_QKW_ARGS);
#undef SOC_QKW_ARGS
            return;
        }
    }
    // few tokens: one head per wave; many tokens: a workgroup walks all heads of its token
    const int hpw = N >= 256 ? (heads + 3) / 4 : 1;
    const dim3 grid(N, (heads + 4 * hpw - 1) / (4 * hpw));
#define SOC_QK_ARGS (const T*)qkv, (T*)q_out, (T*)k_out, (T*)v_out, (T*)k_pool, (T*)v_pool, block_table, \
        table_width, token_rows, positions, q_gain, k_gain, inv_freq, Hq, Hkv, D, rotary_dim, BS, eps, hpw
    if (D <= 64) hipLaunchKernelGGL((qk_norm_rope_kernel<T, 1>), grid, dim3(256), 0, stream, SOC_QK_ARGS);
    else if (D <= 128) hipLaunchKernelGGL((qk_norm_rope_kernel<T, 2>), grid, dim3(256), 0, stream, SOC_QK_ARGS);
    else hipLaunchKernelGGL((qk_norm_rope_kernel<T, 4>), grid, dim3(256), 0, stream, SOC_QK_ARGS);
#undef SOC_QK_ARGS
}

SOC_EXPORT int soc_qk_norm_rope(const void* qkv, void* q_out, void* k_out, void* v_out, void* k_pool,
                                void* v_pool, const int* block_table, int table_width,
                                const int* token_rows, const int* positions, const float* q_gain,
                                const float* k_gain, const float* inv_freq, int N, int Hq, int Hkv,
                                int D, int rotary_dim, int BS, float eps, int dtype,
                                hipStream_t stream) {
    if (N <= 0) return 0;
    if (D > SOC_MAX_HEAD || D < 1 || D % 4) return (int)hipErrorInvalidValue;
    if ((Hq + 2 * Hkv + 3) / 4 > 65535) return (int)hipErrorInvalidValue;
    // a lane owns 1, 2 or 4 consecutive elements (head size up to 64, 128, 256); half the
    // rotary width must be a whole number of lanes
    const int ve = D <= 64 ? 1 : (D <= 128 ? 2 : 4);
    if (inv_freq && (rotary_dim % (2 * ve) || rotary_dim > D)) return (int)hipErrorInvalidValue;
    if (dtype == 0)
        launch_qk_norm_rope<float>(qkv, q_out, k_out, v_out, k_pool, v_pool, block_table, table_width,
                                   token_rows, positions, q_gain, k_gain, inv_freq, N, Hq, Hkv, D,
                                   rotary_dim, BS, eps, stream);
    else
        launch_qk_norm_rope<bf16>(qkv, q_out, k_out, v_out, k_pool, v_pool, block_table, table_width,
                                  token_rows, positions, q_gain, k_gain, inv_freq, N, Hq, Hkv, D,
                                  rotary_dim, BS, eps, stream);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Rotation alone, in place on x [N, H, D].
template <typename T>
__global__ void rope_kernel(T* __restrict__ x, const int* __restrict__ positions,
                            const float* __restrict__ inv_freq, int H, int D, int rotary_dim) {
    const int n = blockIdx.x;
    const int half = rotary_dim / 2;
    const int pos = positions[n];
    T* row = x + (size_t)n * H * D;
    for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
        const int h = i / half, j = i % half;
        T* p = row + (size_t)h * D;
        const float a = to_float(p[j]), b = to_float(p[j + half]);
        float s, c;
        sincosf((float)pos * inv_freq[j], &s, &c);
        p[j] = from_float<T>(a * c - b * s);
        p[j + half] = from_float<T>(b * c + a * s);
    }
}

SOC_EXPORT int soc_rope(void* x, const int* positions, const float* inv_freq, int N, int H, int D,
                        int rotary_dim, int dtype, hipStream_t stream) {
    if (N <= 0 || H <= 0) return 0;
    if (dtype == 0)
        hipLaunchKernelGGL(rope_kernel<float>, dim3(N), dim3(256), 0, stream, (float*)x, positions,
                           inv_freq, H, D, rotary_dim);
    else
        hipLaunchKernelGGL(rope_kernel<bf16>, dim3(N), dim3(256), 0, stream, (bf16*)x, positions,
                           inv_freq, H, D, rotary_dim);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Store k, v [N, Hkv, D] into the pages of each token's row at its position.
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                T* __restrict__ k_pool, T* __restrict__ v_pool,
                                const int* __restrict__ block_table, int table_width,
                                const int* __restrict__ token_rows,
                                const int* __restrict__ positions, int Hkv, int D, int BS) {
    const int n = blockIdx.x;
    const int pos = positions[n];
    const int page = block_table[(size_t)token_rows[n] * table_width + pos / BS];
    const size_t base = ((size_t)page * Hkv * BS + (size_t)(pos % BS)) * D;
    for (int i = threadIdx.x; i < Hkv * D; i += blockDim.x) {
        const int h = i / D, e = i % D;
        const size_t dst = base + (size_t)h * BS * D + e;
        k_pool[dst] = k[(size_t)n * Hkv * D + i];
        v_pool[dst] = v[(size_t)n * Hkv * D + i];
    }
}

SOC_EXPORT int soc_kv_write(const void* k, const void* v, void* k_pool, void* v_pool,
                            const int* block_table, int table_width, const int* token_rows,
                            const int* positions, int N, int Hkv, int D, int BS, int dtype,
                            hipStream_t stream) {
    if (N <= 0 || Hkv <= 0) return 0;
    if (dtype == 0)
        hipLaunchKernelGGL(kv_write_kernel<float>, dim3(N), dim3(256), 0, stream, (const float*)k,
                           (const float*)v, (float*)k_pool, (float*)v_pool, block_table, table_width,
                           token_rows, positions, Hkv, D, BS);
    else
        hipLaunchKernelGGL(kv_write_kernel<bf16>, dim3(N), dim3(256), 0, stream, (const bf16*)k,
                           (const bf16*)v, (bf16*)k_pool, (bf16*)v_pool, block_table, table_width,
                           token_rows, positions, Hkv, D, BS);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// The rotation's cosines and sines by position, with the arithmetic of the kernels above
// (float32 angle position * inv_freq, sincosf): out [n_pos][2][half], cosines then sines.
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, int half, int first_pos, int n_pos,
                                  float* __restrict__ out) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n_pos * half) return;
    const int p = (int)(i / half), j = (int)(i % half);
    float sn, cs;
    sincosf((float)(first_pos + p) * inv_freq[j], &sn, &cs);
    out[((size_t)p * 2) * half + j] = cs;
    out[((size_t)p * 2 + 1) * half + j] = sn;
}

SOC_EXPORT int soc_rope_table(const float* inv_freq, int half, int first_pos, int n_pos, float* out,
                              hipStream_t stream) {
    if (n_pos <= 0) return 0;
    if (half < 1 || first_pos < 0) return (int)hipErrorInvalidValue;
    const size_t total = (size_t)n_pos * half;
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, inv_freq,
                       half, first_pos, n_pos, out);
    return soc_last_error();
}
