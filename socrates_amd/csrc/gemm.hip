// Matrix products C[M, N] = A[M, K] * W[N, K]^T (both operands K-contiguous, the layout of
// activations and of nn.Linear weights; model/qwen/qwen_kv_paged.py:140-143, 224).
//
//  gemm_generic_kernel   any sizes and any mix of float32 / bfloat16 operands; plain FMA in
//                        float32, K summed in order. This is the true 32-bit path.
//  gemm_bf16_mfma_kernel bfloat16 operands, 128x128x64 tiles through LDS, 16x16x32 MFMA with
//                        float32 accumulators. The library's product is faster for many rows
//                        and is what the engine uses there; this kernel stays as the
//                        package's own path (HipKernels.library_gemm = False).
//  gemm_bf16_skinny_kernel bfloat16, M <= 64 (the engine uses it up to 16 rows: decode). Bound
//                        by streaming W once from HBM: 16-byte slices of 16 weight rows per
//                        wave load, two buffers in flight, weights as the MFMA's first
//                        operand so that one lane ends up with four consecutive outputs,
//                        optional split of K over workgroups (float32 partial sums) and an
//                        optional SwiGLU epilogue.
//  gemm_bf16_sweep_kernel the same product for at most 16 rows with one workgroup per compute
//                        unit that keeps its slices of x in registers and walks over the
//                        weight tiles (K up to 5,120).
//  gemm_bf16_sweep_parts_kernel 17 to 64 rows: K split over such workgroups, float32 partial
//                        sums for a consumer that adds them.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// ---------------------------------------------------------------------------------------------
constexpr int GT = 64, GK = 16;

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M,
                    int N, int K) {
    __shared__ float As[GK][GT + 1];
    __shared__ float Ws[GK][GT + 1];
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int am = m0 + lrow, wn = n0 + lrow;
            As[lk + j][lrow] = (am < M && k < K) ? to_float(A[(size_t)am * K + k]) : 0.f;
            Ws[lk + j][lrow] = (wn < N && k < K) ? to_float(W[(size_t)wn * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[k][ty + 16 * i]; b[i] = Ws[k][tx + 16 * i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty + 16 * i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n < N) C[(size_t)m * N + n] = from_float<TC>(acc[i][j]);
        }
    }
}

template <typename TA, typename TW, typename TC>
static int launch_generic(const void* A, const void* W, void* C, int M, int N, int K, hipStream_t s) {
    dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
    hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TC>), grid, dim3(256), 0, s, (const TA*)A,
                       (const TW*)W, (TC*)C, M, N, K);
    return soc_last_error();
}

// dtypes: 0 float32, 1 bfloat16
SOC_EXPORT int soc_gemm_generic(const void* A, const void* W, void* C, int M, int N, int K, int a_dtype,
                                int w_dtype, int c_dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if ((M + GT - 1) / GT > 65535) return (int)hipErrorInvalidValue;
    const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
    switch (key) {
        case 0: return launch_generic<float, float, float>(A, W, C, M, N, K, stream);
        case 1: return launch_generic<float, float, bf16>(A, W, C, M, N, K, stream);
        case 2: return launch_generic<float, bf16, float>(A, W, C, M, N, K, stream);
        case 3: return launch_generic<float, bf16, bf16>(A, W, C, M, N, K, stream);
        case 4: return launch_generic<bf16, float, float>(A, W, C, M, N, K, stream);
        case 5: return launch_generic<bf16, float, bf16>(A, W, C, M, N, K, stream);
        case 6: return launch_generic<bf16, bf16, float>(A, W, C, M, N, K, stream);
        case 7: return launch_generic<bf16, bf16, bf16>(A, W, C, M, N, K, stream);
    }
    return (int)hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64, LDS_STRIDE = BK + 8;   // bf16 elements per LDS row

__device__ __forceinline__ uint4 load_chunk(const bf16* base, int row, int rows, int k, int K) {
    if (row < rows && k < K) return *reinterpret_cast<const uint4*>(base + (size_t)row * K + k);
    return make_uint4(0u, 0u, 0u, 0u);
}

template <typename TC>
__global__ void __launch_bounds__(256)
gemm_bf16_mfma_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, TC* __restrict__ C,
                      int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t Ws[BN * LDS_STRIDE];
    const int tid = threadIdx.x, wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int li = lane % 16, lk = (lane / 16) * 8;

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // 128 rows x 8 chunks of 16 bytes per operand tile; 4 chunks per thread and operand
    uint4 ra[4], rw[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + 256 * i, row = c / 8, kc = (c % 8) * 8;
            ra[i] = load_chunk(A, m0 + row, M, k0 + kc, K);
            rw[i] = load_chunk(W, n0 + row, N, k0 + kc, K);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + 256 * i, row = c / 8, kc = (c % 8) * 8;
            *reinterpret_cast<uint4*>(&As[row * LDS_STRIDE + kc]) = ra[i];
            *reinterpret_cast<uint4*>(&Ws[row * LDS_STRIDE + kc]) = rw[i];
        }
    };

    fetch(0);
    stash();
    __syncthreads();
    for (int k0 = 0; k0 < K; k0 += BK) {
        const bool more = k0 + BK < K;
        if (more) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK; ks += 32) {
            bf16x8 af[4], wf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *reinterpret_cast<const bf16x8*>(&As[(wm * 64 + i * 16 + li) * LDS_STRIDE + ks + lk]);
                wf[i] = *reinterpret_cast<const bf16x8*>(&Ws[(wn * 64 + i * 16 + li) * LDS_STRIDE + ks + lk]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
        if (more) { stash(); __syncthreads(); }
    }
    // acc[i][j][r] is C[row = 4 * (lane / 16) + r of tile i][col = lane % 16 of tile j]
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = m0 + wm * 64 + i * 16 + (lane / 16) * 4 + r;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn * 64 + j * 16 + li;
                if (n < N) C[(size_t)m * N + n] = from_float<TC>(acc[i][j][r]);
            }
        }
}

SOC_EXPORT int soc_gemm_bf16_mfma(const void* A, const void* W, void* C, int M, int N, int K,
                                  int c_dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K % 8 || K < 8) return (int)hipErrorInvalidValue;       // rows must start on 16 bytes
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    if (c_dtype == 0)
        hipLaunchKernelGGL(gemm_bf16_mfma_kernel<float>, grid, dim3(256), 0, stream, (const bf16*)A,
                           (const bf16*)W, (float*)C, M, N, K);
    else
        hipLaunchKernelGGL(gemm_bf16_mfma_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)A,
                           (const bf16*)W, (bf16*)C, M, N, K);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// (A zero operand below is always written as a prvalue: `cond ? *p : zero` with a named
// `zero` is an lvalue conditional, which selects between a global and a stack address and
// then loads through a generic pointer.)
// Skinny GEMM (M <= 64). A workgroup owns RW tiles of 16 rows of W and one of `k_splits`
// ranges of K; its waves split that range. For every 32 k a lane loads one 16-byte slice of
// each of its RW weight rows and one slice of X per 16 rows of M: a slice of X is used RW
// times, which keeps the re-reading of X (it comes from L2 for every workgroup) well below
// the weight traffic. Two buffers of SK_UNROLL slices keep the loads of the next 128 k in
// flight while the MFMAs of the current ones run. With k_splits > 1 the workgroups of one
// row tile write float32 partial sums [k_splits, M, N] that the consumer adds in order (the
// residual-add + norm kernel does).
constexpr int SK_UNROLL = 4;            // 16-byte slices per lane, row and buffer (4 x 32 = 128 k)
constexpr int SK_STEP = 32 * SK_UNROLL;
constexpr int SK_MAX_WAVES = 8;
constexpr int SK_MAX_WAVES_SWIGLU = 16;     // gate waves and up waves

template <int MT, int RW> struct SkBuf { uint4 w[RW][SK_UNROLL]; uint4 x[MT][SK_UNROLL]; };

// SWIGLU (RW = 1): the weight's rows are interleaved in blocks of 16, 16 gate rows and then
// the 16 up rows of the same output columns. The first half of a workgroup's waves takes the
// gate tile and the second half the up tile, each half splitting K; the epilogue writes
// silu(gate) * up, [M, N / 2], instead of both products. (One tile per wave streams the
// weights faster than two.)
//
// Two more forms (one tile of 16 rows of x, one weight tile per workgroup, no split of K over
// workgroups) take the residual sum and the RMSNorm out of a kernel of their own, for steps
// of at most 16 tokens, where such a kernel costs as much as a small product:
//  ADDNORM  the product is a branch's last projection. The epilogue adds it to the float32
//           residual stream in place (a workgroup owns its 16 columns of every row), stores
//           x' = bf16(h * gain) for the norm that follows, h being the new residual, and
//           the sum of h^2 over its 16 columns per row: ssq [M, tiles rounded up to 4].
//  SCALED   x is such an x' with its ssq. The norm's factor 1 / sqrt(mean(h^2) + eps) is the
//           same for a whole row, so it is applied to the sums after the product instead of
//           to x before it: out = (W x') / sqrt(sum_t ssq[m, t] / dim + eps). Statistics and
//           factor stay float32; x' is rounded once, as the norm's output would be.
struct SkNorm {
    const float* ssq_in;        // SCALED: [M, ssq_tiles rounded up to a multiple of 4]
    int ssq_tiles;
    float inv_dim, eps;
    float* residual;            // ADDNORM: [M, N] float32, updated in place
    const float* gain;          // ADDNORM: [N], the following norm's weight
    bf16* x_out;                // ADDNORM: [M, N]
    float* ssq_out;             // ADDNORM: [M, gridDim.x rounded up to a multiple of 4]
    float* split_sums;          // ADDNORM with K split over workgroups: [tiles, splits, 256], scratch
    int* split_count;           // the same: [tiles], zero before the launch and after it
};
constexpr int SK_SWIGLU = 1, SK_SCALED = 2, SK_ADDNORM = 4;
constexpr int SK_W_TILED = 1, SK_X_TILED = 2, SK_C_TILED = 4;     // the `layout` argument of the entry points
constexpr int SK_SSQ_MAX_PAIRS = 16 * 16;       // 16 rows x 16 segments of 256 tiles: norms over up to 65,536 elements

// SCALED: the factor of each of the 16 rows, from the partial sums of squares ssq [M, stride]
// (stride: the tiles rounded up to a multiple of 4, so that rows start on 16 bytes). A wave
// takes (row, segment of 256 tiles) pairs wave, wave + n_waves, ...; a lane loads four
// consecutive tiles of its pair, so a row of up to 256 tiles is one load of one wave. The
// first SK_SSQ_AHEAD pairs of a wave are asked for before the weights (no branch: a pair
// outside the matrix loads the first element in all lanes, which costs one request, and is
// left out of the sum), so that their way from memory is not waited for at the end.
constexpr int SK_SSQ_AHEAD = 4;

__device__ __forceinline__ int sk_ssq_stride(int tiles) { return (tiles + 3) & ~3; }

__device__ __forceinline__ float4 sk_ssq_load(const SkNorm& nm, int M, int pair, int lane) {
    const int row = pair % 16, t = (pair / 16) * 256 + lane * 4;
    const float* p = (row < M && t < nm.ssq_tiles) ? nm.ssq_in + (size_t)row * sk_ssq_stride(nm.ssq_tiles) + t
                                                   : nm.ssq_in;
    return *reinterpret_cast<const float4*>(p);
}

__device__ __forceinline__ float sk_ssq_masked(const SkNorm& nm, int M, int pair, int lane, float4 v) {
    const int row = pair % 16, t = (pair / 16) * 256 + lane * 4, T = nm.ssq_tiles;
    float s = 0.f;
    if (row < M) {                                     // in this order for every shape
        s += t < T ? v.x : 0.f;
        s += t + 1 < T ? v.y : 0.f;
        s += t + 2 < T ? v.z : 0.f;
        s += t + 3 < T ? v.w : 0.f;
    }
    return s;
}

__device__ __forceinline__ void sk_ssq_ahead(const SkNorm& nm, int M, int wave, int lane, float4 (&v)[SK_SSQ_AHEAD]) {
    const int n_waves = blockDim.x / SOC_WAVE;
#pragma unroll
    for (int u = 0; u < SK_SSQ_AHEAD; ++u) v[u] = sk_ssq_load(nm, M, wave + u * n_waves, lane);
}

// Before the workgroup's barrier: the sum of each of this wave's pairs into LDS, part[pair].
__device__ __forceinline__ void sk_ssq_shares(const SkNorm& nm, int M, int wave, int lane,
                                              const float4 (&v)[SK_SSQ_AHEAD], float* part) {
    const int n_waves = blockDim.x / SOC_WAVE;
    const int pairs = 16 * ((nm.ssq_tiles + 255) / 256);
#pragma unroll
    for (int u = 0; u < SK_SSQ_AHEAD; ++u) {
        const int pair = wave + u * n_waves;                 // the same in all lanes
        if (pair >= pairs || pair >= SK_SSQ_MAX_PAIRS) continue;
        // (a row beyond M has no sum to take: nothing reads its place)
        const float s = pair % 16 < M ? wave_sum(sk_ssq_masked(nm, M, pair, lane, v[u])) : 0.f;
        if (lane == 0) part[pair] = s;
    }
    for (int pair = wave + SK_SSQ_AHEAD * n_waves; pair < pairs && pair < SK_SSQ_MAX_PAIRS; pair += n_waves) {
        const float s = wave_sum(sk_ssq_masked(nm, M, pair, lane, sk_ssq_load(nm, M, pair, lane)));
        if (lane == 0) part[pair] = s;
    }
}

// After the barrier: the factor of row m, the same bits in every thread that asks.
__device__ __forceinline__ float sk_row_factor(const SkNorm& nm, const float* part, int m) {
    float total = 0.f;
    for (int seg = 0; seg * 256 < nm.ssq_tiles; ++seg) total += part[seg * 16 + m];
    return 1.0f / sqrtf(total * nm.inv_dim + nm.eps);
}

// waves of a workgroup: the forms with one tile of each operand may take 16 (their sums in
// LDS stay small)
__host__ __device__ constexpr int sk_max_waves(int MT, int RW, int MODE) {
    return MT * RW == 1 ? SK_MAX_WAVES_SWIGLU : SK_MAX_WAVES;
}

template <typename TC, int MT, int RW, int MODE = 0>
__global__ void __launch_bounds__(64 * sk_max_waves(MT, RW, MODE))
gemm_bf16_skinny_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, TC* __restrict__ C,
                        float* __restrict__ Cpart, int M, int N, int K, int k_per_split,
                        int k_per_wave, SkNorm nm, int layout = 0, int tile_h = 16) {
    constexpr bool SWIGLU = MODE & SK_SWIGLU, SCALED = MODE & SK_SCALED, ADDNORM = MODE & SK_ADDNORM;
    static_assert(!(SCALED || ADDNORM) || (MT == 1 && RW == 1), "the norm forms take one tile of each");
    __shared__ float red[sk_max_waves(MT, RW, MODE) * MT * RW * 256];
    __shared__ float norm_part[SCALED ? SK_SSQ_MAX_PAIRS : 1];      // [segment][16] sums of squares of the rows of x
    __shared__ float sq_part[ADDNORM ? 16 * 16 : 1];        // [16][16] squares of the new residual
    __shared__ bool split_last;
    // the wave index is the same in all lanes: say so, and the K loop runs on scalar registers
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / SOC_WAVE), lane = tid % SOC_WAVE;
    const int n_waves = blockDim.x / SOC_WAVE;
    const int k_waves = SWIGLU ? n_waves / 2 : n_waves;        // waves that share one tile's K
    // tile_h (the ADDNORM form; 16 elsewhere): weight rows of a workgroup, at most 16. Fewer
    // than 16 spread a narrow output over more workgroups (2,560 outputs are 160 tiles of 16,
    // which leave 96 of 256 compute units idle, and 256 tiles of 10); the rows from tile_h on
    // of the 16 that a product takes are not there.
    const int n0 = SWIGLU ? blockIdx.x * 32 + (wave / k_waves) * 16 : ADDNORM ? blockIdx.x * tile_h : blockIdx.x * 16 * RW;
    const int li = lane % 16, lk = (lane / 16) * 8;
    const int split_begin = blockIdx.y * k_per_split;
    const int split_end = min(K, split_begin + k_per_split);
    const int k_begin = split_begin + (wave % k_waves) * k_per_wave;
    const int k_end = min(split_end, k_begin + k_per_wave);
    // The weights lie row by row, [N, K], or by tile (w_tiled: [N / 16, K / 32, 16, 32], N a
    // multiple of 16 and K of 32): a wave's load of 16 rows x 32 k is then 1 KB in one piece
    // instead of sixteen pieces of 64 bytes. Either way a tile of 16 rows starts at 16 K t.
    // x (at most 16 rows, the norm forms) and the SwiGLU form's output may lie by tile too,
    // [K / 32, 16, 32] with the rows from M on never written or read: what such a product
    // hands to the next one is then read in pieces of M x 64 bytes instead of M pieces.
    const bool w_tiled = layout & SK_W_TILED, x_tiled = layout & SK_X_TILED, c_tiled = layout & SK_C_TILED;
    const int w_rs = w_tiled ? 32 : K;              // elements from a row of a tile to the next
    const int w_ss = w_tiled ? 32 * tile_h : 32;    // elements from a step of 32 k to the next
    const int x_rs = x_tiled ? 32 : K, x_ss = x_tiled ? 512 : 32;
    // Element offsets of this lane's rows (offsets, not pointers: the loads stay global
    // loads); a row outside the matrix is never loaded.
    size_t w_off[RW];
    bool w_ok[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        w_ok[r] = n0 + r * 16 + li < N && li < tile_h;
        w_off[r] = w_ok[r] ? (size_t)(n0 + r * 16) * K + (size_t)li * w_rs + lk : (size_t)n0 * K + lk;
    }
    // X is read through a buffer descriptor that covers its M rows: a lane whose row lies
    // outside (M = 8 leaves half of the 16 lanes of a tile without one) gets zeros and asks
    // memory for nothing. X comes from L2 for every workgroup, so this halves that traffic.
    const int x_bytes = x_tiled ? K * 32 : M * K * 2;
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(X), (short)0, x_bytes, 0x00020000);
    uint32_t x_off[MT];                                  // bytes; by tile a row from M on starts where the buffer ends
#pragma unroll
    for (int t = 0; t < MT; ++t)
        x_off[t] = x_tiled && t * 16 + li >= M ? (uint32_t)x_bytes : (uint32_t)(((t * 16 + li) * x_rs + lk) * 2);
    f32x4 acc[MT][RW];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < RW; ++r) acc[t][r] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // ADDNORM: the element of the residual and the gain that this thread's output meets, asked
    // for ahead of the weights (every thread loads, from a clamped place: no branch here)
    float4 ssq_v[SK_SSQ_AHEAD];
    if constexpr (SCALED) sk_ssq_ahead(nm, M, wave, lane, ssq_v);
    float old_h = 0.f, out_gain = 0.f;
    if constexpr (ADDNORM) {
        const int ln = (tid % 256) / 4, e = tid % 4;
        const int m = min(ln % 16, M - 1), n = min(n0 + min(4 * (ln / 16) + e, tile_h - 1), N - 1);
        old_h = nm.residual[(size_t)m * N + n];
        out_gain = nm.gain[n];
    }

    // Full steps of 128 k load without any predicate (a weight row outside the matrix reads
    // row 0 and its results are dropped at the store; X rows outside read zeros through the
    // descriptor), so the loop body is straight-line code and the loads of the next step stay
    // in flight under the MFMAs of the current one.
#define SK_LOAD(B, K0)                                                                              \
    _Pragma("unroll") for (int u = 0; u < SK_UNROLL; ++u) {                                          \
        _Pragma("unroll") for (int r = 0; r < RW; ++r)                                               \
            B.w[r][u] = *reinterpret_cast<const uint4*>(W + w_off[r] + (size_t)((K0) / 32 + u) * w_ss); \
        _Pragma("unroll") for (int t = 0; t < MT; ++t)                                               \
            B.x[t][u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(              \
                x_rsrc, x_off[t] + (uint32_t)(((K0) / 32 + u) * x_ss * 2), 0, 0));                   \
    }
#define SK_COMPUTE(B)                                                                               \
    _Pragma("unroll") for (int u = 0; u < SK_UNROLL; ++u)                                            \
        _Pragma("unroll") for (int t = 0; t < MT; ++t)                                               \
            _Pragma("unroll") for (int r = 0; r < RW; ++r)                                           \
                acc[t][r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(                                 \
                    __builtin_bit_cast(bf16x8, B.w[r][u]), __builtin_bit_cast(bf16x8, B.x[t][u]),    \
                    acc[t][r], 0, 0, 0);

    SkBuf<MT, RW> b0, b1;
    const int steps = max(k_end - k_begin, 0) / SK_STEP;
    const int k_full = k_begin + steps * SK_STEP;
    if (steps > 0) {
        SK_LOAD(b0, k_begin)
        int s = 1;
        // steady state: no branch between a load and the MFMAs that must not wait for it
        for (; s + 1 < steps; s += 2) {
            SK_LOAD(b1, k_begin + s * SK_STEP)
            SK_COMPUTE(b0)
            SK_LOAD(b0, k_begin + (s + 1) * SK_STEP)
            SK_COMPUTE(b1)
        }
        if (s < steps) {
            SK_LOAD(b1, k_begin + s * SK_STEP)
            SK_COMPUTE(b0)
            SK_COMPUTE(b1)
        } else {
            SK_COMPUTE(b0)
        }
    }
#undef SK_LOAD
    // The last, partial step of the range (only where K is no multiple of 128): slices past
    // the end contribute zeros.
    if (k_full < k_end) {
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int kk = k_full + 32 * u;
            const bool in = kk + lk < k_end;
#pragma unroll
            for (int r = 0; r < RW; ++r)
                b0.w[r][u] = in ? *reinterpret_cast<const uint4*>(W + w_off[r] + (size_t)(kk / 32) * w_ss + kk % 32)
                                : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
            for (int t = 0; t < MT; ++t)
                b0.x[t][u] = in ? __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                                      x_rsrc, x_off[t] + (uint32_t)(((kk / 32) * x_ss + kk % 32) * 2), 0, 0))
                                : make_uint4(0u, 0u, 0u, 0u);
        }
        SK_COMPUTE(b0)
    }
#undef SK_COMPUTE
    // acc[t][r][e] is the partial of C[m = 16 t + lane % 16][n = n0 + 16 r + 4 * (lane / 16) + e]
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                red[(((wave * MT + t) * RW + r) * 64 + lane) * 4 + e] = acc[t][r][e];
    if constexpr (SCALED) sk_ssq_shares(nm, M, wave, lane, ssq_v, norm_part);
    __syncthreads();
    if constexpr (SWIGLU) {
        static_assert(!SWIGLU || (RW == 1 && MT == 1), "one tile per wave, gate waves then up waves");
        for (int idx = tid; idx < 256; idx += blockDim.x) {
            const int ln = idx / 4, e = idx % 4;
            float g = 0.f, u = 0.f;
            for (int w = 0; w < k_waves; ++w) {
                g += red[(w * 64 + ln) * 4 + e];
                u += red[((k_waves + w) * 64 + ln) * 4 + e];
            }
            const int m = ln % 16, col = blockIdx.x * 16 + 4 * (ln / 16) + e;
            if constexpr (SCALED) { const float f = sk_row_factor(nm, norm_part, m); g *= f; u *= f; }
            if (m < M && 2 * col < N)
                C[c_tiled ? ((size_t)(col / 32) * 16 + m) * 32 + col % 32 : (size_t)m * (N / 2) + col] =
                    from_float<TC>(u * (g / (1.0f + expf(-g))));
        }
        return;
    }
    if constexpr (ADDNORM) {
        // 256 outputs, one per thread of the first four waves: thread 4 * ln + e has row
        // ln % 16 and column 4 * (ln / 16) + e of the tile
        const int ln = (tid % 256) / 4, e = tid % 4;
        const int m = ln % 16, c = 4 * (ln / 16) + e, n = n0 + c;
        float sum = 0.f;
        if (tid < 256) {
            for (int w = 0; w < n_waves; ++w) sum += red[(w * 64 + ln) * 4 + e];
            if constexpr (SCALED) sum *= sk_row_factor(nm, norm_part, m);
        }
        if (gridDim.y > 1) {
            // K is split over gridDim.y workgroups per tile. Each leaves its 256 sums in memory
            // and is counted; the one counted last adds all of them, in the order of the
            // splits whoever came last, and goes on alone. No fence (a fence writes back and
            // invalidates this chip's whole L2, which costs more than the kernel): the sums
            // are written through the caches and read past them (agent-scope atomic stores and
            // loads), and a wait for the stores' acknowledgement orders them before the count.
            float* mine = nm.split_sums + ((size_t)blockIdx.x * gridDim.y + blockIdx.y) * 256;
            if (tid < 256) __hip_atomic_store(mine + tid, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (tid == 0) {
                const int before = __hip_atomic_fetch_add(nm.split_count + blockIdx.x, 1, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT);
                split_last = before == (int)gridDim.y - 1;
                // the count is left at zero for the next launch that uses it
                if (split_last) __hip_atomic_store(nm.split_count + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            if (!split_last) return;
            if (tid < 256) {
                const float* all = nm.split_sums + (size_t)blockIdx.x * gridDim.y * 256 + tid;
                sum = 0.f;
                for (int sp = 0; sp < (int)gridDim.y; ++sp)
                    sum += __hip_atomic_load(all + sp * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        if (tid < 256) {
            float h = 0.f;
            if (m < M && n < N && c < tile_h) {
                h = old_h + sum;
                nm.residual[(size_t)m * N + n] = h;
                nm.x_out[(size_t)m * N + n] = from_float<bf16>(h * out_gain);
            }
            sq_part[m * 16 + c] = h * h;
        }
        __syncthreads();
        if (tid < M) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) ss += sq_part[tid * 16 + i];
            nm.ssq_out[(size_t)tid * sk_ssq_stride(gridDim.x) + blockIdx.x] = ss;
        }
        return;
    }
    for (int idx = tid; idx < MT * RW * 256; idx += blockDim.x) {
        const int tr = idx / 256, ln = (idx % 256) / 4, e = idx % 4;
        const int t = tr / RW, r = tr % RW;
        float sum = 0.f;
        for (int w = 0; w < n_waves; ++w) sum += red[((w * MT * RW + tr) * 64 + ln) * 4 + e];
        const int m = t * 16 + ln % 16, n = n0 + r * 16 + 4 * (ln / 16) + e;
        if constexpr (SCALED) sum *= sk_row_factor(nm, norm_part, m % 16);
        if (m < M && n < N) {
            if (Cpart) Cpart[((size_t)blockIdx.y * M + m) * N + n] = sum;
            else C[(size_t)m * N + n] = from_float<TC>(sum);
        }
    }
}

template <typename TC, int MT, int RW>
static int launch_skinny(const void* X, const void* W, void* C, float* Cpart, int M, int N, int K,
                         int n_waves, int k_splits, int layout, hipStream_t stream) {
    // ranges are multiples of the 128-k step, so only the end of K can be a partial step
    const int k_per_split = ((K + k_splits - 1) / k_splits + SK_STEP - 1) / SK_STEP * SK_STEP;
    const int k_per_wave = ((k_per_split + n_waves - 1) / n_waves + SK_STEP - 1) / SK_STEP * SK_STEP;
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TC, MT, RW>), dim3((N + 16 * RW - 1) / (16 * RW), k_splits),
                       dim3(n_waves * 64), 0, stream, (const bf16*)X, (const bf16*)W, (TC*)C, Cpart, M, N,
                       K, k_per_split, k_per_wave, SkNorm{}, layout);
    return soc_last_error();
}

// x [M <= 16, K] times w [N, K]^T with gate and up rows interleaved in blocks of 16, then
// silu(gate) * up: C [M, N / 2]. N a multiple of 32, K a multiple of 8.
// ssq_in (may be null): x is a following norm's input x' = bf16(h * gain) with the partial
// sums of squares ssq_in [M, ssq_tiles] of its rows h of `norm_dim` elements; the norm's
// factor is applied to the sums (the SCALED form above). bfloat16 output only then.
SOC_EXPORT int soc_gemm_bf16_skinny_swiglu(const void* X, const void* W, void* C, int M, int N, int K,
                                           int c_dtype, int n_waves, const float* ssq_in, int ssq_tiles,
                                           int norm_dim, float eps, int layout, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if ((layout & ~7) || ((layout & SK_W_TILED) && (N % 16 || K % 32)) || ((layout & SK_X_TILED) && K % 32) ||
        ((layout & SK_C_TILED) && (N % 64 || c_dtype != 1)))
        return (int)hipErrorInvalidValue;
    if (M > 16 || K % 8 || K < 8 || K > (1 << 23) || N % 32) return (int)hipErrorInvalidValue;
    if (n_waves < 2 || n_waves > SK_MAX_WAVES_SWIGLU || n_waves % 2) return (int)hipErrorInvalidValue;
    if (ssq_in && (ssq_tiles < 1 || ssq_tiles > 16 * SK_SSQ_MAX_PAIRS || norm_dim < 1 || c_dtype != 1))
        return (int)hipErrorInvalidValue;
    const int k_waves = n_waves / 2;
    const int k_per_wave = ((K + k_waves - 1) / k_waves + SK_STEP - 1) / SK_STEP * SK_STEP;
    const int k_per_split = k_per_wave * k_waves;
    SkNorm nm{};
    nm.ssq_in = ssq_in; nm.ssq_tiles = ssq_tiles; nm.inv_dim = 1.0f / (float)max(norm_dim, 1); nm.eps = eps;
    if (ssq_in)
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<bf16, 1, 1, SK_SWIGLU | SK_SCALED>), dim3(N / 32, 1),
                           dim3(n_waves * 64), 0, stream, (const bf16*)X, (const bf16*)W, (bf16*)C,
                           (float*)nullptr, M, N, K, k_per_split, k_per_wave, nm, layout);
    else if (c_dtype == 0)
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<float, 1, 1, SK_SWIGLU>), dim3(N / 32, 1), dim3(n_waves * 64), 0,
                           stream, (const bf16*)X, (const bf16*)W, (float*)C, (float*)nullptr, M, N, K,
                           k_per_split, k_per_wave, nm, layout);
    else
        hipLaunchKernelGGL((gemm_bf16_skinny_kernel<bf16, 1, 1, SK_SWIGLU>), dim3(N / 32, 1), dim3(n_waves * 64), 0,
                           stream, (const bf16*)X, (const bf16*)W, (bf16*)C, (float*)nullptr, M, N, K,
                           k_per_split, k_per_wave, nm, layout);
    return soc_last_error();
}

// The norm forms of the skinny product, M <= 16, one weight tile per workgroup, K not split
// over workgroups. ssq_in (may be null): x is an x' with its partial sums of squares, as
// above. residual (may be null): the product is added to residual [M, N] in place, and
// x_out [M, N] = bf16(residual * gain), ssq_out [M, ceil(N / 16)] are written for the norm of
// `N` elements that follows; C is then not written. At least one of the two is given.
// k_splits > 1 (with residual only): K is split over that many workgroups per tile, which meet
// through split_sums [tiles, k_splits, 256] floats (scratch) and split_count
// [tiles] ints, which must be zero before the call and are zero again after it. Two
// launches that may run at the same time need counts of their own.
// tile_h (with residual; 16 otherwise): weight rows of a workgroup, 1 to 16; tiles = ceil(N /
// tile_h) workgroups (times k_splits), ssq_out [M, tiles rounded up to 4]; weights by tile then
// lie [N / tile_h, K / 32, tile_h, 32] (N a multiple of tile_h).
SOC_EXPORT int soc_gemm_bf16_skinny_norm(const void* X, const void* W, void* C, int M, int N, int K,
                                         int n_waves, const float* ssq_in, int ssq_tiles, int norm_dim,
                                         float eps, float* residual, const float* gain, void* x_out,
                                         float* ssq_out, int k_splits, float* split_sums, int* split_count,
                                         int layout, int tile_h, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (tile_h < 1 || tile_h > 16 || (tile_h != 16 && !residual)) return (int)hipErrorInvalidValue;
    if ((layout & ~3) || ((layout & SK_W_TILED) && (N % tile_h || K % 32)) || ((layout & SK_X_TILED) && K % 32))
        return (int)hipErrorInvalidValue;
    if (M > 16 || K % 8 || K < 8 || K > (1 << 23)) return (int)hipErrorInvalidValue;
    if (n_waves < 1 || n_waves > SK_MAX_WAVES_SWIGLU) return (int)hipErrorInvalidValue;
    if (!ssq_in && !residual) return (int)hipErrorInvalidValue;
    if (ssq_in && (ssq_tiles < 1 || ssq_tiles > 16 * SK_SSQ_MAX_PAIRS || norm_dim < 1)) return (int)hipErrorInvalidValue;
    if (residual ? (!gain || !x_out || !ssq_out) : !C) return (int)hipErrorInvalidValue;
    if (residual) n_waves = max(n_waves, 4);            // its epilogue has one output per thread of four waves
    if (k_splits < 1 || k_splits > 64 || (k_splits > 1 && (!residual || !split_sums || !split_count)))
        return (int)hipErrorInvalidValue;
    const int k_per_wave = ((K + k_splits * n_waves - 1) / (k_splits * n_waves) + SK_STEP - 1) / SK_STEP * SK_STEP;
    const int k_per_split = k_per_wave * n_waves;
    SkNorm nm{};
    nm.split_sums = split_sums; nm.split_count = split_count;
    nm.ssq_in = ssq_in; nm.ssq_tiles = ssq_tiles; nm.inv_dim = 1.0f / (float)max(norm_dim, 1); nm.eps = eps;
    nm.residual = residual; nm.gain = gain; nm.x_out = (bf16*)x_out; nm.ssq_out = ssq_out;
    const dim3 grid((N + tile_h - 1) / tile_h, k_splits), block(n_waves * 64);
#define SOC_SKN(MODE_) \
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<bf16, 1, 1, MODE_>), grid, block, 0, stream, (const bf16*)X, \
                       (const bf16*)W, (bf16*)C, (float*)nullptr, M, N, K, k_per_split, k_per_wave, nm, layout, tile_h)
    if (ssq_in && residual) SOC_SKN(SK_SCALED | SK_ADDNORM);
    else if (residual) SOC_SKN(SK_ADDNORM);
    else SOC_SKN(SK_SCALED);
#undef SOC_SKN
    return soc_last_error();
}

// Shape heuristics shared with the host wrapper (which sizes the partial buffer): rows per
// workgroup (in tiles of 16), waves of a workgroup, and workgroups that split K, for an
// [M <= 64] x [N, K] product.
SOC_EXPORT void soc_gemm_skinny_plan(int M, int N, int K, int allow_split, int* row_tiles, int* n_waves,
                                     int* k_splits) {
    // From measurements on an MI355X at the products of 4B-, 8B- and 32B-sized layers
    // (N 2560..51200, K 2560..25600): one tile per workgroup and eight waves over K is within
    // a few per cent of the best everywhere from N = 4096 on; a long K over a middling N gains
    // from two workgroups per tile; narrow outputs need that to fill the GPU.
    int rw, nw, ks = 1;
    if (M > 16) { rw = 2; nw = N >= 16384 ? 4 : 8; }
    else if (N >= 4096) { rw = 1; nw = 8; if (allow_split && K >= 8192 && N < 16384) ks = 2; }
    else if (allow_split && K >= 2048) { rw = 2; nw = 8; ks = 2; }
    else { rw = 1; nw = 8; }
    while (nw > 1 && K / (nw * ks) < 128) nw /= 2;
    while (ks > 1 && K / (nw * ks) < 128) ks /= 2;
    *row_tiles = rw;
    *n_waves = nw;
    *k_splits = ks;
}

// M <= 64, K a multiple of 8. k_splits == 1: C [M, N] in c_dtype. k_splits > 1: float32
// partial sums Cpart [k_splits, M, N] (C is not written). layout (here and in the entry
// points around): SK_W_TILED, W lies by tile, [N / 16, K / 32, 16, 32], N a multiple of 16 and
// K of 32; SK_X_TILED, x (at most 16 rows) lies [K / 32, 16, 32], rows from M on never read;
// SK_C_TILED (SwiGLU forms, bfloat16), the output is written that way.
SOC_EXPORT int soc_gemm_bf16_skinny(const void* X, const void* W, void* C, float* Cpart, int M, int N,
                                    int K, int c_dtype, int row_tiles, int n_waves, int k_splits,
                                    int layout, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if ((layout & ~3) || ((layout & SK_W_TILED) && (N % 16 || K % 32)) || ((layout & SK_X_TILED) && (K % 32 || M > 16)))
        return (int)hipErrorInvalidValue;
    if (M > 64 || K % 8 || K < 8 || K > (1 << 23)) return (int)hipErrorInvalidValue;   // 32-bit byte offsets into X
    if (n_waves < 1 || n_waves > (M <= 16 && row_tiles == 1 ? SK_MAX_WAVES_SWIGLU : SK_MAX_WAVES) || k_splits < 1 ||
        k_splits > 65535)
        return (int)hipErrorInvalidValue;
    if ((k_splits > 1) != (Cpart != nullptr)) return (int)hipErrorInvalidValue;
    const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    if (row_tiles != 2 && !((row_tiles == 4 || row_tiles == 1) && MT == 1)) return (int)hipErrorInvalidValue;
#define SOC_SK(TC_, MT_, RW_) \
    return launch_skinny<TC_, MT_, RW_>(X, W, C, Cpart, M, N, K, n_waves, k_splits, layout, stream)
    if (c_dtype == 0) {
        if (MT == 1 && row_tiles == 4) SOC_SK(float, 1, 4);
        if (MT == 1 && row_tiles == 1) SOC_SK(float, 1, 1);
        if (MT == 1) SOC_SK(float, 1, 2);
        if (MT == 2) SOC_SK(float, 2, 2);
        SOC_SK(float, 4, 2);
    }
    if (MT == 1 && row_tiles == 4) SOC_SK(bf16, 1, 4);
    if (MT == 1 && row_tiles == 1) SOC_SK(bf16, 1, 1);
    if (MT == 1) SOC_SK(bf16, 1, 2);
    if (MT == 2) SOC_SK(bf16, 2, 2);
    SOC_SK(bf16, 4, 2);
#undef SOC_SK
}

// ---------------------------------------------------------------------------------------------
// Sweep form of the skinny product (M <= 16; plain, SCALED and SWIGLU forms, K not split over
// workgroups). In the kernel above every workgroup reads all rows of x for its 16 weight
// rows, and with some hundred workgroups per product that re-reading costs a quarter of the
// kernel's time at 8 rows and a third at 16 (a build without the loads of x runs at the
// one-row speed whatever M is). Here a product has at most one workgroup per compute unit,
// of 16 waves that split K as before; a wave keeps its slices of x in registers for the
// whole kernel (at most 8 steps of 32 k, or two halves of 5: K up to 5,120), and the workgroup sweeps over
// weight tiles g, g + G, g + 2 G, ...: per tile a wave loads only weights, multiplies, and
// leaves its sums in LDS, where the first four waves add them and do the epilogue while the
// others go on. The weights of two tiles are on their way at any time, and x is read once per
// workgroup. With the weights row by row, the form of a workgroup per tile streams them 8 %
// faster at one row and this one wins from 3 rows on (gate+up of a 4B-sized layer at 8 rows:
// 23.3 against 27.0 us, at 16 rows 24.8 against 33.8 us; the output head of 151,936 rows at 8
// rows: 141 against 169 us); with the weights by tile it wins at every number of rows
// (gate+up 19.7 us at 8 rows).
// SWIGLU: an item is a pair of tiles (gate rows, then up rows of the same 16 outputs), swept
// one after the other; the gate sums wait in registers for the up sums.
// (The form with a residual epilogue stays with the kernel above: its few tiles with a long K
// need K split over workgroups, and workgroups that sweep and meet in memory were measured
// at twice its time.)
constexpr uint32_t SW_NOWHERE = 0xfffffff0u;        // an offset past the end of every buffer: reads as zeros, asks memory for nothing

struct SwPlan {
    int k_per_wave;                 // a multiple of 32
    int items;                      // weight tiles (tile pairs with SWIGLU)
};

// HALVES 2 (K from 4,097 to 16 x 2 x 5 x 32 = 5,120): a wave's share of K in two halves of at most
// MAXS steps. Its slices of x for both stay in registers; the two buffers of weights hold the
// two halves of one tile, each asked for anew (for the next tile) as soon as it is multiplied,
// so a tile's worth of weights is on its way at any time, as with one half.
template <typename TC, int MODE, int MAXS, int HALVES = 1>
__global__ void __launch_bounds__(1024)
gemm_bf16_sweep_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, TC* __restrict__ C, int M,
                       int N, int K, SwPlan pl, SkNorm nm, int layout) {
    constexpr bool SWIGLU = MODE & SK_SWIGLU, SCALED = MODE & SK_SCALED;
    const bool w_tiled = layout & SK_W_TILED, c_tiled = layout & SK_C_TILED;
    static_assert(!(MODE & SK_ADDNORM), "the residual epilogue stays with the skinny kernel");
    constexpr int SUB = SWIGLU ? 2 : 1;
    __shared__ __attribute__((aligned(16))) float red[2][16 * 256];     // [tile parity][wave][lane][4]
    __shared__ float row_fac[16];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / SOC_WAVE), lane = tid % SOC_WAVE;
    const int n_waves = blockDim.x / SOC_WAVE;
    const int g = blockIdx.x, G = gridDim.x;
    const int li = lane % 16, lk = (lane / 16) * 8;
    const int k_begin = wave * pl.k_per_wave, k_end = min(K, k_begin + pl.k_per_wave);
    const int my_items = pl.items > g ? (pl.items - g + G - 1) / G : 0;
    const int n_sub = my_items * SUB;                                    // tiles this workgroup sweeps
    auto tile_of = [&](int q) {
        const int item = g + (q / SUB) * G;
        return SWIGLU ? 2 * item + (q % SUB) : item;
    };

    // Both operands through buffer descriptors that end with their matrices: rows of x beyond
    // M, weight rows beyond N and every slice chosen to lie nowhere read as zeros. No branch
    // lies between a load and its use.
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(X), (short)0, M * K * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(W), (short)0, (int)((size_t)N * K * 2), 0x00020000);
    // (the weights row by row or by tile, as in the skinny kernel)
    const int w_rs = w_tiled ? 32 : K, w_ss = w_tiled ? 512 : 32;
    uint4 xr[HALVES][MAXS];
    uint32_t k_off[HALVES][MAXS];                       // byte offset of the slice from its tile's row 0, or nowhere
#pragma unroll
    for (int h = 0; h < HALVES; ++h)
#pragma unroll
        for (int s = 0; s < MAXS; ++s) {
            const int step = h * MAXS + s, k = k_begin + 32 * step + lk;
            k_off[h][s] = k < k_end ? (uint32_t)((((k_begin / 32 + step) * w_ss) + li * w_rs + lk) * 2) : SW_NOWHERE;
            xr[h][s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                           x_rsrc, k < k_end ? (uint32_t)((li * K + k) * 2) : SW_NOWHERE, 0, 0));
        }
    auto load_w = [&](uint4 (&wb)[MAXS], int q, int h = 0) {
        const bool live = q < n_sub;                    // the same for the whole workgroup
        // a tile starts at 16 K t either way; a weight row beyond N lies beyond the descriptor's end
        const uint32_t row = live ? (uint32_t)((size_t)tile_of(live ? q : 0) * 16 * K * 2) : 0u;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
            wb[s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                        w_rsrc, live && k_off[h][s] != SW_NOWHERE ? row + k_off[h][s] : SW_NOWHERE, 0, 0));
    };
    auto compute = [&](const uint4 (&wb)[MAXS], int h = 0, f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f}) {
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wb[s]),
                                                          __builtin_bit_cast(bf16x8, xr[h][s]), acc, 0, 0, 0);
        return acc;
    };

    uint4 wa[MAXS], wb2[MAXS];
    load_w(wa, 0);
    load_w(wb2, HALVES == 1 ? 1 : 0, HALVES - 1);
    if constexpr (SCALED) {
        // the norm's factor of every row, once per workgroup, while the first loads are on their way
        const int stride = sk_ssq_stride(nm.ssq_tiles);
        for (int m = wave; m < 16; m += n_waves) {
            float s = 0.f;
            if (m < M)
                for (int t = lane; t < nm.ssq_tiles; t += SOC_WAVE) s += nm.ssq_in[(size_t)m * stride + t];
            s = wave_sum(s);
            if (lane == 0) row_fac[m] = 1.0f / sqrtf(s * nm.inv_dim + nm.eps);
        }
    }

    // A reducer (the first 256 threads): row rm of x, column rc of the tile. acc[e] of lane l of
    // a wave is the partial sum for row l % 16 and column 4 (l / 16) + e.
    const int rm = (tid % 256) / 16, rc = tid % 16;
    const int red_at = ((rc / 4) * 16 + rm) * 4 + rc % 4;
    float held = 0.f;                                   // SWIGLU: the gate sum, until the up sum is there
    auto leave = [&](f32x4 acc, int p) {
        *reinterpret_cast<float4*>(&red[p][wave * 256 + lane * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        __syncthreads();
    };
    auto finish = [&](int q, int p) {
        if (tid >= 256 || q >= n_sub) return;           // whole waves leave
        const int tile = tile_of(q);
        float sum = 0.f;
        for (int w = 0; w < n_waves; ++w) sum += red[p][w * 256 + red_at];
        if constexpr (SCALED) sum *= row_fac[rm];
        if constexpr (SWIGLU) {
            if (q % 2 == 0) { held = sum; return; }
            const int col = (tile / 2) * 16 + rc, half = N / 2;
            if (rm < M && col < half)
                C[c_tiled ? ((size_t)(col / 32) * 16 + rm) * 32 + col % 32 : (size_t)rm * half + col] =
                    from_float<TC>(sum * (held / (1.0f + expf(-held))));
        } else {
            const int n = tile * 16 + rc;
            if (rm < M && n < N) C[(size_t)rm * N + n] = from_float<TC>(sum);
        }
    };

    // Two tiles' weights are on their way: a buffer is asked for anew as soon as its tile's
    // sums are in LDS, before the epilogue. The sums of a tile go to the half of `red` of its
    // parity: the reducers read one half while the next tile's sums are written to the other,
    // and one barrier per tile orders both. Past the end of the sweep a round loads zeros
    // from nowhere and has no epilogue, but the barrier all the same.
    if constexpr (HALVES == 1) {
        for (int q = 0; q < n_sub; q += 2) {
            leave(compute(wa), 0);
            load_w(wa, q + 2);
            finish(q, 0);
            leave(compute(wb2), 1);
            load_w(wb2, q + 3);
            finish(q + 1, 1);
        }
    } else {
        // `wa` holds the first half of a tile's K, `wb2` the second
        auto one = [&](int q, int p) {
            f32x4 acc = compute(wa, 0);
            load_w(wa, q + 1, 0);
            acc = compute(wb2, 1, acc);
            load_w(wb2, q + 1, 1);
            leave(acc, p);
            finish(q, p);
        };
        for (int q = 0; q < n_sub; q += 2) {
            one(q, 0);
            one(q + 1, 1);
        }
    }
}

// Shape of a sweep for an [M <= 16] x [N, K] product: waves per workgroup and workgroups; 0
// if the sweep form does not apply (K longer than 16 waves x 320). The tiles (pairs) are
// shared out so that the GPU's 256 compute units get at most one workgroup each, with equal
// numbers of tiles as far as that goes.
SOC_EXPORT int soc_gemm_sweep_plan(int N, int K, int swiglu, int* n_waves, int* workgroups) {
    const int nw = 16;
    if (K > nw * 320) return 0;                         // 8 steps of 32 per wave, or two halves of 5
    const int items = swiglu ? N / 32 : (N + 15) / 16;
    if (items < 1) return 0;
    const int per_wg = (items + 255) / 256;
    *n_waves = nw;
    *workgroups = (items + per_wg - 1) / per_wg;
    return 1;
}

// mode: SK_SWIGLU (C [M, N / 2], N a multiple of 32) or 0 (C [M, N] in c_dtype), each with or
// without SK_SCALED (ssq_in, ssq_tiles, norm_dim, eps; bfloat16 output). K / n_waves rounded
// up to 32 must not exceed 320. The matrices lie below 4 GiB.
SOC_EXPORT int soc_gemm_bf16_sweep(const void* X, const void* W, void* C, int M, int N, int K, int c_dtype,
                                   int mode, int n_waves, int workgroups, const float* ssq_in, int ssq_tiles,
                                   int norm_dim, float eps, int layout, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if ((layout & ~5) || ((layout & SK_W_TILED) && (N % 16 || K % 32)) ||
        ((layout & SK_C_TILED) && (!(mode & SK_SWIGLU) || N % 64)))
        return (int)hipErrorInvalidValue;
    if (M > 16 || K % 8 || K < 8 || !C) return (int)hipErrorInvalidValue;
    if (((size_t)N + 32) * K * 2 >= 0xfffffff0ull) return (int)hipErrorInvalidValue;
    if (n_waves < 1 || n_waves > 16 || workgroups < 1) return (int)hipErrorInvalidValue;
    const bool swiglu = mode & SK_SWIGLU, scaled = mode & SK_SCALED;
    if ((mode & ~3) || (swiglu && N % 32)) return (int)hipErrorInvalidValue;
    if (scaled && (!ssq_in || ssq_tiles < 1 || norm_dim < 1)) return (int)hipErrorInvalidValue;
    if (c_dtype != 0 && c_dtype != 1) return (int)hipErrorInvalidValue;
    if (c_dtype == 0 && mode != 0) return (int)hipErrorInvalidValue;            // float32 output: the plain form only
    SwPlan pl;
    pl.k_per_wave = ((K + n_waves - 1) / n_waves + 31) / 32 * 32;
    if (pl.k_per_wave > 320) return (int)hipErrorInvalidValue;
    pl.items = swiglu ? N / 32 : (N + 15) / 16;
    SkNorm nm{};
    nm.ssq_in = ssq_in; nm.ssq_tiles = ssq_tiles; nm.inv_dim = 1.0f / (float)max(norm_dim, 1); nm.eps = eps;
    const dim3 grid(workgroups < pl.items ? workgroups : pl.items), block(n_waves * 64);
    const int steps = pl.k_per_wave / 32;
#define SOC_SW(TC_, MODE_, MAXS_) \
    hipLaunchKernelGGL((gemm_bf16_sweep_kernel<TC_, MODE_, MAXS_>), grid, block, 0, stream, (const bf16*)X, \
                       (const bf16*)W, (TC_*)C, M, N, K, pl, nm, layout)
#define SOC_SW_STEPS(TC_, MODE_)                                                           \
    do {                                                                                   \
        if (steps <= 2) SOC_SW(TC_, MODE_, 2); else if (steps <= 4) SOC_SW(TC_, MODE_, 4); \
        else if (steps <= 5) SOC_SW(TC_, MODE_, 5); else if (steps <= 8) SOC_SW(TC_, MODE_, 8); \
        else hipLaunchKernelGGL((gemm_bf16_sweep_kernel<TC_, MODE_, 5, 2>), grid, block, 0, stream, (const bf16*)X, \
                                (const bf16*)W, (TC_*)C, M, N, K, pl, nm, layout);         \
    } while (0)
    if (c_dtype == 0) { SOC_SW_STEPS(float, 0); return soc_last_error(); }
    switch (mode) {
        case 0: SOC_SW_STEPS(bf16, 0); break;
        case SK_SCALED: SOC_SW_STEPS(bf16, SK_SCALED); break;
        case SK_SWIGLU: SOC_SW_STEPS(bf16, SK_SWIGLU); break;
        case SK_SWIGLU | SK_SCALED: SOC_SW_STEPS(bf16, SK_SWIGLU | SK_SCALED); break;
        default: return (int)hipErrorInvalidValue;
    }
#undef SOC_SW_STEPS
#undef SOC_SW
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// The sweep for 17 to 64 rows: float32 partial sums of a product whose K is split over
// workgroups. With N split alone, a compute unit would have to bring in all M rows of x for
// its share of the weights (64 rows x K against N / 256 rows x K: at a projection back to the
// model's width, six times the weights), so here a workgroup owns a part of K as well: it
// keeps M rows of its K / parts elements of x in registers (MT blocks of 16 rows; a wave
// holds at most 4 steps of 32 k for 4 blocks, 5 for 2) and sweeps over the weight tiles
// g, g + G, ... of that part. What it leaves is P[part][M][N]; the kernel that adds the
// residual and norms takes such parts and adds them in order. Measured on an MI355X, cold
// weights, 64 rows: [2,560 x 9,728] 17 to 18 us (the library's product 28 us), [2,560 x 4,096]
// 10 us (11 us); 32 rows: 14 us (21 us) and 7.5 us (9 us).
struct SwParts {
    int parts;                      // of K
    int k_part;                     // elements of K per part, a multiple of 32
    int k_per_wave;                 // a multiple of 32
    int tiles;                      // of 16 weight rows
};

template <int MT, int MAXS>
__global__ void __launch_bounds__(1024)
gemm_bf16_sweep_parts_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, float* __restrict__ P,
                             int M, int N, int K, SwParts pl, int layout) {
    extern __shared__ __attribute__((aligned(16))) float parts_red[];          // [tile parity][MT][wave][lane][4]
    const bool w_tiled = layout & SK_W_TILED, x_tiled = layout & SK_X_TILED;
    const int x_rows = layout >> 8;                     // x by tile: [K / 32][x_rows][32], x_rows >= M a multiple of 16
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / SOC_WAVE), lane = tid % SOC_WAVE;
    const int n_waves = blockDim.x / SOC_WAVE;
    const int part = blockIdx.x % pl.parts, g = blockIdx.x / pl.parts, G = gridDim.x / pl.parts;
    const int li = lane % 16, lk = (lane / 16) * 8;
    const int part_end = min(K, (part + 1) * pl.k_part);
    const int k_begin = part * pl.k_part + wave * pl.k_per_wave, k_end = min(part_end, k_begin + pl.k_per_wave);
    const int n_sub = pl.tiles > g ? (pl.tiles - g + G - 1) / G : 0;
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(X), (short)0, (x_tiled ? x_rows : M) * K * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(W), (short)0, (int)((size_t)N * K * 2), 0x00020000);
    const int w_rs = w_tiled ? 32 : K, w_ss = w_tiled ? 512 : 32;
    const int x_rs = x_tiled ? 32 : K, x_ss = x_tiled ? 32 * x_rows : 32;
    uint4 xr[MT][MAXS];
    uint32_t k_off[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const int k = k_begin + 32 * s + lk;
        k_off[s] = k < k_end ? (uint32_t)((((k_begin / 32 + s) * w_ss) + li * w_rs + lk) * 2) : SW_NOWHERE;
        // (row by row, a row beyond M lies beyond the descriptor's end; by tile, a row from M on
        // holds anything or lies beyond x_rows, and its sums are never stored)
#pragma unroll
        for (int t = 0; t < MT; ++t)
            xr[t][s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                           x_rsrc, k < k_end && (!x_tiled || t * 16 + li < x_rows)
                               ? (uint32_t)(((k / 32) * x_ss + (t * 16 + li) * x_rs + k % 32) * 2)
                               : SW_NOWHERE, 0, 0));
    }
    auto load_w = [&](uint4 (&wb)[MAXS], int q) {
        const bool live = q < n_sub;
        const uint32_t row = live ? (uint32_t)((size_t)(g + q * G) * 16 * K * 2) : 0u;
#pragma unroll
        for (int s = 0; s < MAXS; ++s)
            wb[s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                        w_rsrc, live && k_off[s] != SW_NOWHERE ? row + k_off[s] : SW_NOWHERE, 0, 0));
    };
    auto leave = [&](const uint4 (&wb)[MAXS], int p) {
        float* dst = parts_red + (size_t)p * MT * 4096 + wave * 256 + lane * 4;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wb[s]),
                                                              __builtin_bit_cast(bf16x8, xr[t][s]), acc, 0, 0, 0);
            *reinterpret_cast<float4*>(dst + t * 4096) = make_float4(acc[0], acc[1], acc[2], acc[3]);
        }
        __syncthreads();
    };
    // Every thread adds the waves' sums for some outputs: element e of lane l of a wave is row
    // l % 16 of the block and column 4 (l / 16) + e of the tile, and thread r takes l = r / 4,
    // e = r % 4, so that a wave reads consecutive words of LDS.
    auto finish = [&](int q, int p) {
        if (q >= n_sub) return;
        const int n0 = (g + q * G) * 16;
        for (int idx = tid; idx < MT * 256; idx += blockDim.x) {
            const int t = idx / 256, r = idx % 256, l = r / 4;
            const float* src = parts_red + (size_t)p * MT * 4096 + t * 4096 + r;
            float sum = 0.f;
            for (int w = 0; w < n_waves; ++w) sum += src[w * 256];
            const int m = t * 16 + l % 16, n = n0 + 4 * (l / 16) + r % 4;
            if (m < M && n < N) P[((size_t)part * M + m) * N + n] = sum;
        }
    };
    uint4 wa[MAXS], wb2[MAXS];
    load_w(wa, 0);
    load_w(wb2, 1);
    for (int q = 0; q < n_sub; q += 2) {
        leave(wa, 0);
        load_w(wa, q + 2);
        finish(q, 0);
        leave(wb2, 1);
        load_w(wb2, q + 3);
        finish(q + 1, 1);
    }
}

// Shape of such a sweep for M rows (17 to 64): parts of K, K per wave and groups of workgroups
// (parts x groups workgroups in all, at most 256); 0 if it does not apply. The fewest parts
// whose K fits the registers of 16 waves, or up to twice as many if that shares the weights
// out more evenly: what counts is the tiles times the steps of the busiest workgroup.
SOC_EXPORT int soc_gemm_sweep_parts_plan(int M, int N, int K, int* parts, int* k_per_wave, int* groups) {
    if (M < 1 || M > 64 || N < 1 || K < 32) return 0;
    const int max_steps = (M <= 32 ? 5 : 3) * 16;
    const int steps = (K + 31) / 32, tiles = (N + 15) / 16;
    const int least = (steps + max_steps - 1) / max_steps;
    if (least > 64) return 0;
    int best = 0, best_cost = 0, best_groups = 0;
    for (int p = least; p <= 2 * least && p <= 256; ++p) {
        const int room = 256 / p;
        const int per = (tiles + room - 1) / room, cost = per * ((steps + p - 1) / p);
        if (!best || cost < best_cost) { best = p; best_cost = cost; best_groups = (tiles + per - 1) / per; }
    }
    *parts = best;
    *k_per_wave = (((steps + best - 1) / best) + 15) / 16 * 32;
    *groups = best_groups;
    return 1;
}

// P [parts, M, N] float32 = the partial sums of X [M <= 64, K] times W [N, K] transposed, part p
// over the p-th run of ceil(K / 32 / parts) * 32 elements of K. layout: SK_W_TILED; SK_X_TILED with
// R << 8: x lies [K / 32][R][32], R a multiple of 16 from M to 64 (K a multiple of 32).
SOC_EXPORT int soc_gemm_bf16_sweep_parts(const void* X, const void* W, float* P, int M, int N, int K, int parts,
                                         int k_per_wave, int groups, int layout, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    const int x_rows = layout >> 8;
    if (((layout & 0xff) & ~(SK_W_TILED | SK_X_TILED)) || ((layout & SK_W_TILED) && (N % 16 || K % 32))) return (int)hipErrorInvalidValue;
    if ((layout & SK_X_TILED) ? (K % 32 || x_rows < M || x_rows > 64 || x_rows % 16) : x_rows != 0) return (int)hipErrorInvalidValue;
    if (M > 64 || K % 8 || K < 8 || !P) return (int)hipErrorInvalidValue;
    if (((size_t)N + 32) * K * 2 >= 0xfffffff0ull) return (int)hipErrorInvalidValue;
    if (parts < 1 || groups < 1 || parts * groups > 65535 || k_per_wave < 32 || k_per_wave % 32)
        return (int)hipErrorInvalidValue;
    SwParts pl;
    pl.parts = parts;
    pl.k_part = ((K + 31) / 32 + parts - 1) / parts * 32;
    pl.k_per_wave = k_per_wave;
    pl.tiles = (N + 15) / 16;
    const int n_waves = (pl.k_part + k_per_wave - 1) / k_per_wave, steps = k_per_wave / 32;
    const int MT = M <= 32 ? 2 : 4;
    if (n_waves > 16 || steps > (MT == 2 ? 5 : 4)) return (int)hipErrorInvalidValue;
    const dim3 grid(parts * (groups < pl.tiles ? groups : pl.tiles)), block(n_waves * 64);
    const size_t lds = (size_t)2 * MT * 4096 * sizeof(float);
    // (more LDS than a kernel gets unasked: said once per form; not a stream operation)
#define SOC_SWP(MT_, S_)                                                                                       \
    do {                                                                                                       \
        static bool asked = false;                                                                             \
        if (!asked) {                                                                                          \
            const hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_sweep_parts_kernel<MT_, S_>,       \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);    \
            if (e != hipSuccess) return (int)e;                                                                \
            asked = true;                                                                                      \
        }                                                                                                      \
        hipLaunchKernelGGL((gemm_bf16_sweep_parts_kernel<MT_, S_>), grid, block, lds, stream, (const bf16*)X,  \
                           (const bf16*)W, P, M, N, K, pl, layout);                                            \
    } while (0)
#define SOC_SWP_STEPS(MT_)                                                                     \
    do {                                                                                       \
        if (steps <= 1) SOC_SWP(MT_, 1); else if (steps <= 2) SOC_SWP(MT_, 2);                 \
        else if (steps <= 3) SOC_SWP(MT_, 3); else SOC_SWP(MT_, 4);                            \
    } while (0)
    if (MT == 2) { if (steps == 5) SOC_SWP(2, 5); else SOC_SWP_STEPS(2); }
    else SOC_SWP_STEPS(4);
#undef SOC_SWP_STEPS
#undef SOC_SWP
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Products of 17 to 64 rows whose consumer wants whole sums (QKV, gate / up with its activation,
// the output head): K outermost. The sweeps above keep a wave's slices of x in registers and
// walk over weight tiles, which ends at 16 rows of K = 5,120; with more rows x does not fit, and
// a workgroup that re-reads it per tile brings more of x than of the weights into its compute
// unit. Here a workgroup (at most one per compute unit, 8 waves) owns up to T weight tiles
// per pass and keeps their sums, not x, in registers: round r of the walk over K gives wave w
// the 32 k of step 8 r + w, for which it loads MT slices of x (its rows, used for all T tiles
// and never again) and T slices of weights, and multiplies. x thus enters a compute unit once
// per pass and goes through no LDS; the weights of two rounds are on their way at any time.
// At the end of K the eight waves' sums of a tile meet in LDS (one barrier per tile) and the
// workgroup's threads add them and write the outputs, with the activation for a pair of
// gate and up tiles. A workgroup with more than T tiles takes further passes (x is read
// again in each).
struct StPlan {
    int items;                      // weight tiles (tile pairs with SWIGLU)
    int per_wg;                     // items of a workgroup: g, g + G, ...
};

template <typename TC, int MT, int T, int MODE>
__global__ void __launch_bounds__(512)
gemm_bf16_stream_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, TC* __restrict__ C, int M,
                        int N, int K, StPlan pl, int layout) {
    constexpr bool SWIGLU = MODE & SK_SWIGLU;
    constexpr int SUB = SWIGLU ? 2 : 1, J = T / SUB, NW = 8;
    static_assert(T % SUB == 0, "whole pairs");
    const bool w_tiled = layout & SK_W_TILED, x_tiled = layout & SK_X_TILED, c_tiled = layout & SK_C_TILED;
    __shared__ __attribute__((aligned(16))) float red[2][NW][MT][256];   // [tile parity][wave][row block][lane][4]
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / SOC_WAVE), lane = tid % SOC_WAVE;
    const int g = blockIdx.x, G = gridDim.x;
    const int li = lane % 16, lk = (lane / 16) * 8;
    const int steps = (K + 31) / 32, rounds = (steps + NW - 1) / NW;
    // x row by row [M][K], or by tile [K / 32][16 MT][32] (rows from M on hold anything: their
    // sums are never stored)
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(X), (short)0, (x_tiled ? 16 * MT : M) * K * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16*>(W), (short)0, (int)((size_t)N * K * 2), 0x00020000);
    const int w_rs = w_tiled ? 32 : K, w_ss = w_tiled ? 512 : 32;
    const int x_rs = x_tiled ? 32 : K, x_ss = x_tiled ? 16 * MT * 32 : 32;

    for (int pass = 0; pass * J < pl.per_wg; ++pass) {
        // this pass's tiles: byte offset of each tile's first row, or nowhere
        uint32_t tile_at[T];
        int tile_no[T];
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int j = pass * J + t / SUB, item = g + j * G;
            const bool live = j < pl.per_wg && item < pl.items;
            tile_no[t] = live ? (SWIGLU ? 2 * item + t % SUB : item) : -1;
            tile_at[t] = live ? (uint32_t)((size_t)tile_no[t] * 16 * K * 2) : SW_NOWHERE;
        }
        if (tile_no[0] < 0) break;                          // the same in the whole workgroup
        f32x4 acc[T][MT];
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
            for (int b = 0; b < MT; ++b) acc[t][b] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // Loads of round r: nothing touches what they bring before their products (no branch
        // around a load, no select on its result); a slice beyond K, a tile beyond the
        // workgroup's share and a row beyond M are asked of nowhere and read as zeros.
        auto load = [&](int r, uint4 (&wb)[T], uint4 (&xb)[MT]) {
            const int step = r * NW + wave, k = step * 32 + lk;
            const bool ok = r < rounds && k < K;
            const uint32_t k_off = (uint32_t)(((step * w_ss) + li * w_rs + lk) * 2);
#pragma unroll
            for (int b = 0; b < MT; ++b)
                xb[b] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                            x_rsrc, ok ? (uint32_t)((step * x_ss + (b * 16 + li) * x_rs + lk) * 2) : SW_NOWHERE, 0, 0));
#pragma unroll
            for (int t = 0; t < T; ++t)
                wb[t] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(
                            w_rsrc, ok && tile_at[t] != SW_NOWHERE ? tile_at[t] + k_off : SW_NOWHERE, 0, 0));
        };
        auto multiply = [&](const uint4 (&wb)[T], const uint4 (&xb)[MT]) {
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[t][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wb[t]),
                                                                        __builtin_bit_cast(bf16x8, xb[b]), acc[t][b], 0, 0, 0);
        };
        uint4 wa[T], xa[MT], wb2[T], xb2[MT];
        load(0, wa, xa);
        load(1, wb2, xb2);
        for (int r = 0; r < rounds; r += 2) {
            multiply(wa, xa);
            load(r + 2, wa, xa);
            multiply(wb2, xb2);
            load(r + 3, wb2, xb2);
        }
        // The waves' sums of one tile at a time through LDS. acc[e] of lane l is row l % 16 of
        // the block and column 4 (l / 16) + e of the tile. A thread adds the eight waves' sums
        // of two neighbouring columns of one row: thread i takes row i / 8 of the MT * 16 and
        // columns 2 (i % 8), + 1.
        float held[2] = {0.f, 0.f};                          // SWIGLU: the gate sums, until the up sums are there
#pragma unroll
        for (int t = 0; t < T; ++t) {
            const int p = t % 2;
#pragma unroll
            for (int b = 0; b < MT; ++b)
                *reinterpret_cast<float4*>(&red[p][wave][b][lane * 4]) =
                    make_float4(acc[t][b][0], acc[t][b][1], acc[t][b][2], acc[t][b][3]);
            __syncthreads();
            if (tile_no[t] < 0) continue;                    // the same in the whole workgroup
            for (int i = tid; i < MT * 16 * 8; i += 512) {
                const int m = i / 8, c2 = (i % 8) * 2;
                const int at = ((c2 / 4) * 16 + m % 16) * 4 + c2 % 4;
                float s0 = 0.f, s1 = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float2 v = *reinterpret_cast<const float2*>(&red[p][w][m / 16][at]);
                    s0 += v.x; s1 += v.y;
                }
                if constexpr (SWIGLU) {
                    if (t % 2 == 0) { held[0] = s0; held[1] = s1; continue; }
                    const int col = (tile_no[t] / 2) * 16 + c2, half = N / 2;
                    if (m < M && col < half) {
                        const float a0 = s0 * (held[0] / (1.0f + expf(-held[0])));
                        const float a1 = s1 * (held[1] / (1.0f + expf(-held[1])));
                        // (by tile: [half / 32][16 MT][32], for the product that reads it next)
                        TC* at = c_tiled ? C + ((size_t)(col / 32) * (16 * MT) + m) * 32 + col % 32 : C + (size_t)m * half + col;
                        at[0] = from_float<TC>(a0);
                        if (col + 1 < half) at[1] = from_float<TC>(a1);
                    }
                } else {
                    const int n = tile_no[t] * 16 + c2;
                    if (m < M && n < N) {
                        C[(size_t)m * N + n] = from_float<TC>(s0);
                        if (n + 1 < N) C[(size_t)m * N + n + 1] = from_float<TC>(s1);
                    }
                }
            }
        }
        __syncthreads();                                     // the next pass writes `red` again
    }
}

// Shape of such a product: workgroups and items (tiles, or tile pairs with SWIGLU) per
// workgroup; 0 if the form does not apply.
SOC_EXPORT int soc_gemm_stream_plan(int M, int N, int K, int swiglu, int* workgroups, int* per_wg) {
    if (M < 1 || M > 64 || N < 1 || K < 8 || K % 8) return 0;
    if (swiglu && N % 32) return 0;
    const int items = swiglu ? N / 32 : (N + 15) / 16;
    const int per = (items + 255) / 256;
    *per_wg = per;
    *workgroups = (items + per - 1) / per;
    return 1;
}

// C = X [M <= 64, K] times W [N, K] transposed, in c_dtype (0 float32, 1 bfloat16), or with
// mode SK_SWIGLU C [M, N / 2] = silu(gate) * up over weight rows that alternate in blocks of 16
// (bfloat16 out). layout: SK_W_TILED, and SK_X_TILED: x is laid out [K / 32][R][32] with R = 32 for
// M <= 32, 48 for M <= 48 and 64 above (K a multiple of 32); SK_C_TILED (with SK_SWIGLU, N a multiple of
// 64): C is written [N / 64][R][32] with the same R. The matrices lie below 4 GiB.
SOC_EXPORT int soc_gemm_bf16_stream(const void* X, const void* W, void* C, int M, int N, int K, int c_dtype,
                                    int mode, int workgroups, int per_wg, int layout, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if ((layout & ~(SK_W_TILED | SK_X_TILED | SK_C_TILED)) || ((layout & SK_W_TILED) && (N % 16 || K % 32)) ||
        ((layout & SK_X_TILED) && K % 32) || ((layout & SK_C_TILED) && (!(mode & SK_SWIGLU) || N % 64)))
        return (int)hipErrorInvalidValue;
    if (M > 64 || K % 8 || K < 8 || !C) return (int)hipErrorInvalidValue;
    if (((size_t)N + 32) * K * 2 >= 0xfffffff0ull || (size_t)64 * K * 2 >= 0xfffffff0ull) return (int)hipErrorInvalidValue;
    const bool swiglu = mode & SK_SWIGLU;
    if ((mode & ~SK_SWIGLU) || (swiglu && (N % 32 || c_dtype != 1))) return (int)hipErrorInvalidValue;
    if (c_dtype != 0 && c_dtype != 1) return (int)hipErrorInvalidValue;
    StPlan pl;
    pl.items = swiglu ? N / 32 : (N + 15) / 16;
    if (workgroups < 1 || per_wg < 1 || (long)workgroups * per_wg < pl.items) return (int)hipErrorInvalidValue;
    pl.per_wg = per_wg;
    const dim3 grid(workgroups < pl.items ? workgroups : pl.items), block(512);
    const int tiles_wg = per_wg * (swiglu ? 2 : 1);          // tiles of a workgroup: as many per pass as fit
    const int T = tiles_wg <= 2 ? 2 : tiles_wg <= 4 ? 4 : tiles_wg % 6 == 0 || tiles_wg > 8 ? 6 : 4;
#define SOC_ST(TC_, MT_, T_, MODE_) \
    hipLaunchKernelGGL((gemm_bf16_stream_kernel<TC_, MT_, T_, MODE_>), grid, block, 0, stream, (const bf16*)X, \
                       (const bf16*)W, (TC_*)C, M, N, K, pl, layout)
#define SOC_ST_T(TC_, MT_, MODE_) \
    do { if (T == 2) SOC_ST(TC_, MT_, 2, MODE_); else if (T == 4) SOC_ST(TC_, MT_, 4, MODE_); else SOC_ST(TC_, MT_, 6, MODE_); } while (0)
#define SOC_ST_MT(TC_, MODE_) \
    do { if (M <= 32) SOC_ST_T(TC_, 2, MODE_); else if (M <= 48) SOC_ST_T(TC_, 3, MODE_); else SOC_ST_T(TC_, 4, MODE_); } while (0)
    if (swiglu) SOC_ST_MT(bf16, SK_SWIGLU);
    else if (c_dtype == 1) SOC_ST_MT(bf16, 0);
    else SOC_ST_MT(float, 0);
#undef SOC_ST_MT
#undef SOC_ST_T
#undef SOC_ST
    return soc_last_error();
}
