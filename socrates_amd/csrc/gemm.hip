// Matrix products C[M, N] = A[M, K] * W[N, K]^T (both operands K-contiguous, the layout of
// activations and of nn.Linear weights; model/qwen/qwen_kv_paged.py:140-143, 224).
//
//  gemm_generic_kernel   any sizes and any mix of float32 / bfloat16 operands; plain FMA in
//                        float32, K summed in order. This is the true 32-bit path.
//  gemm_bf16_mfma_kernel bfloat16 operands, 128x128x64 tiles through LDS, 16x16x32 MFMA with
//                        float32 accumulators: prompt portions (large M).
//  gemm_bf16_skinny_kernel bfloat16, M <= 64 (decode): bound by streaming W once from HBM. A
//                        workgroup owns 16 rows of W, its waves split K, every lane keeps
//                        several 16-byte loads of W in flight, the weights are the MFMA's
//                        first operand so that one lane ends up with four consecutive
//                        outputs; the waves' partial tiles are summed through LDS in a fixed
//                        order.
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
constexpr int SK_UNROLL = 4;            // 16-byte loads of W in flight per lane
constexpr int SK_MAX_PARTS = 32;        // waves x m-tiles whose partials fit the LDS buffer

template <typename TC, int MT>
__global__ void __launch_bounds__(1024)
gemm_bf16_skinny_kernel(const bf16* __restrict__ X, const bf16* __restrict__ W, TC* __restrict__ C,
                        int M, int N, int K, int k_per_wave) {
    __shared__ float red[SK_MAX_PARTS * 256];
    const int tid = threadIdx.x, wave = tid / SOC_WAVE, lane = tid % SOC_WAVE;
    const int n_waves = blockDim.x / SOC_WAVE;
    const int n0 = blockIdx.x * 16;
    const int li = lane % 16, lk = (lane / 16) * 8;
    const int k_begin = wave * k_per_wave, k_end = min(K, k_begin + k_per_wave);
    const bool w_row_ok = n0 + li < N;
    const bf16* w_row = W + (size_t)(w_row_ok ? n0 + li : 0) * K;

    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

    for (int k0 = k_begin; k0 < k_end; k0 += 32 * SK_UNROLL) {
        uint4 wf[SK_UNROLL];
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k = k0 + 32 * u + lk;
            wf[u] = (w_row_ok && k < k_end) ? *reinterpret_cast<const uint4*>(w_row + k)
                                            : make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < SK_UNROLL; ++u) {
            const int k = k0 + 32 * u + lk;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int m = t * 16 + li;
                uint4 xf = (m < M && k < k_end) ? *reinterpret_cast<const uint4*>(X + (size_t)m * K + k)
                                                : make_uint4(0u, 0u, 0u, 0u);
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    *reinterpret_cast<bf16x8*>(&wf[u]), *reinterpret_cast<bf16x8*>(&xf), acc[t], 0, 0, 0);
            }
        }
    }
    // acc[t][r] is the partial of C[m = 16 t + lane % 16][n = n0 + 4 * (lane / 16) + r]
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[((wave * MT + t) * 64 + lane) * 4 + r] = acc[t][r];
    __syncthreads();
    for (int idx = tid; idx < MT * 256; idx += blockDim.x) {
        const int t = idx / 256, ln = (idx % 256) / 4, r = idx % 4;
        float sum = 0.f;
        for (int w = 0; w < n_waves; ++w) sum += red[((w * MT + t) * 64 + ln) * 4 + r];
        const int m = t * 16 + ln % 16, n = n0 + 4 * (ln / 16) + r;
        if (m < M && n < N) C[(size_t)m * N + n] = from_float<TC>(sum);
    }
}

template <typename TC, int MT>
static int launch_skinny(const void* X, const void* W, void* C, int M, int N, int K, int n_waves,
                         hipStream_t stream) {
    int k_per_wave = ((K + n_waves - 1) / n_waves + 31) / 32 * 32;
    hipLaunchKernelGGL((gemm_bf16_skinny_kernel<TC, MT>), dim3((N + 15) / 16), dim3(n_waves * 64), 0,
                       stream, (const bf16*)X, (const bf16*)W, (TC*)C, M, N, K, k_per_wave);
    return soc_last_error();
}

// M <= 64, K a multiple of 8. n_waves (1..16) is how many waves of a workgroup split K;
// 0 lets the kernel choose from the shape.
SOC_EXPORT int soc_gemm_bf16_skinny(const void* X, const void* W, void* C, int M, int N, int K,
                                    int c_dtype, int n_waves, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 || K < 8) return (int)hipErrorInvalidValue;
    const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    if (n_waves <= 0) {
        const int tiles = (N + 15) / 16;
        n_waves = tiles >= 2048 ? 4 : (tiles >= 512 ? 8 : 16);
    }
    while (n_waves > 1 && (n_waves * MT > SK_MAX_PARTS || K / n_waves < 128)) n_waves /= 2;
    if (n_waves > 16) n_waves = 16;
#define SOC_SK(TC_, MT_) return launch_skinny<TC_, MT_>(X, W, C, M, N, K, n_waves, stream)
    if (c_dtype == 0) {
        if (MT == 1) SOC_SK(float, 1);
        if (MT == 2) SOC_SK(float, 2);
        SOC_SK(float, 4);
    }
    if (MT == 1) SOC_SK(bf16, 1);
    if (MT == 2) SOC_SK(bf16, 2);
    SOC_SK(bf16, 4);
#undef SOC_SK
}
