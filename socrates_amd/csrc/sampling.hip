// Next-token choice from float32 logits, one workgroup per row.
//
// temperature 0: argmax, the lowest index among equal maxima (the reference is greedy
// only: model/inference_paged.py:166, 193; ties: bench/day_8/equivalence.py:105-107).
// temperature T > 0: an inverse-CDF draw from softmax(logits / T). The uniform number
// comes from a counter-based hash of the request's seed and the number of draws it has
// made, so a request's tokens do not depend on its neighbours in the batch. Every sum is
// float32 and taken in a fixed order.
#include "common.h"
#include "sampling.h"

#include <mutex>
#include <stdio.h>

constexpr int SAMPLE_THREADS = 1024;

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

__device__ __forceinline__ float uniform_of(uint64_t seed, uint64_t draw) {
    const uint64_t h = splitmix64(splitmix64(seed) ^ (draw * 0xD1342543DE82EF95ull));
    return (float)(h >> 40) * (1.0f / 16777216.0f);          // 24 bits: exact in float32
}

struct MaxIdx { float v; int i; };

__device__ __forceinline__ MaxIdx better(MaxIdx a, MaxIdx b) {
    // NaN never wins; equal values keep the lower index
    if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
    return a;
}

__device__ MaxIdx block_argmax(const float* __restrict__ x, int V, MaxIdx* scratch) {
    MaxIdx best = {-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < V; i += blockDim.x) best = better(best, MaxIdx{x[i], i});
#pragma unroll
    for (int m = SOC_WAVE / 2; m > 0; m >>= 1) {
        MaxIdx o = {__shfl_xor(best.v, m, SOC_WAVE), __shfl_xor(best.i, m, SOC_WAVE)};
        best = better(best, o);
    }
    const int wave = threadIdx.x / SOC_WAVE, lane = threadIdx.x % SOC_WAVE;
    if (lane == 0) scratch[wave] = best;
    __syncthreads();
    MaxIdx r = scratch[0];
    for (int w = 1; w < blockDim.x / SOC_WAVE; ++w) r = better(r, scratch[w]);
    __syncthreads();
    if (r.i == 0x7fffffff) r.i = 0;                          // a row of NaN or -inf
    return r;
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
              const long long* __restrict__ seed, const long long* __restrict__ draws,
              int* __restrict__ out, int V) {
    __shared__ MaxIdx scratch[SAMPLE_THREADS / SOC_WAVE];
    __shared__ float chunk_sum[SAMPLE_THREADS];
    __shared__ int chosen;
    const int row = blockIdx.x;
    const float* x = logits + (size_t)row * V;
    const MaxIdx top = block_argmax(x, V, scratch);
    const float T = temperature ? temperature[row] : 0.f;
    if (!(T > 0.f)) {
        if (threadIdx.x == 0) out[row] = top.i;
        return;
    }
    // Each thread owns a run of consecutive entries so that the CDF is taken in index order.
    const int per = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int begin = min(V, (int)threadIdx.x * per), end = min(V, begin + per);
    const float inv_T = 1.0f / T;
    float s = 0.f;
    for (int i = begin; i < end; ++i) s += expf((x[i] - top.v) * inv_T);
    chunk_sum[threadIdx.x] = s;
    if (threadIdx.x == 0) chosen = -1;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int t = 0; t < SAMPLE_THREADS; ++t) total += chunk_sum[t];
        const float target = uniform_of((uint64_t)seed[row], (uint64_t)draws[row]) * total;
        float run = 0.f;
        int t = 0;
        for (; t < SAMPLE_THREADS - 1; ++t) {
            if (run + chunk_sum[t] > target) break;
            run += chunk_sum[t];
        }
        // walk the owning run; the first entry whose cumulative weight exceeds the target
        const int b = min(V, t * per), e = min(V, b + per);
        int pick = top.i;
        for (int i = b; i < e; ++i) {
            run += expf((x[i] - top.v) * inv_T);
            if (run > target) { pick = i; break; }
        }
        chosen = pick;
    }
    __syncthreads();
    if (threadIdx.x == 0) out[row] = chosen;
}

// Greedy choice for many rows at once: a row is cut into chunks, one workgroup per chunk
// finds its best (value, index), and the last step picks among the chunks, lowest index first.
constexpr int ARGMAX_THREADS = 256;

__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_chunks_kernel(const float* __restrict__ logits, MaxIdx* __restrict__ partial, int V, int chunk) {
    __shared__ MaxIdx scratch[ARGMAX_THREADS / SOC_WAVE];
    const int row = blockIdx.y, c = blockIdx.x;
    const int begin = c * chunk, end = min(V, begin + chunk);
    const float* x = logits + (size_t)row * V;
    MaxIdx best = {-INFINITY, 0x7fffffff};
    for (int i = begin + threadIdx.x; i < end; i += ARGMAX_THREADS) best = better(best, MaxIdx{x[i], i});
#pragma unroll
    for (int m = SOC_WAVE / 2; m > 0; m >>= 1) {
        MaxIdx o = {__shfl_xor(best.v, m, SOC_WAVE), __shfl_xor(best.i, m, SOC_WAVE)};
        best = better(best, o);
    }
    if (threadIdx.x % SOC_WAVE == 0) scratch[threadIdx.x / SOC_WAVE] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        MaxIdx r = scratch[0];
        for (int w = 1; w < ARGMAX_THREADS / SOC_WAVE; ++w) r = better(r, scratch[w]);
        partial[(size_t)row * gridDim.x + c] = r;
    }
}

__global__ void argmax_pick_kernel(const MaxIdx* __restrict__ partial, int* __restrict__ out, int n_chunks) {
    const int row = blockIdx.x;
    MaxIdx best = {-INFINITY, 0x7fffffff};
    for (int c = threadIdx.x; c < n_chunks; c += SOC_WAVE) best = better(best, partial[(size_t)row * n_chunks + c]);
#pragma unroll
    for (int m = SOC_WAVE / 2; m > 0; m >>= 1) {
        MaxIdx o = {__shfl_xor(best.v, m, SOC_WAVE), __shfl_xor(best.i, m, SOC_WAVE)};
        best = better(best, o);
    }
    if (threadIdx.x == 0) out[row] = best.i == 0x7fffffff ? 0 : best.i;
}

// logits [n, V] float32 -> out [n] int32. partial: scratch of n * n_chunks (float, int) pairs.
SOC_EXPORT int soc_argmax(const float* logits, void* partial, int* out, int n, int V, int n_chunks,
                          hipStream_t stream) {
    if (n <= 0) return 0;
    if (V < 1 || n_chunks < 1 || n > 65535) return (int)hipErrorInvalidValue;
    const int chunk = (V + n_chunks - 1) / n_chunks;
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(n_chunks, n), dim3(ARGMAX_THREADS), 0, stream, logits,
                       (MaxIdx*)partial, V, chunk);
    hipLaunchKernelGGL(argmax_pick_kernel, dim3(n), dim3(SOC_WAVE), 0, stream, (const MaxIdx*)partial, out,
                       n_chunks);
    return soc_last_error();
}

// ---------------------------------------------------------------------------------------------
// Greedy choice without a workspace argument and without an allocation (see sampling.h): the
// chunk results go to a file-scope device array. Host code never uses the array's name as an
// address: it is looked up once per device with hipGetSymbolAddress, and the kernels get the
// looked-up pointer as an argument, exactly as they get the caller's workspace in soc_argmax.
static __device__ __align__(256) MaxIdx scratch[SOC_ARGMAX_STATIC_MAX_ROWS * SOC_ARGMAX_STATIC_MAX_CHUNKS];

constexpr int STATIC_MAX_DEVICES = 64;
static MaxIdx* scratch_of_device[STATIC_MAX_DEVICES];          // null until looked up
static std::mutex scratch_lock;

static void say(char* message, int message_len, const char* text, long a = 0, long b = 0) {
    if (message && message_len > 0) snprintf(message, (size_t)message_len, text, a, b);
}

// The array's address on the current device, looked up at the first call on that device.
static int static_scratch(MaxIdx** ptr, char* message, int message_len) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) {
        say(message, message_len, "soc_argmax_static: hipGetDevice failed (HIP error %ld)", (long)err);
        return (int)err;
    }
    if (device < 0 || device >= STATIC_MAX_DEVICES) {
        say(message, message_len, "soc_argmax_static: device %ld is beyond the %ld this library keeps a pointer for",
            device, STATIC_MAX_DEVICES);
        return (int)hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (!scratch_of_device[device]) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p) {
            say(message, message_len, "soc_argmax_static: hipGetSymbolAddress failed on device %ld (HIP error %ld)",
                device, (long)err);
            return err != hipSuccess ? (int)err : (int)hipErrorInvalidSymbol;
        }
        scratch_of_device[device] = (MaxIdx*)p;
    }
    *ptr = scratch_of_device[device];
    return 0;
}

SOC_EXPORT int soc_argmax_static_init(char* message, int message_len) {
    MaxIdx* p = nullptr;
    return static_scratch(&p, message, message_len);
}

SOC_EXPORT int soc_argmax_static(const float* logits, int* out, int n, int V, hipStream_t stream,
                                 char* message, int message_len) {
    if (n <= 0) return 0;
    if (n > SOC_ARGMAX_STATIC_MAX_ROWS) {
        say(message, message_len, "soc_argmax_static: %ld rows asked for, the static workspace holds %ld; "
            "use soc_argmax with a workspace of your own", n, SOC_ARGMAX_STATIC_MAX_ROWS);
        return (int)hipErrorInvalidValue;
    }
    if (V < 1 || !logits || !out) {
        say(message, message_len, "soc_argmax_static: needs logits, out and a vocabulary of at least 1 (got %ld)", V);
        return (int)hipErrorInvalidValue;
    }
    MaxIdx* partial = nullptr;
    const int err = static_scratch(&partial, message, message_len);
    if (err) return err;
    const int n_chunks = max(1, min(SOC_ARGMAX_STATIC_MAX_CHUNKS, V / 2048));
    const int chunk = (V + n_chunks - 1) / n_chunks;
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(n_chunks, n), dim3(ARGMAX_THREADS), 0, stream, logits,
                       partial, V, chunk);
    hipLaunchKernelGGL(argmax_pick_kernel, dim3(n), dim3(SOC_WAVE), 0, stream, (const MaxIdx*)partial, out,
                       n_chunks);
    const int launched = soc_last_error();
    if (launched) say(message, message_len, "soc_argmax_static: launch failed (HIP error %ld)", launched);
    return launched;
}

// logits [n, V] float32; temperature [n] float32 or null (all greedy); seed, draws [n] int64.
SOC_EXPORT int soc_sample(const float* logits, const float* temperature, const long long* seed,
                          const long long* draws, int* out, int n, int V, hipStream_t stream) {
    if (n <= 0) return 0;
    if (V < 1) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(sample_kernel, dim3(n), dim3(SAMPLE_THREADS), 0, stream, logits, temperature,
                       seed, draws, out, V);
    return soc_last_error();
}
