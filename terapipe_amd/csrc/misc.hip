// Error plumbing and the small helper kernels of the C ABI.
#include "common.h"

#include <cstdarg>
#include <cstdio>

namespace tp {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

template <typename T>
__global__ __launch_bounds__(256) void accum_cast_kernel(T* __restrict__ dst, const float* __restrict__ src,
                                                         long n, int accumulate) {
    long i = (long)blockIdx.x * 256 + threadIdx.x;
    const long stride = (long)gridDim.x * 256;
    for (; i < n; i += stride) {
        float v = src[i];
        if (accumulate) v += Elem<T>::to_float(dst[i]);
        dst[i] = Elem<T>::from_float(v);
    }
}

// one thread per column, 32 rows per block; partial sums go to the fp32 accumulators with atomics
template <typename T>
__global__ __launch_bounds__(256) void colsum_acc_kernel(const T* __restrict__ x, long ldx, float* acc, int M, int N) {
    const int col = blockIdx.x * 256 + threadIdx.x;
    if (col >= N) return;
    const int r0 = blockIdx.y * 32, r1 = min(M, r0 + 32);
    float s = 0.f;
    for (int r = r0; r < r1; ++r) s += Elem<T>::to_float(x[(long)r * ldx + col]);
    atomicAdd(acc + col, s);
}

__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* dst, long n) {
    long i = (long)blockIdx.x * 256 + threadIdx.x;
    const long stride = (long)gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = 0u;
}

static int launch_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", what, hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

}  // namespace tp

extern "C" int tp_version(void) { return 100; }

extern "C" const char* tp_last_error(void) { return tp::g_err; }

extern "C" int tp_accum_cast(void* dst, const float* src, int64_t n, int accumulate, int dtype, void* stream) {
    using namespace tp;
    if (!dst || !src || n <= 0) { set_error("tp_accum_cast: bad arguments"); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_accum_cast: bad dtype %d", dtype); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int grid = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
    switch (dtype) {
    case TP_F32: accum_cast_kernel<float><<<grid, 256, 0, s>>>((float*)dst, src, n, accumulate); break;
    case TP_F16: accum_cast_kernel<f16><<<grid, 256, 0, s>>>((f16*)dst, src, n, accumulate); break;
    default: accum_cast_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)dst, src, n, accumulate); break;
    }
    return launch_status("tp_accum_cast");
}

extern "C" int tp_colsum_acc(const void* x, int64_t ldx, float* acc, int M, int N, int dtype, void* stream) {
    using namespace tp;
    if (!x || !acc || M <= 0 || N <= 0 || ldx < N) { set_error("tp_colsum_acc: bad arguments"); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_colsum_acc: bad dtype %d", dtype); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    dim3 grid((N + 255) / 256, (M + 31) / 32);
    switch (dtype) {
    case TP_F32: colsum_acc_kernel<float><<<grid, 256, 0, s>>>((const float*)x, ldx, acc, M, N); break;
    case TP_F16: colsum_acc_kernel<f16><<<grid, 256, 0, s>>>((const f16*)x, ldx, acc, M, N); break;
    default: colsum_acc_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)x, ldx, acc, M, N); break;
    }
    return launch_status("tp_colsum_acc");
}

extern "C" int tp_zero_words(void* dst, int64_t n_words, void* stream) {
    using namespace tp;
    if (!dst || n_words <= 0 || ((uintptr_t)dst & 3)) { set_error("tp_zero_words: bad arguments"); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int grid = (int)((n_words + 255) / 256 < 4096 ? (n_words + 255) / 256 : 4096);
    zero_words_kernel<<<grid, 256, 0, s>>>((uint32_t*)dst, n_words);
    return launch_status("tp_zero_words");
}
