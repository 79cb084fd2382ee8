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

// Measurement aid (bench.py --fill-path): what the global -> LDS path of a CU delivers when nothing else runs.
// Four waves per workgroup, each streaming 8 KB batches (eight global_load_lds_dwordx4) into its own 32 KB of LDS
// with four batches in flight -- 128 KB per workgroup, one workgroup per CU, the footprint of a GEMM tile ring.  A
// batch comes either from the wave's own stretch of `big` (a region far larger than the caches: HBM) or from
// `small` (a region the L2 holds): all from small when hits_per_miss < 0, all from big when it is 0, else one big
// batch after every hits_per_miss small ones.  row_stride = 0: a batch is 8 KB of consecutive bytes.  row_stride > 0:
// a batch is a 64-row x 128-byte tile of a row-major matrix with that many bytes between rows, and the next batch of
// the same source is the tile 128 bytes further along the rows -- the way a GEMM's k loop walks a k-major operand.
// No arithmetic, nothing is read back from LDS.
__global__ __launch_bounds__(256) void fill_probe_kernel(const char* big, long big_bytes, const char* small_, long small_bytes,
                                                         int hits_per_miss, int batches, long row_stride) {
    constexpr int DEPTH = 4, NLD = 8, BATCH = NLD * 1024;
    __shared__ __attribute__((aligned(16))) unsigned char ring[4 * DEPTH * BATCH];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const long wid = (long)blockIdx.x * 4 + wave;
    const unsigned lds0 = lds_addr(ring) + (unsigned)(wave * DEPTH * BATCH);
    // lane's byte offset inside a batch's first load, and between the eight loads of a batch
    const unsigned off = row_stride ? (unsigned)((lane >> 3) * row_stride + (lane & 7) * 16) : (unsigned)lane * 16u;
    const unsigned step = row_stride ? (unsigned)(8 * row_stride) : 1024u;
    // tiled: a wave owns blocks of 64 rows; batch j of a source is tile (j % tiles_per_row) of block (j / tiles_per_row)
    const long tiles_per_row = row_stride ? row_stride / 128 : 1;
    const long big_blocks = row_stride ? big_bytes / (64 * row_stride) : 1, small_blocks = row_stride ? small_bytes / (64 * row_stride) : 1;
    int nb = 0, ns = 0;     // batches taken from big / small so far
    for (int b = 0; b < batches; ++b) {
        const bool miss = hits_per_miss == 0 || (hits_per_miss > 0 && b % (hits_per_miss + 1) == 0);   // wave-uniform
        const char* src;
        if (row_stride == 0) {
            src = miss ? big + ((wid * batches + b) * (long)BATCH) % big_bytes
                       : small_ + ((wid * 7 + b) * (long)BATCH) % small_bytes;
        } else if (miss) {
            const long blk = (wid * ((batches + tiles_per_row - 1) / tiles_per_row + 1) + nb / tiles_per_row) % big_blocks;
            src = big + blk * 64 * row_stride + (nb % tiles_per_row) * 128;
            ++nb;
        } else {
            const long blk = (wid * 3 + ns / tiles_per_row) % small_blocks;
            src = small_ + blk * 64 * row_stride + (ns % tiles_per_row) * 128;
            ++ns;
        }
        src = uniform_ptr(src);
        const unsigned dst = lds0 + (unsigned)((b % DEPTH) * BATCH);
#pragma unroll
        for (int i = 0; i < NLD; ++i) dma16_saddr_lds(off + (unsigned)i * step, src, dst + (unsigned)(i * 1024));
        wait_vmcnt<(DEPTH - 1) * NLD>();
    }
    wait_vmcnt<0>();
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

extern "C" int tp_fill_probe(const void* big, int64_t big_bytes, const void* small_region, int64_t small_bytes,
                             int hits_per_miss, int workgroups, int batches_per_wave, int64_t row_stride, void* stream) {
    using namespace tp;
    if (!big || !small_region || workgroups <= 0 || workgroups > 65535 || batches_per_wave <= 0 ||
        big_bytes < 8192 || small_bytes < 8192 || big_bytes % 8192 || small_bytes % 8192 ||
        (((uintptr_t)big | (uintptr_t)small_region) & 15)) {
        set_error("tp_fill_probe: regions must be 16-byte aligned whole multiples of 8192 bytes, counts positive");
        return TP_ERR_ARG;
    }
    if (row_stride < 0 || row_stride % 128 || (row_stride > 0 && (64 * row_stride > small_bytes || 64 * row_stride > big_bytes ||
                                                                   8 * row_stride > 0x7fffffffL))) {
        set_error("tp_fill_probe: row_stride must be 0 or a multiple of 128 with 64 rows inside either region");
        return TP_ERR_ARG;
    }
    fill_probe_kernel<<<workgroups, 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        (const char*)big, big_bytes, (const char*)small_region, small_bytes, hits_per_miss, batches_per_wave, (long)row_stride);
    return launch_status("tp_fill_probe");
}
