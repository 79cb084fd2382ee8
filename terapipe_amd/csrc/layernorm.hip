// Fused LayerNorm forward / backward: one workgroup per row, the row cached in registers, 16-byte
// coalesced accesses, fp32 statistics, wave64 shuffle + LDS block reductions.
#include "common.h"

namespace tp {

template <int NREDUCE>
__device__ __forceinline__ void block_sum(float (&v)[NREDUCE], float* scratch /* [NREDUCE][16] */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
#pragma unroll
    for (int i = 0; i < NREDUCE; ++i) v[i] = wave_sum(v[i]);
    __syncthreads();  // scratch may still be read by the previous reduction
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < NREDUCE; ++i) scratch[i * 16 + wave] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NREDUCE; ++i) {
        float s = 0.f;
        for (int w = 0; w < nw; ++w) s += scratch[i * 16 + w];
        v[i] = s;
    }
}

template <typename T> __device__ __forceinline__ void load_chunk(const T* p, float* out) {
    constexpr int CH = 16 / sizeof(T);
    uint4 raw = *reinterpret_cast<const uint4*>(p);
    if constexpr (sizeof(T) == 2) {
        const T* h = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int e = 0; e < CH; ++e) out[e] = Elem<T>::to_float(h[e]);
    } else {
        const float* f = reinterpret_cast<const float*>(&raw);
#pragma unroll
        for (int e = 0; e < CH; ++e) out[e] = f[e];
    }
}

template <typename T> __device__ __forceinline__ void store_chunk(T* p, const float* v) {
    constexpr int CH = 16 / sizeof(T);
    uint4 raw;
    if constexpr (sizeof(T) == 2) {
        T* h = reinterpret_cast<T*>(&raw);
#pragma unroll
        for (int e = 0; e < CH; ++e) h[e] = Elem<T>::from_float(v[e]);
    } else {
        float* f = reinterpret_cast<float*>(&raw);
#pragma unroll
        for (int e = 0; e < CH; ++e) f[e] = v[e];
    }
    *reinterpret_cast<uint4*>(p) = raw;
}

// Where the kernels take their input row from when it is still the fp32 partial sums of a k-split GEMM:
// value = sum_z partial[z][row][col] (+ bias[col]) (+ resid[row][col]), rounded to T, written to out16 (the
// tensor the split-K reduce kernel would have produced) and used from there on.  partial == nullptr: the
// row is read from the kernel's ordinary input pointer.
struct LnPartialSrc {
    const float* partial; int nsplit; long zstride;
    const void* bias; const void* resid; void* out16;
};

template <typename T>
__device__ __forceinline__ void load_input_chunk(const LnPartialSrc& ps, const T* direct, long row, int c, int E,
                                                 float* out) {
    constexpr int CH = 16 / sizeof(T);
    const long off = row * E + (long)c * CH;
    if (ps.partial == nullptr) {
        load_chunk<T>(direct + off, out);
        return;
    }
#pragma unroll
    for (int e = 0; e < CH; ++e) out[e] = 0.f;
    for (int z = 0; z < ps.nsplit; ++z) {
        const float* pp = ps.partial + (long)z * ps.zstride + off;
#pragma unroll
        for (int q = 0; q < CH / 4; ++q) {
            const float4 v = *reinterpret_cast<const float4*>(pp + 4 * q);
            out[4 * q] += v.x; out[4 * q + 1] += v.y; out[4 * q + 2] += v.z; out[4 * q + 3] += v.w;
        }
    }
    if (ps.bias) {
        float b[CH];
        load_chunk<T>(reinterpret_cast<const T*>(ps.bias) + (long)c * CH, b);
#pragma unroll
        for (int e = 0; e < CH; ++e) out[e] += b[e];
    }
    if (ps.resid) {
        float r[CH];
        load_chunk<T>(reinterpret_cast<const T*>(ps.resid) + off, r);
#pragma unroll
        for (int e = 0; e < CH; ++e) out[e] += r[e];
    }
    // round through T exactly as the stand-alone reduce kernel does, and keep the rounded tensor
#pragma unroll
    for (int e = 0; e < CH; ++e) out[e] = Elem<T>::to_float(Elem<T>::from_float(out[e]));
    store_chunk<T>(reinterpret_cast<T*>(ps.out16) + off, out);
}

template <typename T, int MAXC>
__global__ __launch_bounds__(1024) void ln_fwd_kernel(LnPartialSrc ps, const T* __restrict__ x, const T* __restrict__ gamma,
                                                      const T* __restrict__ beta, T* __restrict__ y,
                                                      float* __restrict__ mean, float* __restrict__ rstd,
                                                      int M, int E, float eps) {
    constexpr int CH = 16 / sizeof(T);
    __shared__ float scratch[16];
    const int row = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
    const int nch = E / CH;
    float v[MAXC][CH];
    float s[1] = {0.f};
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        int c = tid + i * nt;
        if (c < nch) {
            load_input_chunk<T>(ps, x, row, c, E, v[i]);
#pragma unroll
            for (int e = 0; e < CH; ++e) s[0] += v[i][e];
        }
    }
    block_sum<1>(s, scratch);
    const float mu = s[0] / (float)E;
    float q[1] = {0.f};
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        int c = tid + i * nt;
        if (c < nch) {
#pragma unroll
            for (int e = 0; e < CH; ++e) { float d = v[i][e] - mu; q[0] += d * d; }
        }
    }
    block_sum<1>(q, scratch);
    const float rs = 1.0f / sqrtf(q[0] / (float)E + eps);
    if (tid == 0) { mean[row] = mu; rstd[row] = rs; }
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        int c = tid + i * nt;
        if (c < nch) {
            float gm[CH], bt[CH], o[CH];
            load_chunk<T>(gamma + (long)c * CH, gm);
            load_chunk<T>(beta + (long)c * CH, bt);
#pragma unroll
            for (int e = 0; e < CH; ++e) o[e] = (v[i][e] - mu) * rs * gm[e] + bt[e];
            store_chunk<T>(y + (long)row * E + (long)c * CH, o);
        }
    }
}

template <typename T, int MAXC>
__global__ __launch_bounds__(1024) void ln_bwd_kernel(LnPartialSrc ps, const T* __restrict__ dy, const T* __restrict__ x,
                                                      const float* __restrict__ mean, const float* __restrict__ rstd,
                                                      const T* __restrict__ gamma, const T* __restrict__ dres,
                                                      T* __restrict__ dx, float* dgamma, float* dbeta,
                                                      float* cs_dres, float* cs_dx, int M, int E) {
    constexpr int CH = 16 / sizeof(T);
    __shared__ float scratch[32];
    const int tid = threadIdx.x, nt = blockDim.x;
    const int nch = E / CH;
    float gm[MAXC][CH], a_dg[MAXC][CH], a_db[MAXC][CH], a_dr[MAXC][CH], a_dx[MAXC][CH];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        int c = tid + i * nt;
        if (c < nch) load_chunk<T>(gamma + (long)c * CH, gm[i]);
#pragma unroll
        for (int e = 0; e < CH; ++e) { a_dg[i][e] = 0.f; a_db[i][e] = 0.f; a_dr[i][e] = 0.f; a_dx[i][e] = 0.f; }
    }
    for (int row = blockIdx.x; row < M; row += gridDim.x) {
        const float mu = mean[row], rs = rstd[row];
        float g[MAXC][CH], xh[MAXC][CH];
        float s[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            int c = tid + i * nt;
            if (c < nch) {
                float d[CH], xv[CH];
                load_input_chunk<T>(ps, dy, row, c, E, d);
                load_chunk<T>(x + (long)row * E + (long)c * CH, xv);
#pragma unroll
                for (int e = 0; e < CH; ++e) {
                    xh[i][e] = (xv[e] - mu) * rs;
                    g[i][e] = d[e] * gm[i][e];
                    s[0] += g[i][e];
                    s[1] += g[i][e] * xh[i][e];
                    a_dg[i][e] += d[e] * xh[i][e];
                    a_db[i][e] += d[e];
                }
            }
        }
        block_sum<2>(s, scratch);
        const float m1 = s[0] / (float)E, m2 = s[1] / (float)E;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            int c = tid + i * nt;
            if (c < nch) {
                float o[CH];
#pragma unroll
                for (int e = 0; e < CH; ++e) o[e] = rs * (g[i][e] - m1 - xh[i][e] * m2);
                if (dres) {
                    float r[CH];
                    load_chunk<T>(dres + (long)row * E + (long)c * CH, r);
#pragma unroll
                    for (int e = 0; e < CH; ++e) { o[e] += r[e]; a_dr[i][e] += r[e]; }
                }
#pragma unroll
                for (int e = 0; e < CH; ++e) a_dx[i][e] += o[e];
                store_chunk<T>(dx + (long)row * E + (long)c * CH, o);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        int c = tid + i * nt;
        if (c < nch) {
#pragma unroll
            for (int e = 0; e < CH; ++e) {
                long col = (long)c * CH + e;
                if (dgamma) {
                    atomicAdd(dgamma + col, a_dg[i][e]);
                    atomicAdd(dbeta + col, a_db[i][e]);
                }
                if (cs_dres && dres) atomicAdd(cs_dres + col, a_dr[i][e]);
                if (cs_dx) atomicAdd(cs_dx + col, a_dx[i][e]);
            }
        }
    }
}

// dgamma / dbeta over a block of rows: 256 threads = 32 column chunks (8 columns each) x 8 row lanes,
// 64 rows per block, row lanes combined in LDS, one atomic per column per block.
template <typename T>
__global__ __launch_bounds__(256) void ln_param_grads_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                             const float* __restrict__ mean,
                                                             const float* __restrict__ rstd, float* dgamma,
                                                             float* dbeta, int M, int E) {
    __shared__ float sg[8][256], sb[8][256];
    const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int col0 = (blockIdx.x * 32 + cl) * 8;
    const int rbase = blockIdx.y * 64;
    float ag[8], ab[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { ag[e] = 0.f; ab[e] = 0.f; }
    if (col0 < E) {
        for (int rr = 0; rr < 8; ++rr) {
            const int row = rbase + rr * 8 + rl;
            if (row < M) {
                const float mu = mean[row], rs = rstd[row];
                float d[8], xv[8];
                if constexpr (sizeof(T) == 2) {
                    load_chunk<T>(dy + (long)row * E + col0, d);
                    load_chunk<T>(x + (long)row * E + col0, xv);
                } else {
                    load_chunk<T>(dy + (long)row * E + col0, d);
                    load_chunk<T>(dy + (long)row * E + col0 + 4, d + 4);
                    load_chunk<T>(x + (long)row * E + col0, xv);
                    load_chunk<T>(x + (long)row * E + col0 + 4, xv + 4);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) { ag[e] += d[e] * (xv[e] - mu) * rs; ab[e] += d[e]; }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) { sg[rl][cl * 8 + e] = ag[e]; sb[rl][cl * 8 + e] = ab[e]; }
    __syncthreads();
    const int c = threadIdx.x, col = blockIdx.x * 256 + c;
    if (col < E) {
        float tg = 0.f, tb = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) { tg += sg[r][c]; tb += sb[r][c]; }
        atomicAdd(dgamma + col, tg);
        atomicAdd(dbeta + col, tb);
    }
}

// The vector-parameter gradients of a layer in ONE launch: up to kVecGradMax reductions over the rows of a step,
// each either column sums of dy (a bias gradient) or the LayerNorm pair (dgamma += sum dy * xhat, dbeta += sum dy).
// A block of 256 threads = 32 column chunks (8 columns, 16-byte loads for 16-bit types) x 8 row lanes covers
// 256 columns x kVecGradRows rows of one problem; the row lanes are combined in LDS and every column then costs one
// atomic per block.  Blocks are numbered problem by problem (first_block[]).
constexpr int kVecGradMax = 8;
constexpr int kVecGradRows = 128;
struct VecGradProblem {
    const void* dy; const void* x; const float* mean; const float* rstd;
    float* acc0; float* acc1;
    long ld; int M, N;
};
struct VecGradArgs {
    VecGradProblem p[kVecGradMax];
    int first_block[kVecGradMax + 1];
    int n;
};

template <typename T>
__global__ __launch_bounds__(256) void vec_param_grads_kernel(VecGradArgs args) {
    __shared__ float sg[8][256], sb[8][256];
    int pi = 0;
#pragma unroll
    for (int i = 1; i < kVecGradMax; ++i)
        if (i < args.n && (int)blockIdx.x >= args.first_block[i]) pi = i;
    // (constant indices only: a dynamically indexed kernel argument would be copied to scratch memory)
    VecGradProblem pr = args.p[0];
    int first = args.first_block[0];
#pragma unroll
    for (int i = 1; i < kVecGradMax; ++i)
        if (pi == i) { pr = args.p[i]; first = args.first_block[i]; }
    const int ncb = (pr.N + 255) / 256;
    const int local = (int)blockIdx.x - first;
    const int cb = local % ncb, rb = local / ncb;
    const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int col0 = (cb * 32 + cl) * 8;
    const int r0 = rb * kVecGradRows, r1 = min(pr.M, r0 + kVecGradRows);
    const T* dy = reinterpret_cast<const T*>(pr.dy);
    const T* x = reinterpret_cast<const T*>(pr.x);
    float ag[8], ab[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { ag[e] = 0.f; ab[e] = 0.f; }
    if (col0 < pr.N) {
        for (int row = r0 + rl; row < r1; row += 8) {
            float d[8];
            load_chunk<T>(dy + (long)row * pr.ld + col0, d);
            if constexpr (sizeof(T) == 4) load_chunk<T>(dy + (long)row * pr.ld + col0 + 4, d + 4);
            if (x) {
                const float mu = pr.mean[row], rs = pr.rstd[row];
                float xv[8];
                load_chunk<T>(x + (long)row * pr.ld + col0, xv);
                if constexpr (sizeof(T) == 4) load_chunk<T>(x + (long)row * pr.ld + col0 + 4, xv + 4);
#pragma unroll
                for (int e = 0; e < 8; ++e) ag[e] += d[e] * (xv[e] - mu) * rs;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) ab[e] += d[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) { sg[rl][cl * 8 + e] = ag[e]; sb[rl][cl * 8 + e] = ab[e]; }
    __syncthreads();
    const int c = threadIdx.x, col = cb * 256 + c;
    if (col < pr.N) {
        float tg = 0.f, tb = 0.f;
#pragma unroll
        for (int r = 0; r < 8; ++r) { tg += sg[r][c]; tb += sb[r][c]; }
        if (x) {
            atomicAdd(pr.acc0 + col, tg);
            atomicAdd(pr.acc1 + col, tb);
        } else {
            atomicAdd(pr.acc0 + col, tb);
        }
    }
}

static int ln_geometry(int E, int dtype, int* threads, int* maxc) {
    const int ch = dtype == TP_F32 ? 4 : 8;
    if (E <= 0 || E % ch) { set_error("layernorm: E=%d must be a positive multiple of %d", E, ch); return TP_ERR_UNSUPPORTED; }
    const int nch = E / ch;
    int nt = 64;
    while (nt < nch && nt < 1024) nt *= 2;
    int mc = (nch + nt - 1) / nt;
    if (mc > 4) { set_error("layernorm: E=%d too large (max %d)", E, 1024 * 4 * ch); return TP_ERR_UNSUPPORTED; }
    *threads = nt;
    *maxc = mc <= 1 ? 1 : (mc <= 2 ? 2 : 4);
    return TP_OK;
}

template <typename T>
static void launch_ln_fwd(int maxc, int nt, const LnPartialSrc& ps, const void* x, const void* gamma,
                          const void* beta, void* y, float* mean, float* rstd, int M, int E, float eps, hipStream_t s) {
    const T* xp = (const T*)x; const T* gp = (const T*)gamma; const T* bp = (const T*)beta; T* yp = (T*)y;
    if (maxc == 1) ln_fwd_kernel<T, 1><<<M, nt, 0, s>>>(ps, xp, gp, bp, yp, mean, rstd, M, E, eps);
    else if (maxc == 2) ln_fwd_kernel<T, 2><<<M, nt, 0, s>>>(ps, xp, gp, bp, yp, mean, rstd, M, E, eps);
    else ln_fwd_kernel<T, 4><<<M, nt, 0, s>>>(ps, xp, gp, bp, yp, mean, rstd, M, E, eps);
}

template <typename T>
static void launch_ln_bwd(int maxc, int nt, int grid, const LnPartialSrc& ps, const void* dy, const void* x, const float* mean,
                          const float* rstd, const void* gamma, const void* dres, void* dx, float* dg,
                          float* db, float* cr, float* cx, int M, int E, hipStream_t s) {
    const T* dyp = (const T*)dy; const T* xp = (const T*)x; const T* gp = (const T*)gamma;
    const T* rp = (const T*)dres; T* dxp = (T*)dx;
    if (maxc == 1) ln_bwd_kernel<T, 1><<<grid, nt, 0, s>>>(ps, dyp, xp, mean, rstd, gp, rp, dxp, dg, db, cr, cx, M, E);
    else if (maxc == 2) ln_bwd_kernel<T, 2><<<grid, nt, 0, s>>>(ps, dyp, xp, mean, rstd, gp, rp, dxp, dg, db, cr, cx, M, E);
    else ln_bwd_kernel<T, 4><<<grid, nt, 0, s>>>(ps, dyp, xp, mean, rstd, gp, rp, dxp, dg, db, cr, cx, M, E);
}

static int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", what, hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

}  // namespace tp

static int ln_fwd_impl(const tp::LnPartialSrc& ps, const void* x, const void* gamma, const void* beta, void* y,
                       float* mean, float* rstd, int M, int E, float eps, int dtype, void* stream) {
    using namespace tp;
    if (!x || !gamma || !beta || !y || !mean || !rstd) { set_error("tp_layernorm_fwd: null pointer"); return TP_ERR_ARG; }
    if (M <= 0) { set_error("tp_layernorm_fwd: M=%d", M); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_layernorm_fwd: bad dtype %d", dtype); return TP_ERR_ARG; }
    if (((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)beta | (uintptr_t)y) & 15) { set_error("tp_layernorm_fwd: pointers must be 16-byte aligned"); return TP_ERR_ARG; }
    int nt, maxc;
    int rc = ln_geometry(E, dtype, &nt, &maxc);
    if (rc != TP_OK) return rc;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
    case TP_F32: launch_ln_fwd<float>(maxc, nt, ps, x, gamma, beta, y, mean, rstd, M, E, eps, s); break;
    case TP_F16: launch_ln_fwd<f16>(maxc, nt, ps, x, gamma, beta, y, mean, rstd, M, E, eps, s); break;
    default: launch_ln_fwd<bf16>(maxc, nt, ps, x, gamma, beta, y, mean, rstd, M, E, eps, s); break;
    }
    return check_launch("tp_layernorm_fwd");
}

extern "C" int tp_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean,
                                float* rstd, int M, int E, float eps, int dtype, void* stream) {
    tp::LnPartialSrc ps = {nullptr, 0, 0, nullptr, nullptr, nullptr};
    return ln_fwd_impl(ps, x, gamma, beta, y, mean, rstd, M, E, eps, dtype, stream);
}

static int check_partials(const char* who, const float* partials, int nsplit, const void* out16) {
    if (!partials || nsplit < 1 || !out16) { tp::set_error("%s: partials, nsplit >= 1 and the output tensor are required", who); return TP_ERR_ARG; }
    if (((uintptr_t)partials | (uintptr_t)out16) & 15) { tp::set_error("%s: pointers must be 16-byte aligned", who); return TP_ERR_ARG; }
    return TP_OK;
}

extern "C" int tp_layernorm_fwd_partials(const float* partials, int nsplit, const void* bias, const void* residual,
                                         void* x_out, const void* gamma, const void* beta, void* y, float* mean,
                                         float* rstd, int M, int E, float eps, int dtype, void* stream) {
    int rc = check_partials("tp_layernorm_fwd_partials", partials, nsplit, x_out);
    if (rc != TP_OK) return rc;
    if (((uintptr_t)bias | (uintptr_t)residual) & 15) { tp::set_error("tp_layernorm_fwd_partials: pointers must be 16-byte aligned"); return TP_ERR_ARG; }
    tp::LnPartialSrc ps = {partials, nsplit, (long)M * E, bias, residual, x_out};
    return ln_fwd_impl(ps, x_out, gamma, beta, y, mean, rstd, M, E, eps, dtype, stream);
}

static int ln_bwd_impl(const tp::LnPartialSrc& ps, const void* dy, const void* x, const float* mean, const float* rstd,
                       const void* gamma, const void* dres, void* dx, float* dgamma_acc,
                       float* dbeta_acc, float* colsum_dres_acc, float* colsum_dx_acc, int M, int E,
                       int dtype, void* stream) {
    using namespace tp;
    if (!dy || !x || !mean || !rstd || !gamma || !dx) { set_error("tp_layernorm_bwd: null pointer"); return TP_ERR_ARG; }
    if ((dgamma_acc == nullptr) != (dbeta_acc == nullptr)) { set_error("tp_layernorm_bwd: dgamma_acc and dbeta_acc must both be given or both be NULL"); return TP_ERR_ARG; }
    if (M <= 0) { set_error("tp_layernorm_bwd: M=%d", M); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_layernorm_bwd: bad dtype %d", dtype); return TP_ERR_ARG; }
    if (((uintptr_t)dy | (uintptr_t)x | (uintptr_t)gamma | (uintptr_t)dres | (uintptr_t)dx) & 15) { set_error("tp_layernorm_bwd: pointers must be 16-byte aligned"); return TP_ERR_ARG; }
    int nt, maxc;
    int rc = ln_geometry(E, dtype, &nt, &maxc);
    if (rc != TP_OK) return rc;
    // with accumulators every block ends in E atomics per array, so fewer blocks sweep more rows each;
    // without them one block per row
    int grid = (dgamma_acc || colsum_dres_acc || colsum_dx_acc) ? (M < 128 ? M : 128) : M;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
    case TP_F32: launch_ln_bwd<float>(maxc, nt, grid, ps, dy, x, mean, rstd, gamma, dres, dx, dgamma_acc, dbeta_acc, colsum_dres_acc, colsum_dx_acc, M, E, s); break;
    case TP_F16: launch_ln_bwd<f16>(maxc, nt, grid, ps, dy, x, mean, rstd, gamma, dres, dx, dgamma_acc, dbeta_acc, colsum_dres_acc, colsum_dx_acc, M, E, s); break;
    default: launch_ln_bwd<bf16>(maxc, nt, grid, ps, dy, x, mean, rstd, gamma, dres, dx, dgamma_acc, dbeta_acc, colsum_dres_acc, colsum_dx_acc, M, E, s); break;
    }
    return check_launch("tp_layernorm_bwd");
}

extern "C" int tp_layernorm_bwd(const void* dy, const void* x, const float* mean, const float* rstd,
                                const void* gamma, const void* dres, void* dx, float* dgamma_acc,
                                float* dbeta_acc, float* colsum_dres_acc, float* colsum_dx_acc, int M, int E,
                                int dtype, void* stream) {
    tp::LnPartialSrc ps = {nullptr, 0, 0, nullptr, nullptr, nullptr};
    return ln_bwd_impl(ps, dy, x, mean, rstd, gamma, dres, dx, dgamma_acc, dbeta_acc, colsum_dres_acc, colsum_dx_acc,
                       M, E, dtype, stream);
}

extern "C" int tp_layernorm_bwd_partials(const float* partials, int nsplit, void* dy_out, const void* x,
                                         const float* mean, const float* rstd, const void* gamma, const void* dres,
                                         void* dx, float* dgamma_acc, float* dbeta_acc, float* colsum_dres_acc,
                                         float* colsum_dx_acc, int M, int E, int dtype, void* stream) {
    int rc = check_partials("tp_layernorm_bwd_partials", partials, nsplit, dy_out);
    if (rc != TP_OK) return rc;
    tp::LnPartialSrc ps = {partials, nsplit, (long)M * E, nullptr, nullptr, dy_out};
    return ln_bwd_impl(ps, dy_out, x, mean, rstd, gamma, dres, dx, dgamma_acc, dbeta_acc, colsum_dres_acc,
                       colsum_dx_acc, M, E, dtype, stream);
}

extern "C" int tp_ln_param_grads(const void* dy, const void* x, const float* mean, const float* rstd,
                                 float* dgamma_acc, float* dbeta_acc, int M, int E, int dtype, void* stream) {
    using namespace tp;
    if (!dy || !x || !mean || !rstd || !dgamma_acc || !dbeta_acc) { set_error("tp_ln_param_grads: null pointer"); return TP_ERR_ARG; }
    if (M <= 0 || E <= 0 || E % 8) { set_error("tp_ln_param_grads: M=%d, E=%d (E must be a multiple of 8)", M, E); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_ln_param_grads: bad dtype %d", dtype); return TP_ERR_ARG; }
    if (((uintptr_t)dy | (uintptr_t)x) & 15) { set_error("tp_ln_param_grads: pointers must be 16-byte aligned"); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    dim3 grid((E + 255) / 256, (M + 63) / 64);
    switch (dtype) {
    case TP_F32: ln_param_grads_kernel<float><<<grid, 256, 0, s>>>((const float*)dy, (const float*)x, mean, rstd, dgamma_acc, dbeta_acc, M, E); break;
    case TP_F16: ln_param_grads_kernel<f16><<<grid, 256, 0, s>>>((const f16*)dy, (const f16*)x, mean, rstd, dgamma_acc, dbeta_acc, M, E); break;
    default: ln_param_grads_kernel<bf16><<<grid, 256, 0, s>>>((const bf16*)dy, (const bf16*)x, mean, rstd, dgamma_acc, dbeta_acc, M, E); break;
    }
    return check_launch("tp_ln_param_grads");
}

extern "C" int tp_vec_param_grads(const tp_vecgrad_desc* descs, int n, int dtype, void* stream) {
    using namespace tp;
    if (!descs || n < 1 || n > kVecGradMax) { set_error("tp_vec_param_grads: 1 to %d problems (n=%d)", kVecGradMax, n); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_vec_param_grads: bad dtype %d", dtype); return TP_ERR_ARG; }
    VecGradArgs args;
    int blocks = 0;
    for (int i = 0; i < n; ++i) {
        const tp_vecgrad_desc& d = descs[i];
        if (!d.dy || !d.acc0 || d.M <= 0 || d.N <= 0 || d.N % 8 || d.ld < d.N || d.ld % 8) {
            set_error("tp_vec_param_grads: problem %d: null pointer or bad shape (M=%d N=%d ld=%ld; N and ld multiples of 8)", i, d.M, d.N, (long)d.ld);
            return TP_ERR_ARG;
        }
        if (d.x && (!d.mean || !d.rstd || !d.acc1)) { set_error("tp_vec_param_grads: problem %d: the LayerNorm pair needs mean, rstd and acc1", i); return TP_ERR_ARG; }
        if (((uintptr_t)d.dy | (uintptr_t)d.x) & 15) { set_error("tp_vec_param_grads: problem %d: pointers must be 16-byte aligned", i); return TP_ERR_ARG; }
        args.p[i] = {d.dy, d.x, d.mean, d.rstd, d.acc0, d.acc1, (long)d.ld, d.M, d.N};
        args.first_block[i] = blocks;
        blocks += ((d.N + 255) / 256) * ((d.M + kVecGradRows - 1) / kVecGradRows);
    }
    for (int i = n; i < kVecGradMax; ++i) { args.p[i] = args.p[0]; args.first_block[i] = blocks; }
    args.first_block[kVecGradMax] = blocks;
    args.n = n;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
    case TP_F32: vec_param_grads_kernel<float><<<blocks, 256, 0, s>>>(args); break;
    case TP_F16: vec_param_grads_kernel<f16><<<blocks, 256, 0, s>>>(args); break;
    default: vec_param_grads_kernel<bf16><<<blocks, 256, 0, s>>>(args); break;
    }
    return check_launch("tp_vec_param_grads");
}
