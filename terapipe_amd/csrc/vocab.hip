// Token embedding lookup and vocabulary cross-entropy (the two ends of the layer stack at tensor-parallel
// size 1: reference mpu/layers.py:126-141 and mpu/cross_entropy.py:25-104).
#include "common.h"

namespace tp {

// out[m, :] = W[ids[m], :]; one workgroup per token, 16-byte chunks
template <typename T>
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const int64_t* __restrict__ ids, const T* __restrict__ W,
                                                            T* __restrict__ out, int E, int V) {
    constexpr int CH = 16 / sizeof(T);
    const long m = blockIdx.x;
    const int64_t id = ids[m];
    const bool ok = id >= 0 && id < V;          // out-of-range ids give a zero row (masked rows of the reference)
    const uint4* src = reinterpret_cast<const uint4*>(W + (ok ? id : 0) * (long)E);
    uint4* dst = reinterpret_cast<uint4*>(out + m * (long)E);
    for (int c = threadIdx.x; c < E / CH; c += 256) dst[c] = ok ? src[c] : make_uint4(0, 0, 0, 0);
}

// dW_acc[ids[m], :] += dout[m, :] (fp32 accumulators, atomics: a token id may repeat)
template <typename T>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int64_t* __restrict__ ids, const T* __restrict__ dout,
                                                            float* dW, int E, int V) {
    const long m = blockIdx.x;
    const int64_t id = ids[m];
    if (id < 0 || id >= V) return;
    for (int e = threadIdx.x; e < E; e += 256) atomicAdd(dW + id * (long)E + e, Elem<T>::to_float(dout[m * (long)E + e]));
}

__device__ __forceinline__ float block_reduce(float v, float* scratch, bool is_max) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float u = __shfl_xor(v, o, 64);
        v = is_max ? fmaxf(v, u) : v + u;
    }
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float r = scratch[0];
    for (int w = 1; w < nw; ++w) r = is_max ? fmaxf(r, scratch[w]) : r + scratch[w];
    return r;
}

// One workgroup per row of logits [M, ld] (columns >= V are padding and ignored):
//   loss[m] = log(sum_v exp(z_v - max)) + max - z[target[m]]
//   logits[m, v] <- (softmax_v - [v == target[m]]) * grad_scale   (in place, as the reference overwrites its
//   input with the softmax and returns it as the gradient); padding columns <- 0.
template <typename T>
__global__ __launch_bounds__(1024) void cross_entropy_kernel(T* __restrict__ logits, long ld, const int64_t* __restrict__ target,
                                                             float* __restrict__ loss, int V, int Vpad, float grad_scale) {
    __shared__ float scratch[16];
    const long m = blockIdx.x;
    T* z = logits + m * ld;
    float mx = -INFINITY;
    for (int v = threadIdx.x; v < V; v += blockDim.x) mx = fmaxf(mx, Elem<T>::to_float(z[v]));
    mx = block_reduce(mx, scratch, true);
    float s = 0.f;
    for (int v = threadIdx.x; v < V; v += blockDim.x) s += expf(Elem<T>::to_float(z[v]) - mx);
    s = block_reduce(s, scratch, false);
    const int64_t t = target[m];
    const bool tok = t >= 0 && t < V;
    if (threadIdx.x == 0) loss[m] = logf(s) + mx - (tok ? Elem<T>::to_float(z[t]) : 0.f);
    __syncthreads();        // z[t] is read above before any thread overwrites it
    const float inv = 1.0f / s;
    for (int v = threadIdx.x; v < Vpad; v += blockDim.x) {
        float g = 0.f;
        if (v < V) g = (expf(Elem<T>::to_float(z[v]) - mx) * inv - ((tok && v == t) ? 1.f : 0.f)) * grad_scale;
        z[v] = Elem<T>::from_float(g);
    }
}

// The same with 16-byte accesses (rows 16-byte aligned, Vpad a whole number of chunks): the row is read from
// HBM once for the maximum, the two later passes find it in the caches, and the gradient goes out in
// 16-byte stores.
template <typename T>
__global__ __launch_bounds__(1024) void cross_entropy_vec_kernel(T* __restrict__ logits, long ld, const int64_t* __restrict__ target,
                                                                 float* __restrict__ loss, int V, int Vpad, float grad_scale) {
    constexpr int CH = 16 / sizeof(T);
    __shared__ float scratch[16];
    const long m = blockIdx.x;
    T* z = logits + m * ld;
    const uint4* zv = reinterpret_cast<const uint4*>(z);
    const int nch = Vpad / CH;
    float mx = -INFINITY;
    for (int c = threadIdx.x; c < nch; c += blockDim.x) {
        const uint4 raw = zv[c];
        const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int i = 0; i < CH; ++i)
            if (c * CH + i < V) mx = fmaxf(mx, Elem<T>::to_float(e[i]));
    }
    mx = block_reduce(mx, scratch, true);
    float s = 0.f;
    for (int c = threadIdx.x; c < nch; c += blockDim.x) {
        const uint4 raw = zv[c];
        const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int i = 0; i < CH; ++i)
            if (c * CH + i < V) s += expf(Elem<T>::to_float(e[i]) - mx);
    }
    s = block_reduce(s, scratch, false);
    const int64_t t = target[m];
    const bool tok = t >= 0 && t < V;
    if (threadIdx.x == 0) loss[m] = logf(s) + mx - (tok ? Elem<T>::to_float(z[t]) : 0.f);
    __syncthreads();        // z[t] is read above before any thread overwrites it
    const float inv = 1.0f / s;
    for (int c = threadIdx.x; c < nch; c += blockDim.x) {
        const uint4 raw = zv[c];
        const T* e = reinterpret_cast<const T*>(&raw);
        uint4 outv;
        T* o = reinterpret_cast<T*>(&outv);
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int v = c * CH + i;
            float g = 0.f;
            if (v < V) g = (expf(Elem<T>::to_float(e[i]) - mx) * inv - ((tok && v == t) ? 1.f : 0.f)) * grad_scale;
            o[i] = Elem<T>::from_float(g);
        }
        reinterpret_cast<uint4*>(z)[c] = outv;
    }
}

// Rows of up to 1024 * NCH chunks (65536 columns): the row is read once into registers (NCH 16-byte chunks per
// lane), maximum, sum and gradient are taken from there -- one read and one write of the logits in all.
template <typename T, int NCH>
__global__ __launch_bounds__(1024) void cross_entropy_reg_kernel(T* __restrict__ logits, long ld, const int64_t* __restrict__ target,
                                                                 float* __restrict__ loss, int V, int Vpad, float grad_scale) {
    constexpr int CH = 16 / sizeof(T);
    __shared__ float scratch[16];
    const long m = blockIdx.x;
    T* z = logits + m * ld;
    const uint4* zv = reinterpret_cast<const uint4*>(z);
    const int nch = Vpad / CH;
    const int64_t t = target[m];
    const bool tok = t >= 0 && t < V;
    const float zt = tok ? Elem<T>::to_float(z[t]) : 0.f;      // read before anything is overwritten
    // (the row stays in its 16-bit / fp32 form: 8 chunks are 32 registers, which keeps two workgroups on a CU;
    // holding exp(z - max) as floats instead costs 64 registers, one workgroup per CU and 1.5x the time)
    uint4 row[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = k * 1024 + threadIdx.x;
        row[k] = c < nch ? zv[c] : make_uint4(0, 0, 0, 0);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const T* e = reinterpret_cast<const T*>(&row[k]);
        const int v0 = (k * 1024 + threadIdx.x) * CH;
#pragma unroll
        for (int i = 0; i < CH; ++i)
            if (v0 + i < V) mx = fmaxf(mx, Elem<T>::to_float(e[i]));
    }
    mx = block_reduce(mx, scratch, true);
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const T* e = reinterpret_cast<const T*>(&row[k]);
        const int v0 = (k * 1024 + threadIdx.x) * CH;
#pragma unroll
        for (int i = 0; i < CH; ++i)
            if (v0 + i < V) s += expf(Elem<T>::to_float(e[i]) - mx);
    }
    s = block_reduce(s, scratch, false);
    if (threadIdx.x == 0) loss[m] = logf(s) + mx - zt;
    const float inv = 1.0f / s;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
        const int c = k * 1024 + threadIdx.x;
        if (c >= nch) continue;
        const T* e = reinterpret_cast<const T*>(&row[k]);
        uint4 outv;
        T* o = reinterpret_cast<T*>(&outv);
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int v = c * CH + i;
            float g = 0.f;
            if (v < V) g = (expf(Elem<T>::to_float(e[i]) - mx) * inv - ((tok && v == t) ? 1.f : 0.f)) * grad_scale;
            o[i] = Elem<T>::from_float(g);
        }
        reinterpret_cast<uint4*>(z)[c] = outv;
    }
}

// x[m, :n] *= scale[m] in place (grad_input.mul_(grad_output.unsqueeze(-1)), mpu/cross_entropy.py:97)
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(T* __restrict__ x, long ld, const float* __restrict__ scale, int n) {
    const long m = blockIdx.y;
    const float sc = scale[m];
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v < n) x[m * ld + v] = Elem<T>::from_float(Elem<T>::to_float(x[m * ld + v]) * sc);
}

// the same with 16-byte accesses (rows 16-byte aligned, n a whole number of chunks)
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_vec_kernel(T* __restrict__ x, long ld, const float* __restrict__ scale, int nch) {
    constexpr int CH = 16 / sizeof(T);
    const long m = blockIdx.y;
    const float sc = scale[m];
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= nch) return;
    uint4* p = reinterpret_cast<uint4*>(x + m * ld) + c;
    uint4 raw = *p;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < CH; ++i) e[i] = Elem<T>::from_float(Elem<T>::to_float(e[i]) * sc);
    *p = raw;
}

static int vocab_status(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", what, hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

}  // namespace tp

extern "C" int tp_embedding_fwd(const int64_t* ids, const void* weight, void* out, int M, int E, int V, int dtype,
                                void* stream) {
    using namespace tp;
    if (!ids || !weight || !out || M <= 0 || V <= 0) { set_error("tp_embedding_fwd: bad argument"); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_embedding_fwd: bad dtype %d", dtype); return TP_ERR_ARG; }
    const int ch = dtype == TP_F32 ? 4 : 8;
    if (E <= 0 || E % ch || (((uintptr_t)weight | (uintptr_t)out) & 15)) { set_error("tp_embedding_fwd: E=%d must be a multiple of %d and the tensors 16-byte aligned", E, ch); return TP_ERR_UNSUPPORTED; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
    case TP_F32: embedding_fwd_kernel<float><<<M, 256, 0, s>>>(ids, (const float*)weight, (float*)out, E, V); break;
    case TP_F16: embedding_fwd_kernel<f16><<<M, 256, 0, s>>>(ids, (const f16*)weight, (f16*)out, E, V); break;
    default: embedding_fwd_kernel<bf16><<<M, 256, 0, s>>>(ids, (const bf16*)weight, (bf16*)out, E, V); break;
    }
    return vocab_status("tp_embedding_fwd");
}

extern "C" int tp_embedding_bwd(const int64_t* ids, const void* dout, float* dweight_acc, int M, int E, int V, int dtype,
                                void* stream) {
    using namespace tp;
    if (!ids || !dout || !dweight_acc || M <= 0 || E <= 0 || V <= 0) { set_error("tp_embedding_bwd: bad argument"); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_embedding_bwd: bad dtype %d", dtype); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (dtype) {
    case TP_F32: embedding_bwd_kernel<float><<<M, 256, 0, s>>>(ids, (const float*)dout, dweight_acc, E, V); break;
    case TP_F16: embedding_bwd_kernel<f16><<<M, 256, 0, s>>>(ids, (const f16*)dout, dweight_acc, E, V); break;
    default: embedding_bwd_kernel<bf16><<<M, 256, 0, s>>>(ids, (const bf16*)dout, dweight_acc, E, V); break;
    }
    return vocab_status("tp_embedding_bwd");
}

extern "C" int tp_cross_entropy(void* logits, int64_t ld, const int64_t* target, float* loss, int M, int V, int Vpad,
                                float grad_scale, int dtype, void* stream) {
    using namespace tp;
    if (!logits || !target || !loss || M <= 0 || V <= 0 || Vpad < V || ld < Vpad) { set_error("tp_cross_entropy: bad argument (M=%d V=%d Vpad=%d ld=%ld)", M, V, Vpad, (long)ld); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_cross_entropy: bad dtype %d", dtype); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int ch = dtype == TP_F32 ? 4 : 8;
    if (Vpad % ch == 0 && ld % ch == 0 && ((uintptr_t)logits & 15) == 0) {
        if (Vpad / ch <= 1024 * 8) {
            switch (dtype) {
            case TP_F32: cross_entropy_reg_kernel<float, 8><<<M, 1024, 0, s>>>((float*)logits, ld, target, loss, V, Vpad, grad_scale); break;
            case TP_F16: cross_entropy_reg_kernel<f16, 8><<<M, 1024, 0, s>>>((f16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
            default: cross_entropy_reg_kernel<bf16, 8><<<M, 1024, 0, s>>>((bf16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
            }
            return vocab_status("tp_cross_entropy");
        }
        if (dtype == TP_F32 && Vpad / ch <= 1024 * 16) {
            cross_entropy_reg_kernel<float, 16><<<M, 1024, 0, s>>>((float*)logits, ld, target, loss, V, Vpad, grad_scale);
            return vocab_status("tp_cross_entropy");
        }
        switch (dtype) {
        case TP_F32: cross_entropy_vec_kernel<float><<<M, 1024, 0, s>>>((float*)logits, ld, target, loss, V, Vpad, grad_scale); break;
        case TP_F16: cross_entropy_vec_kernel<f16><<<M, 1024, 0, s>>>((f16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
        default: cross_entropy_vec_kernel<bf16><<<M, 1024, 0, s>>>((bf16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
        }
        return vocab_status("tp_cross_entropy");
    }
    switch (dtype) {
    case TP_F32: cross_entropy_kernel<float><<<M, 1024, 0, s>>>((float*)logits, ld, target, loss, V, Vpad, grad_scale); break;
    case TP_F16: cross_entropy_kernel<f16><<<M, 1024, 0, s>>>((f16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
    default: cross_entropy_kernel<bf16><<<M, 1024, 0, s>>>((bf16*)logits, ld, target, loss, V, Vpad, grad_scale); break;
    }
    return vocab_status("tp_cross_entropy");
}

extern "C" int tp_scale_rows(void* x, int64_t ld, const float* scale, int M, int N, int dtype, void* stream) {
    using namespace tp;
    if (!x || !scale || M <= 0 || N <= 0 || ld < N) { set_error("tp_scale_rows: bad argument"); return TP_ERR_ARG; }
    if (dtype < TP_F32 || dtype > TP_BF16) { set_error("tp_scale_rows: bad dtype %d", dtype); return TP_ERR_ARG; }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int ch = dtype == TP_F32 ? 4 : 8;
    if (N % ch == 0 && ld % ch == 0 && ((uintptr_t)x & 15) == 0) {
        const int nch = N / ch;
        dim3 vgrid((nch + 255) / 256, M);
        switch (dtype) {
        case TP_F32: scale_rows_vec_kernel<float><<<vgrid, 256, 0, s>>>((float*)x, ld, scale, nch); break;
        case TP_F16: scale_rows_vec_kernel<f16><<<vgrid, 256, 0, s>>>((f16*)x, ld, scale, nch); break;
        default: scale_rows_vec_kernel<bf16><<<vgrid, 256, 0, s>>>((bf16*)x, ld, scale, nch); break;
        }
        return vocab_status("tp_scale_rows");
    }
    dim3 grid((N + 255) / 256, M);
    switch (dtype) {
    case TP_F32: scale_rows_kernel<float><<<grid, 256, 0, s>>>((float*)x, ld, scale, N); break;
    case TP_F16: scale_rows_kernel<f16><<<grid, 256, 0, s>>>((f16*)x, ld, scale, N); break;
    default: scale_rows_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)x, ld, scale, N); break;
    }
    return vocab_status("tp_scale_rows");
}
