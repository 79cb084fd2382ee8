// Mixed-precision Adam step over a list of tensors in one launch: the reference's update_weights
// (test_transformer_terapipe.py:245-266: copy the 16-bit gradients to fp32 and divide by the loss scale,
// FusedAdam on the fp32 master weights, zero the gradients, copy the master weights back to 16 bits) as one
// pass over memory.  HBM-bound: per parameter it reads gradient + master + two moments and writes
// master + two moments (+ the 16-bit weight, + the zeroed gradient).
#include "common.h"

namespace tp {

struct AdamArgs {
    const tp_adam_tensor* tensors;
    float lr, beta1, beta2, eps, weight_decay, grad_scale;
    float omb1, omb2;              // 1 - beta, rounded from the double difference
    float inv_bc1, inv_bc2;        // 1 / (1 - beta^step), or 1 without bias correction
    int adam_w_mode, zero_grad;
};

template <typename T> struct Vec4;
typedef float nt_f4 __attribute__((ext_vector_type(4)));
typedef unsigned nt_u2 __attribute__((ext_vector_type(2)));
template <> struct Vec4<float> { typedef nt_f4 type; };
template <> struct Vec4<f16> { typedef nt_u2 type; };
template <> struct Vec4<bf16> { typedef nt_u2 type; };

template <typename T> __device__ __forceinline__ void load4f(const T* p, float (&x)[4]) {
    const typename Vec4<T>::type raw = __builtin_nontemporal_load(reinterpret_cast<const typename Vec4<T>::type*>(p));
    const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = Elem<T>::to_float(e[i]);
}
template <typename T> __device__ __forceinline__ void store4f(T* p, const float (&x)[4]) {
    typename Vec4<T>::type raw;
    T* e = reinterpret_cast<T*>(&raw);
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = Elem<T>::from_float(x[i]);
    __builtin_nontemporal_store(raw, reinterpret_cast<typename Vec4<T>::type*>(p));
}

// One element of the update, in the order apex's multi_tensor_adam states it (csrc/multi_tensor_adam.cu of
// apex, the optimizer the reference constructs at test_transformer_terapipe.py:95):
//   L2 mode:     g += wd * p;  m, v updated;  p -= lr * (m/bc1) / (sqrt(v/bc2) + eps)
//   AdamW mode:                m, v updated;  p -= lr * ((m/bc1) / (sqrt(v/bc2) + eps) + wd * p)
__device__ __forceinline__ void adam_update(float& p, float& m, float& v, float g, const AdamArgs& a) {
    g *= a.grad_scale;
    if (!a.adam_w_mode) g += a.weight_decay * p;
    m = a.beta1 * m + a.omb1 * g;
    v = a.beta2 * v + a.omb2 * g * g;
    const float denom = sqrtf(v * a.inv_bc2) + a.eps;
    float update = (m * a.inv_bc1) / denom;
    if (a.adam_w_mode) update += a.weight_decay * p;
    p -= a.lr * update;
    // The 16-bit weight must be the ROUNDED fp32 master (model_param.copy_(master_param), :266).  Without this
    // barrier the compiler folds the last multiply-add and the conversion into v_fma_mixlo_f16, which rounds
    // the exact result once and differs from the two-step rounding in the last bit now and then.
    asm volatile("" : "+v"(p));
}

// grid = (blocks per tensor, tensors); each workgroup strides over its tensor in 4-element vectors
template <typename GT, typename MT, bool HAS_MODEL>
__global__ __launch_bounds__(256) void adam_kernel(AdamArgs a) {
    const tp_adam_tensor t = a.tensors[blockIdx.y];
    float* __restrict__ P = static_cast<float*>(t.master);
    float* __restrict__ M1 = static_cast<float*>(t.exp_avg);
    float* __restrict__ M2 = static_cast<float*>(t.exp_avg_sq);
    GT* __restrict__ G = static_cast<GT*>(t.grad);
    MT* __restrict__ W = static_cast<MT*>(t.model);
    const long n = t.n, n4 = n >> 2;
    const long stride = (long)gridDim.x * 256;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n4; i += stride) {
        const long o = i << 2;
        float p[4], m[4], v[4], g[4];
        load4f<float>(P + o, p);
        load4f<float>(M1 + o, m);
        load4f<float>(M2 + o, v);
        load4f<GT>(G + o, g);
#pragma unroll
        for (int k = 0; k < 4; ++k) adam_update(p[k], m[k], v[k], g[k], a);
        store4f<float>(P + o, p);
        store4f<float>(M1 + o, m);
        store4f<float>(M2 + o, v);
        if constexpr (HAS_MODEL) store4f<MT>(W + o, p);
        if (a.zero_grad) { const float z[4] = {0.f, 0.f, 0.f, 0.f}; store4f<GT>(G + o, z); }
    }
    // tail of a tensor whose length is not a multiple of 4
    if (blockIdx.x == 0 && threadIdx.x < (n & 3)) {
        const long o = (n4 << 2) + threadIdx.x;
        float p = P[o], m = M1[o], v = M2[o];
        adam_update(p, m, v, Elem<GT>::to_float(G[o]), a);
        P[o] = p; M1[o] = m; M2[o] = v;
        if constexpr (HAS_MODEL) W[o] = Elem<MT>::from_float(p);
        if (a.zero_grad) G[o] = Elem<GT>::from_float(0.f);
    }
}

template <typename GT>
static void launch_adam(const tp_adam_desc* d, const AdamArgs& a, dim3 grid, hipStream_t s) {
    switch (d->model_dtype) {
    case TP_F16: adam_kernel<GT, f16, true><<<grid, 256, 0, s>>>(a); break;
    case TP_BF16: adam_kernel<GT, bf16, true><<<grid, 256, 0, s>>>(a); break;
    default: adam_kernel<GT, float, false><<<grid, 256, 0, s>>>(a); break;
    }
}

}  // namespace tp

extern "C" int tp_adam_check_table(const tp_adam_tensor* t, int n_tensors, int model_dtype) {
    using namespace tp;
    if (!t || n_tensors <= 0) { set_error("tp_adam_check_table: bad argument"); return TP_ERR_ARG; }
    for (int i = 0; i < n_tensors; ++i) {
        if (!t[i].master || !t[i].grad || !t[i].exp_avg || !t[i].exp_avg_sq || (model_dtype != -1 && !t[i].model)) {
            set_error("tp_adam_check_table: tensor %d has a null pointer", i);
            return TP_ERR_ARG;
        }
        if (t[i].n <= 0) { set_error("tp_adam_check_table: tensor %d has length %ld", i, (long)t[i].n); return TP_ERR_ARG; }
        const uintptr_t bits = (uintptr_t)t[i].master | (uintptr_t)t[i].grad | (uintptr_t)t[i].exp_avg |
                               (uintptr_t)t[i].exp_avg_sq | (model_dtype != -1 ? (uintptr_t)t[i].model : 0);
        if (bits & 15) { set_error("tp_adam_check_table: tensor %d is not 16-byte aligned", i); return TP_ERR_UNSUPPORTED; }
    }
    return TP_OK;
}

extern "C" int tp_adam_step(const tp_adam_desc* d, void* stream) {
    using namespace tp;
    if (!d || !d->tensors || d->n_tensors <= 0) { set_error("tp_adam_step: bad argument"); return TP_ERR_ARG; }
    if (d->grad_dtype < TP_F32 || d->grad_dtype > TP_BF16) { set_error("tp_adam_step: bad grad_dtype %d", d->grad_dtype); return TP_ERR_ARG; }
    if (d->model_dtype != -1 && d->model_dtype != TP_F16 && d->model_dtype != TP_BF16) {
        set_error("tp_adam_step: model_dtype %d must be -1 (no 16-bit copy), TP_F16 or TP_BF16", d->model_dtype);
        return TP_ERR_ARG;
    }
    if (d->step < 1) { set_error("tp_adam_step: step %d must count from 1", d->step); return TP_ERR_ARG; }
    if (!(d->beta1 >= 0. && d->beta1 < 1. && d->beta2 >= 0. && d->beta2 < 1.) || !(d->eps >= 0.)) {
        set_error("tp_adam_step: betas must lie in [0, 1) and eps be non-negative");
        return TP_ERR_ARG;
    }
    if (d->n_tensors > 65535) { set_error("tp_adam_step: at most 65535 tensors per call (got %d)", d->n_tensors); return TP_ERR_UNSUPPORTED; }
    AdamArgs a;
    a.tensors = d->tensors;
    a.lr = (float)d->lr; a.beta1 = (float)d->beta1; a.beta2 = (float)d->beta2; a.eps = (float)d->eps;
    a.omb1 = (float)(1.0 - d->beta1); a.omb2 = (float)(1.0 - d->beta2);
    a.weight_decay = (float)d->weight_decay; a.grad_scale = (float)d->grad_scale;
    a.adam_w_mode = d->adam_w_mode; a.zero_grad = d->zero_grad;
    a.inv_bc1 = a.inv_bc2 = 1.f;
    if (d->bias_correction) {
        a.inv_bc1 = (float)(1.0 / (1.0 - pow(d->beta1, (double)d->step)));
        a.inv_bc2 = (float)(1.0 / (1.0 - pow(d->beta2, (double)d->step)));
    }
    const int bpt = d->blocks_per_tensor > 0 ? d->blocks_per_tensor : 256;
    dim3 grid(bpt, d->n_tensors);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (d->grad_dtype) {
    case TP_F32: launch_adam<float>(d, a, grid, s); break;
    case TP_F16: launch_adam<f16>(d, a, grid, s); break;
    default: launch_adam<bf16>(d, a, grid, s); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("tp_adam_step: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}
