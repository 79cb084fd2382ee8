// Pieces shared by the GEMM translation units: the kernel argument block and the per-row epilogue.
#pragma once
#include "common.h"

namespace tp {

struct GemmArgs {
    const void* A; const void* B; void* C;
    long lda, ldb, ldc;
    int M, N, K;
    int epi;
    const void* bias;
    const void* resid; long ldr;
    const void* aux; long ldaux;
    void* aux_out; long ldauxo;
    float* colsum;
    void* q; void* kc; void* vc;
    int batch, heads, hd, T, P;
    long cache_rows;
    long q_rows;     // rows per (batch, head) block of q
    float qscale;
    int kper;        // k extent handled by one split
    int nsplit;
    float* partial;  // [nsplit][M][N] fp32 when nsplit > 1
};

// v_mfma_f32_16x16x32: lane l feeds row / column (l & 15) with the 8 consecutive k values 8 * (l >> 4) .. + 7; the
// 16x16 fp32 result leaves column (l & 15), rows 4 * (l >> 4) + r in register r.
template <typename T> struct Mfma16x16x32;
template <> struct Mfma16x16x32<f16> {
    static __device__ __forceinline__ float4v run(uint4 a, uint4 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};
template <> struct Mfma16x16x32<bf16> {
    static __device__ __forceinline__ float4v run(uint4 a, uint4 b, float4v c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};

__device__ __forceinline__ float gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }
__device__ __forceinline__ float gelu_erf_grad(float z) {
    float cdf = 0.5f * (1.0f + erff(z * 0.70710678118654752f));
    float pdf = 0.3989422804014327f * __expf(-0.5f * z * z);
    return cdf + z * pdf;
}

// Applies the epilogue to 8 consecutive columns of one output row (col0 is a multiple of 8) and
// returns the values written in v (for the column sums).
template <typename T>
__device__ __forceinline__ void epilogue_vec8(const GemmArgs& a, int row, int col0, float* v) {
    typedef Elem<T> E;
    constexpr int CH = E::CH;          // elements per 16-byte access
    constexpr int NV = 8 / CH;         // 16-byte accesses per 8 columns
    auto ld8 = [&](const void* base, long off, float* out) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            uint4 raw = *reinterpret_cast<const uint4*>(reinterpret_cast<const T*>(base) + off + i * CH);
            const T* h = reinterpret_cast<const T*>(&raw);
#pragma unroll
            for (int e = 0; e < CH; ++e) out[i * CH + e] = E::to_float(h[e]);
        }
    };
    auto st8 = [&](void* base, long off, const float* in) {
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            uint4 raw;
            T* h = reinterpret_cast<T*>(&raw);
#pragma unroll
            for (int e = 0; e < CH; ++e) h[e] = E::from_float(in[i * CH + e]);
            *reinterpret_cast<uint4*>(reinterpret_cast<T*>(base) + off + i * CH) = raw;
        }
    };
    float t[8];
    const long co = (long)row * a.ldc + col0;
    switch (a.epi) {
    case TP_EPI_STORE:
        st8(a.C, co, v);
        break;
    case TP_EPI_ACCUMULATE:
        ld8(a.C, co, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] += v[e];
        st8(a.C, co, t);
        break;
    case TP_EPI_BIAS:
        ld8(a.bias, col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
        st8(a.C, co, v);
        break;
    case TP_EPI_BIAS_RELU:
        ld8(a.bias, col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[e] += t[e]; v[e] = v[e] > 0.f ? v[e] : 0.f; }
        st8(a.C, co, v);
        break;
    case TP_EPI_BIAS_GELU:
        ld8(a.bias, col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
        if (a.aux_out) st8(a.aux_out, (long)row * a.ldauxo + col0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = gelu_erf(v[e]);
        st8(a.C, co, v);
        break;
    case TP_EPI_BIAS_RESIDUAL:
        ld8(a.bias, col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
        ld8(a.resid, (long)row * a.ldr + col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
        st8(a.C, co, v);
        break;
    case TP_EPI_RELU_GRAD:
        ld8(a.aux, (long)row * a.ldaux + col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = t[e] > 0.f ? v[e] : 0.f;
        st8(a.C, co, v);
        break;
    case TP_EPI_GELU_GRAD:
        ld8(a.aux, (long)row * a.ldaux + col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] *= gelu_erf_grad(t[e]);
        st8(a.C, co, v);
        break;
    case TP_EPI_QKV_SCATTER: {
        ld8(a.bias, col0, t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
        const int hd3 = 3 * a.hd;
        const int head = col0 / hd3, w = col0 - head * hd3;
        const int part = w / a.hd, d = w - part * a.hd;
        const int tt = row / a.batch, b = row - tt * a.batch;
        const long bh = (long)b * a.heads + head;
        if (part == 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = v[e] * a.qscale;
            st8(a.q, (bh * a.q_rows + tt) * a.hd + d, t);
        } else {
            st8(part == 1 ? a.kc : a.vc, (bh * a.cache_rows + a.P + tt) * a.hd + d, v);
        }
        break;
    }
    }
}

// Compile-time loop: the body sees the index as a constant, so arrays indexed by it stay in registers even
// when the body is too large for the unroller's budget (a rolled loop over the accumulator blocks would put
// the whole accumulator array in scratch memory, main loop included).
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// The weight-streaming kernels of gemm_stream.hip (tile configurations 21 and up of the plan): launches `cfg` on
// `grid` = (column tiles, row tiles, k splits); false when cfg / op / dtype has no such kernel.
bool launch_gemm_stream(int cfg, int op, int dtype, dim3 grid, const GemmArgs& a, hipStream_t s);

}  // namespace tp
