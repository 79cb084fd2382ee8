// MFMA GEMMs (NT / NN / TN) with fused epilogues for the linears of the GPT layer at tensor-parallel
// size 1.  One templated kernel covers the three operand layouts and the three dtypes: an operand is
// either "k-major" (k contiguous in memory: fetched from LDS with ds_read_b128) or "mn-major"
// (k is the slow dimension: fetched with the gfx950 LDS transpose read), see common.h.
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
    float qscale;
    int kper;        // k extent handled by one split
    int nsplit;
    float* partial;  // [nsplit][M][N] fp32 when nsplit > 1
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
            st8(a.q, (bh * a.T + tt) * a.hd + d, t);
        } else {
            st8(part == 1 ? a.kc : a.vc, (bh * a.cache_rows + a.P + tt) * a.hd + d, v);
        }
        break;
    }
    }
}

template <typename T, bool AKM, bool BKM, int BM, int BN, int BK, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) void gemm_kernel(GemmArgs a) {
    typedef Elem<T> E;
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int AR = AKM ? BM : BK, AC = AKM ? BK : BM;
    constexpr int BR = BKM ? BN : BK, BC = BKM ? BK : BN;
    typedef TileLayout<T, AC> LA;
    typedef TileLayout<T, BC> LB;
    static_assert(BK % E::KSTEP == 0, "BK must be a multiple of the MFMA k");
    constexpr int SPITCH = 36;  // fp32 pitch of the per-wave 32x32 epilogue staging block
    constexpr int TILE_BYTES = 2 * (LA::size(AR) + LB::size(BR)) * (int)sizeof(T);
    constexpr int STAGE_BYTES = WM * WN * 32 * SPITCH * 4;
    constexpr int SMEM_BYTES = TILE_BYTES > STAGE_BYTES ? TILE_BYTES : STAGE_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    T* sA0 = reinterpret_cast<T*>(smem);
    T* sB0 = sA0 + 2 * LA::size(AR);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int kbeg = blockIdx.z * a.kper;
    const int kend = min(a.K, kbeg + a.kper);
    const T* A = reinterpret_cast<const T*>(a.A);
    const T* B = reinterpret_cast<const T*>(a.B);

    TileCopy<T, AR, AC, NT> ca;
    TileCopy<T, BR, BC, NT> cb;
    auto gload = [&](int k0) {
        if constexpr (AKM) ca.load(A, a.lda, m0, k0, a.M, kend, tid);
        else ca.load(A, a.lda, k0, m0, kend, a.M, tid);
        if constexpr (BKM) cb.load(B, a.ldb, n0, k0, a.N, kend, tid);
        else cb.load(B, a.ldb, k0, n0, kend, a.N, tid);
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int nk = (kend - kbeg + BK - 1) / BK;
    if (nk > 0) {
        gload(kbeg);
        ca.store(sA0, tid);
        cb.store(sB0, tid);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        if (kt + 1 < nk) gload(kbeg + (kt + 1) * BK);
        const T* tA = sA0 + cur * LA::size(AR);
        const T* tB = sB0 + cur * LB::size(BR);
#pragma unroll
        for (int ks = 0; ks < BK / E::KSTEP; ++ks) {
            typename E::opnd_t fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                int mb = (wm * TM + i) * 32;
                if constexpr (AKM) fa[i] = fetch_km<T, AC>(tA, mb + (lane & 31), ks * E::KSTEP, lane);
                else fa[i] = fetch_tr<T, AC, false>(tA, ks * E::KSTEP, mb, lane);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                int nb = (wn * TN + j) * 32;
                if constexpr (BKM) fb[j] = fetch_km<T, BC>(tB, nb + (lane & 31), ks * E::KSTEP, lane);
                else fb[j] = fetch_tr<T, BC, false>(tB, ks * E::KSTEP, nb, lane);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = E::mfma(fa[i], fb[j], acc[i][j]);
        }
        if (kt + 1 < nk) {
            ca.store(sA0 + (cur ^ 1) * LA::size(AR), tid);
            cb.store(sB0 + (cur ^ 1) * LB::size(BR), tid);
        }
        __syncthreads();
    }

    // Epilogue.  Each wave transposes one 32x32 accumulator block at a time through its own LDS
    // staging block so that a lane ends up with 8 consecutive columns of a row: 16-byte stores,
    // and a vector epilogue.  Lane -> (row = lane / 4 + 16 * pass, columns 8 * (lane % 4) .. + 7).
    float* stage = reinterpret_cast<float*>(smem) + wave * 32 * SPITCH;
    const int g = lane >> 5, li = lane & 31;
    const int er = lane >> 2, ec = (lane & 3) * 8;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col0 = n0 + (wn * TN + j) * 32 + ec;
        float csum[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) csum[e] = 0.f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) stage[acc_row(r, g) * SPITCH + li] = acc[i][j][r];
            // the block is private to the wave: LDS operations of one wave complete in order
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int rr = er + 16 * pass;
                const int row = m0 + (wm * TM + i) * 32 + rr;
                float v[8];
                float4 v0 = *reinterpret_cast<const float4*>(stage + rr * SPITCH + ec);
                float4 v1 = *reinterpret_cast<const float4*>(stage + rr * SPITCH + ec + 4);
                v[0] = v0.x; v[1] = v0.y; v[2] = v0.z; v[3] = v0.w;
                v[4] = v1.x; v[5] = v1.y; v[6] = v1.z; v[7] = v1.w;
                if (row < a.M && col0 < a.N) {
                    if (a.nsplit > 1) {
                        float* dst = a.partial + ((long)blockIdx.z * a.M + row) * a.N + col0;
                        *reinterpret_cast<float4*>(dst) = v0;
                        *reinterpret_cast<float4*>(dst + 4) = v1;
                    } else {
                        epilogue_vec8<T>(a, row, col0, v);
#pragma unroll
                        for (int e = 0; e < 8; ++e) csum[e] += v[e];
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        if (a.nsplit == 1 && a.colsum) {
            // lanes with equal (lane & 3) hold the same columns
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float s = csum[e];
                s += __shfl_xor(s, 4, 64);
                s += __shfl_xor(s, 8, 64);
                s += __shfl_xor(s, 16, 64);
                s += __shfl_xor(s, 32, 64);
                csum[e] = s;
            }
            if (lane < 4 && col0 < a.N) {
#pragma unroll
                for (int e = 0; e < 8; ++e) atomicAdd(a.colsum + col0 + e, csum[e]);
            }
        }
    }
}

// Sums the split-K partials and applies the epilogue.  One thread per 8 columns and rows_per_block
// rows per block, so the column sums cost 8 atomics per thread.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmArgs a, int rows_per_block) {
    const int col0 = (blockIdx.x * 256 + threadIdx.x) * 8;
    if (col0 >= a.N) return;
    const int r0 = blockIdx.y * rows_per_block;
    const int r1 = min(a.M, r0 + rows_per_block);
    float csum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) csum[e] = 0.f;
    for (int row = r0; row < r1; ++row) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
        for (int z = 0; z < a.nsplit; ++z) {
            const float* src = a.partial + ((long)z * a.M + row) * a.N + col0;
            float4 p0 = *reinterpret_cast<const float4*>(src);
            float4 p1 = *reinterpret_cast<const float4*>(src + 4);
            v[0] += p0.x; v[1] += p0.y; v[2] += p0.z; v[3] += p0.w;
            v[4] += p1.x; v[5] += p1.y; v[6] += p1.z; v[7] += p1.w;
        }
        epilogue_vec8<T>(a, row, col0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) csum[e] += v[e];
    }
    if (a.colsum) {
#pragma unroll
        for (int e = 0; e < 8; ++e) atomicAdd(a.colsum + col0 + e, csum[e]);
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static constexpr int kNumCU = 256;  // MI355X

struct GemmPlan {
    int cfg;      // 0: 128x128 tile, 1: 64x64 tile
    int nsplit;
    int kper;
    int gx, gy;
};

static GemmPlan plan_gemm(const tp_gemm_desc* d) {
    GemmPlan p;
    const int bk = (d->dtype == TP_F32) ? 16 : 64;  // k granularity shared by both tile configs
    long t128 = (long)((d->M + 127) / 128) * ((d->N + 127) / 128);
    long t64 = (long)((d->M + 63) / 64) * ((d->N + 63) / 64);
    if (d->dtype != TP_F32 && t128 >= kNumCU) {
        p.cfg = 0;
        p.gx = (d->N + 127) / 128; p.gy = (d->M + 127) / 128;
    } else {
        p.cfg = 1;
        p.gx = (d->N + 63) / 64; p.gy = (d->M + 63) / 64;
    }
    long tiles = (long)p.gx * p.gy;
    int nsplit = 1;
    // split K until about two workgroups per CU exist, keeping at least 4 k-tiles per split;
    // read-modify-write and scatter epilogues run in the reduce kernel just the same.
    if (tiles < 2 * kNumCU) {
        long want = (2 * kNumCU + tiles - 1) / tiles;
        long kt = (d->K + bk - 1) / bk;
        long maxs = kt / 4 > 0 ? kt / 4 : 1;
        nsplit = (int)(want < maxs ? want : maxs);
        if (nsplit > 16) nsplit = 16;
        if (nsplit < 1) nsplit = 1;
    }
    (void)t64;
    long kt = (d->K + bk - 1) / bk;
    long per = (kt + nsplit - 1) / nsplit;
    p.kper = (int)(per * bk);
    p.nsplit = (int)((d->K + p.kper - 1) / p.kper);
    if (p.nsplit < 1) { p.nsplit = 1; p.kper = bk; }
    return p;
}

template <typename T, bool AKM, bool BKM>
static void launch_cfg(const GemmPlan& p, const GemmArgs& a, hipStream_t s) {
    dim3 grid(p.gx, p.gy, p.nsplit);
    if constexpr (sizeof(T) == 4) {
        gemm_kernel<T, AKM, BKM, 64, 64, 16, 2, 2><<<grid, 256, 0, s>>>(a);
    } else {
        if (p.cfg == 0) gemm_kernel<T, AKM, BKM, 128, 128, 32, 2, 2><<<grid, 256, 0, s>>>(a);
        else gemm_kernel<T, AKM, BKM, 64, 64, 64, 2, 2><<<grid, 256, 0, s>>>(a);
    }
}

template <typename T>
static void launch_gemm(const tp_gemm_desc* d, const GemmPlan& p, const GemmArgs& a, hipStream_t s) {
    switch (d->op) {
    case TP_GEMM_NT: launch_cfg<T, true, true>(p, a, s); break;
    case TP_GEMM_NN: launch_cfg<T, true, false>(p, a, s); break;
    default: launch_cfg<T, false, false>(p, a, s); break;
    }
    if (p.nsplit > 1) {
        int rpb = 8;
        dim3 grid((d->N / 8 + 255) / 256, (d->M + rpb - 1) / rpb);
        gemm_splitk_reduce_kernel<T><<<grid, 256, 0, s>>>(a, rpb);
    }
}

static int validate_gemm(const tp_gemm_desc* d) {
    if (!d) { set_error("tp_gemm: null descriptor"); return TP_ERR_ARG; }
    if (d->dtype < TP_F32 || d->dtype > TP_BF16) { set_error("tp_gemm: bad dtype %d", d->dtype); return TP_ERR_ARG; }
    if (d->op < TP_GEMM_NT || d->op > TP_GEMM_TN) { set_error("tp_gemm: bad op %d", d->op); return TP_ERR_ARG; }
    if (d->epilogue < TP_EPI_STORE || d->epilogue > TP_EPI_GELU_GRAD) { set_error("tp_gemm: bad epilogue %d", d->epilogue); return TP_ERR_ARG; }
    if (d->M <= 0 || d->N <= 0 || d->K <= 0) { set_error("tp_gemm: non-positive shape M=%d N=%d K=%d", d->M, d->N, d->K); return TP_ERR_ARG; }
    if (!d->A || !d->B) { set_error("tp_gemm: null operand"); return TP_ERR_ARG; }
    const int ch = d->dtype == TP_F32 ? 4 : 8;
    // contiguous extents of the operands as stored
    int a_cols = d->op == TP_GEMM_TN ? d->M : d->K;
    int b_cols = d->op == TP_GEMM_NT ? d->K : d->N;
    if (a_cols % ch || b_cols % ch || d->lda % ch || d->ldb % ch) {
        set_error("tp_gemm: contiguous extents / leading dimensions must be multiples of %d elements "
                  "(A cols %d lda %ld, B cols %d ldb %ld)", ch, a_cols, (long)d->lda, b_cols, (long)d->ldb);
        return TP_ERR_UNSUPPORTED;
    }
    if (d->lda < a_cols || d->ldb < b_cols) { set_error("tp_gemm: leading dimension smaller than row"); return TP_ERR_ARG; }
    if (((uintptr_t)d->A | (uintptr_t)d->B) & 15) { set_error("tp_gemm: operands must be 16-byte aligned"); return TP_ERR_ARG; }
    if (d->N % 8) { set_error("tp_gemm: N=%d must be a multiple of 8", d->N); return TP_ERR_UNSUPPORTED; }
    if (d->epilogue != TP_EPI_QKV_SCATTER) {
        if (!d->C || d->ldc < d->N || d->ldc % ch || ((uintptr_t)d->C & 15)) { set_error("tp_gemm: bad C / ldc / alignment"); return TP_ERR_ARG; }
    }
    if (((uintptr_t)d->bias | (uintptr_t)d->residual | (uintptr_t)d->aux | (uintptr_t)d->aux_out |
         (uintptr_t)d->q | (uintptr_t)d->k_cache | (uintptr_t)d->v_cache) & 15) {
        set_error("tp_gemm: epilogue tensors must be 16-byte aligned"); return TP_ERR_ARG;
    }
    if ((d->residual && d->ldr % ch) || (d->aux && d->ldaux % ch) || (d->aux_out && d->ldauxo % ch)) {
        set_error("tp_gemm: epilogue leading dimensions must be multiples of %d", ch); return TP_ERR_ARG;
    }
    switch (d->epilogue) {
    case TP_EPI_BIAS: case TP_EPI_BIAS_RELU: case TP_EPI_BIAS_GELU:
        if (!d->bias) { set_error("tp_gemm: epilogue needs bias"); return TP_ERR_ARG; }
        break;
    case TP_EPI_BIAS_RESIDUAL:
        if (!d->bias || !d->residual || d->ldr < d->N) { set_error("tp_gemm: epilogue needs bias and residual"); return TP_ERR_ARG; }
        break;
    case TP_EPI_RELU_GRAD: case TP_EPI_GELU_GRAD:
        if (!d->aux || d->ldaux < d->N) { set_error("tp_gemm: epilogue needs aux"); return TP_ERR_ARG; }
        break;
    case TP_EPI_QKV_SCATTER:
        if (!d->bias || !d->q || !d->k_cache || !d->v_cache) { set_error("tp_gemm: qkv scatter needs bias, q, k_cache, v_cache"); return TP_ERR_ARG; }
        if (d->batch <= 0 || d->heads <= 0 || d->head_dim <= 0 || d->head_dim % 8 || d->cache_len < 0) { set_error("tp_gemm: bad qkv geometry"); return TP_ERR_ARG; }
        if (d->N != 3 * d->heads * d->head_dim) { set_error("tp_gemm: qkv scatter needs N == 3*heads*head_dim (N=%d)", d->N); return TP_ERR_ARG; }
        if (d->M % d->batch) { set_error("tp_gemm: qkv scatter needs M %% batch == 0"); return TP_ERR_ARG; }
        if ((long)d->cache_len + d->M / d->batch > d->cache_rows) {
            set_error("tp_gemm: slice [%d, %d) does not fit a cache of %ld rows", d->cache_len,
                      d->cache_len + d->M / d->batch, (long)d->cache_rows);
            return TP_ERR_ARG;
        }
        break;
    default: break;
    }
    return TP_OK;
}

}  // namespace tp

extern "C" size_t tp_gemm_workspace_bytes(const tp_gemm_desc* d) {
    if (tp::validate_gemm(d) != TP_OK) return 0;
    tp::GemmPlan p = tp::plan_gemm(d);
    return p.nsplit > 1 ? (size_t)p.nsplit * d->M * d->N * sizeof(float) : 0;
}

extern "C" int tp_gemm(const tp_gemm_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = tp::validate_gemm(d);
    if (rc != TP_OK) return rc;
    tp::GemmPlan p = tp::plan_gemm(d);
    size_t need = p.nsplit > 1 ? (size_t)p.nsplit * d->M * d->N * sizeof(float) : 0;
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        tp::set_error("tp_gemm: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        return TP_ERR_WORKSPACE;
    }
    tp::GemmArgs a;
    a.A = d->A; a.B = d->B; a.C = d->C;
    a.lda = d->lda; a.ldb = d->ldb; a.ldc = d->ldc;
    a.M = d->M; a.N = d->N; a.K = d->K;
    a.epi = d->epilogue;
    a.bias = d->bias; a.resid = d->residual; a.ldr = d->ldr;
    a.aux = d->aux; a.ldaux = d->ldaux; a.aux_out = d->aux_out; a.ldauxo = d->ldauxo;
    a.colsum = d->colsum_acc;
    a.q = d->q; a.kc = d->k_cache; a.vc = d->v_cache;
    a.batch = d->batch; a.heads = d->heads; a.hd = d->head_dim;
    a.T = d->epilogue == TP_EPI_QKV_SCATTER ? d->M / d->batch : 0;
    a.P = d->cache_len; a.cache_rows = d->cache_rows; a.qscale = d->q_scale;
    a.kper = p.kper; a.nsplit = p.nsplit; a.partial = reinterpret_cast<float*>(workspace);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (d->dtype) {
    case TP_F32: tp::launch_gemm<float>(d, p, a, s); break;
    case TP_F16: tp::launch_gemm<tp::f16>(d, p, a, s); break;
    default: tp::launch_gemm<tp::bf16>(d, p, a, s); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { tp::set_error("tp_gemm: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}
