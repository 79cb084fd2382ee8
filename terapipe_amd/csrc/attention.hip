// Prefix-cached causal attention for one sequence slice: forward (online softmax, optional split over
// the key range) and backward (recompute from Q, K, LSE; dK/dV accumulated into the gradient caches).
//
// Register layouts.  All products are 32x32 MFMA blocks.  The forward and the dQ kernel compute the
// TRANSPOSED score block S^T = K Q^T, so a lane owns one query (column lane & 31) and 16 keys: the
// softmax row reductions are in-lane plus one exchange with lane ^ 32, and eight accumulator registers
// are, unshuffled, the operand of the following product (P^T or dS^T) once V^T / K^T are fetched from
// LDS in the interleaved row order (fetch_tr<..., true>).  The dK/dV kernel computes S = Q K^T so that a
// lane owns one key and 16 queries, which makes P and dS the operands of dV^T = dO^T P and
// dK^T = Q^T dS in the same way.
#include "common.h"

namespace tp {

struct AttnArgs {
    const void* q; const void* kc; const void* vc; void* o; float* lse;
    const void* d_o; float* delta; void* dqkv; void* gk; void* gv;
    int B, H, T, P;
    long cache_rows;
    int nsplit;
    float* part_o; float* part_lse;
    int accumulate_prefix, has_incoming, zero_slice_rows;
    int dq_only;
    float qscale;
    long q_bhs;      // elements between consecutive (batch, head) blocks of q
    long st_bhs;     // floats between consecutive (batch, head) blocks of lse / delta
};

static constexpr float kLog2e = 1.4426950408889634f;

// v_exp_f32: 2^x at hardware precision (about 1 ulp), results below the normal range flush to zero
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <typename T, int DH>
__device__ __forceinline__ void load_row_operands(typename Elem<T>::opnd_t* reg, const T* rowptr, bool valid, int g) {
    typedef Elem<T> E;
    constexpr int NKS = DH / E::KSTEP;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
        if constexpr (sizeof(T) == 2) {
            reg[ks] = valid ? *reinterpret_cast<const uint4*>(rowptr + ks * 16 + 8 * g) : make_uint4(0, 0, 0, 0);
        } else {
            reg[ks] = valid ? rowptr[ks * 2 + g] : 0.f;
        }
    }
}

// acc[db] += X^T-block (rows db*32.. of the tile's columns, k over tile rows krow_base..+31) times the
// 32x32 accumulator `p` used as the k x n operand.
template <typename T, int DH>
__device__ __forceinline__ void mfma_acc_as_b(float16v* acc, const T* tile, int krow_base, const float16v& p, int lane) {
    typedef Elem<T> E;
    typedef TileLayout<T, DH> L;
    constexpr int NDB = DH / 32;
    const int g = lane >> 5, li = lane & 31;
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            float tmp[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) tmp[e] = p[8 * s + e];
            uint4 bop = pack8<T>(tmp);
            uint4 aop[NDB];
#pragma unroll
            for (int db = 0; db < NDB; ++db) aop[db] = fetch_tr<T, DH, true>(tile, krow_base + 16 * s, db * 32, lane);
            __builtin_amdgcn_sched_barrier(0);   // all fetches in flight before the first MFMA
#pragma unroll
            for (int db = 0; db < NDB; ++db) acc[db] = E::mfma(aop[db], bop, acc[db]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            float bop = p[j];
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                float aop = tile[L::off(krow_base + acc_row(j, g), db * 32 + li)];
                acc[db] = E::mfma(aop, bop, acc[db]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// forward
// ------------------------------------------------------------------------------------------------
template <typename T, int DH, int NW, int BN>
__global__ __launch_bounds__(NW * 64) void attn_fwd_kernel(AttnArgs a) {
    typedef Elem<T> E;
    constexpr int DP = (DH + 31) / 32 * 32;   // LDS tiles and accumulators are padded to whole 32-column blocks
    typedef TileLayout<T, DP> L;
    constexpr int NT = NW * 64, NKB = BN / 32, NDB = DP / 32, NKS = DH / E::KSTEP;
    __shared__ __attribute__((aligned(16))) T sK[L::size(BN)];
    __shared__ __attribute__((aligned(16))) T sV[L::size(BN)];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, li = lane & 31;
    const int bh = blockIdx.y, b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const int q0w = (blockIdx.x * NW + wave) * 32;
    const int tq = q0w + li;
    const int q_wg_end = min(T_, (int)(blockIdx.x + 1) * NW * 32);
    const int kv_end = P + q_wg_end;
    const int ntiles = (kv_end + BN - 1) / BN;
    const int tps = (ntiles + a.nsplit - 1) / a.nsplit;
    const int t_beg = blockIdx.z * tps, t_end = min(ntiles, t_beg + tps);

    typename E::opnd_t qreg[NKS];
    load_row_operands<T, DH>(qreg, reinterpret_cast<const T*>(a.q) + ((long)bh * a.q_bhs + (long)tq * DH), tq < T_, g);

    float16v oacc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;

    const T* Kb = reinterpret_cast<const T*>(a.kc) + (long)bh * a.cache_rows * DH;
    const T* Vb = reinterpret_cast<const T*>(a.vc) + (long)bh * a.cache_rows * DH;
    TileCopy<T, BN, DP, NT> ck, cv;
    if (t_beg < t_end) {
        ck.load(Kb, DH, t_beg * BN, 0, S, DH, tid);
        cv.load(Vb, DH, t_beg * BN, 0, S, DH, tid);
        ck.store(sK, tid);
        cv.store(sV, tid);
    }
    __syncthreads();
    for (int t = t_beg; t < t_end; ++t) {
        if (t + 1 < t_end) {
            ck.load(Kb, DH, (t + 1) * BN, 0, S, DH, tid);
            cv.load(Vb, DH, (t + 1) * BN, 0, S, DH, tid);
        }
        const int key0 = t * BN;
        if (q0w < T_ && key0 <= P + q0w + 31) {
            float16v sacc[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    typename E::opnd_t kop = fetch_km<T, DP>(sK, kb * 32 + li, ks * E::KSTEP, lane);
                    sacc[kb] = E::mfma(kop, qreg[ks], sacc[kb]);
                }
            }
            float mt = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    int key = key0 + kb * 32 + acc_row(j, g);
                    float s = key > P + tq ? -INFINITY : sacc[kb][j];
                    sacc[kb][j] = s;
                    mt = fmaxf(mt, s);
                }
            mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float m_new = fmaxf(m, mt);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = exp2f((m - m_safe) * kLog2e);
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    float p = exp2f((sacc[kb][j] - m_safe) * kLog2e);
                    sacc[kb][j] = p;
                    psum += p;
                }
            lsum = lsum * alpha + psum;
            m = m_new;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) mfma_acc_as_b<T, DP>(oacc, sV, kb * 32, sacc[kb], lane);
        }
        __syncthreads();
        if (t + 1 < t_end) {
            ck.store(sK, tid);
            cv.store(sV, tid);
        }
        __syncthreads();
    }

    const float ltot = lsum + __shfl_xor(lsum, 32, 64);
    if (tq < T_) {
        const float inv = ltot > 0.f ? 1.0f / ltot : 0.f;
        const float lse = ltot > 0.f ? m + logf(ltot) : -INFINITY;
        if (a.nsplit == 1) {
            T* O = reinterpret_cast<T*>(a.o) + ((long)tq * a.B + b) * ((long)a.H * DH) + (long)h * DH;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    int dh = db * 32 + 8 * jq + 4 * g;
                    if (DP != DH && dh >= DH) continue;
                    store4<T>(O + dh, oacc[db][4 * jq] * inv, oacc[db][4 * jq + 1] * inv,
                              oacc[db][4 * jq + 2] * inv, oacc[db][4 * jq + 3] * inv);
                }
            if (g == 0) a.lse[(long)bh * a.st_bhs + tq] = lse;
        } else {
            const long BH = (long)a.B * a.H;
            float* PO = a.part_o + (((long)blockIdx.z * BH + bh) * T_ + tq) * DH;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    int dh = db * 32 + 8 * jq + 4 * g;
                    if (DP != DH && dh >= DH) continue;
                    *reinterpret_cast<float4*>(PO + dh) =
                        make_float4(oacc[db][4 * jq] * inv, oacc[db][4 * jq + 1] * inv,
                                    oacc[db][4 * jq + 2] * inv, oacc[db][4 * jq + 3] * inv);
                }
            if (g == 0) a.part_lse[((long)blockIdx.z * BH + bh) * T_ + tq] = lse;
        }
    }
}

// merges the per-split partial outputs: one wave per (bh, t) row
template <typename T, int DH>
__global__ __launch_bounds__(256) void attn_fwd_merge_kernel(AttnArgs a) {
    const long BH = (long)a.B * a.H;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= BH * a.T) return;
    const int bh = (int)(row / a.T), t = (int)(row - (long)bh * a.T);
    const int b = bh / a.H, h = bh - b * a.H;
    float mx = -INFINITY;
    for (int z = 0; z < a.nsplit; ++z) mx = fmaxf(mx, a.part_lse[(long)z * BH * a.T + row]);
    float wsum = 0.f;
    constexpr int NC = (DH + 63) / 64;
    float acc[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) acc[i] = 0.f;
    for (int z = 0; z < a.nsplit; ++z) {
        float l = a.part_lse[(long)z * BH * a.T + row];
        float w = l == -INFINITY ? 0.f : exp2f((l - mx) * kLog2e);
        wsum += w;
        const float* PO = a.part_o + ((long)z * BH * a.T + row) * DH;
#pragma unroll
        for (int i = 0; i < NC; ++i)
            if (DH % 64 == 0 || lane + 64 * i < DH) acc[i] += w * PO[lane + 64 * i];
    }
    T* O = reinterpret_cast<T*>(a.o) + ((long)t * a.B + b) * ((long)a.H * DH) + (long)h * DH;
    const float inv = 1.0f / wsum;
#pragma unroll
    for (int i = 0; i < NC; ++i)
        if (DH % 64 == 0 || lane + 64 * i < DH) O[lane + 64 * i] = Elem<T>::from_float(acc[i] * inv);
    if (lane == 0) a.lse[(long)bh * a.st_bhs + t] = mx + logf(wsum);
}

// ------------------------------------------------------------------------------------------------
// backward
// ------------------------------------------------------------------------------------------------
// delta[bh][t] = sum_d dO * O, one wave per (t, b, h)
template <typename T, int DH>
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(AttnArgs a) {
    const long n = (long)a.T * a.B * a.H;
    const long idx = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (idx >= n) return;
    const int h = (int)(idx % a.H);
    const long m = idx / a.H;  // row t*B + b
    const int b = (int)(m % a.B), t = (int)(m / a.B);
    const long off = m * ((long)a.H * DH) + (long)h * DH;
    const T* O = reinterpret_cast<const T*>(a.o) + off;
    const T* dO = reinterpret_cast<const T*>(a.d_o) + off;
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < (DH + 63) / 64; ++i)
        if (DH % 64 == 0 || lane + 64 * i < DH)
            s += Elem<T>::to_float(O[lane + 64 * i]) * Elem<T>::to_float(dO[lane + 64 * i]);
    s = wave_sum(s);
    if (lane == 0) a.delta[((long)b * a.H + h) * a.st_bhs + t] = s;
}

// dK / dV: each wave owns 32 keys and walks over the query blocks that can see them.
template <typename T, typename GT, int DH, int NW>
__global__ __launch_bounds__(NW * 64) void attn_bwd_dkdv_kernel(AttnArgs a) {
    typedef Elem<T> E;
    constexpr int DP = (DH + 31) / 32 * 32;
    typedef TileLayout<T, DP> L;
    constexpr int NT = NW * 64, NDB = DP / 32, NKS = DH / E::KSTEP;
    __shared__ __attribute__((aligned(16))) T sQ[L::size(32)];
    __shared__ __attribute__((aligned(16))) T sdO[L::size(32)];
    __shared__ __attribute__((aligned(16))) float sLse[32];
    __shared__ __attribute__((aligned(16))) float sDelta[32];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, li = lane & 31;
    const int bh = blockIdx.y, b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int key0wg = blockIdx.x * NW * 32;
    const int key0w = key0wg + wave * 32;
    const int key = key0w + li;

    typename E::opnd_t kreg[NKS], vreg[NKS];
    load_row_operands<T, DH>(kreg, reinterpret_cast<const T*>(a.kc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);
    load_row_operands<T, DH>(vreg, reinterpret_cast<const T*>(a.vc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);

    float16v dk[NDB], dv[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[db][r] = 0.f; dv[db][r] = 0.f; }

    const T* Qb = reinterpret_cast<const T*>(a.q) + (long)bh * a.q_bhs;
    const T* dOb = reinterpret_cast<const T*>(a.d_o) + (long)b * EE + (long)h * DH;  // row t at stride B*E
    const int nqb = (T_ + 31) / 32;
    const int qb_start = key0wg > P ? (key0wg - P) / 32 : 0;
    TileCopy<T, 32, DP, NT> cq, cdo;
    for (int qb = qb_start; qb < nqb; ++qb) {
        cq.load(Qb, DH, qb * 32, 0, T_, DH, tid);
        cdo.load(dOb, (long)a.B * EE, qb * 32, 0, T_, DH, tid);
        __syncthreads();  // previous iteration's readers are done
        cq.store(sQ, tid);
        cdo.store(sdO, tid);
        if (tid < 32) {
            int t = qb * 32 + tid;
            sLse[tid] = t < T_ ? a.lse[(long)bh * a.st_bhs + t] : 0.f;
            sDelta[tid] = t < T_ ? a.delta[(long)bh * a.st_bhs + t] : 0.f;
        }
        __syncthreads();
        if (key0w < S && key0w <= P + qb * 32 + 31) {
            float16v sacc, pacc;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                typename E::opnd_t qop = fetch_km<T, DP>(sQ, li, ks * E::KSTEP, lane);
                sacc = E::mfma(qop, kreg[ks], sacc);
                typename E::opnd_t doop = fetch_km<T, DP>(sdO, li, ks * E::KSTEP, lane);
                pacc = E::mfma(doop, vreg[ks], pacc);
            }
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                float4 l4 = *reinterpret_cast<const float4*>(sLse + 8 * jq + 4 * g);
                float4 d4 = *reinterpret_cast<const float4*>(sDelta + 8 * jq + 4 * g);
                const float lv[4] = {l4.x, l4.y, l4.z, l4.w};
                const float dl[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    int j = 4 * jq + e;
                    int t = qb * 32 + 8 * jq + 4 * g + e;
                    bool vis = (t < T_) && (key <= P + t) && (key < S);
                    float p = vis ? exp2f((sacc[j] - lv[e]) * kLog2e) : 0.f;
                    float ds = p * (pacc[j] - dl[e]);
                    sacc[j] = p;
                    pacc[j] = ds;
                }
            }
            mfma_acc_as_b<T, DP>(dv, sdO, 0, sacc, lane);
            mfma_acc_as_b<T, DP>(dk, sQ, 0, pacc, lane);
        }
    }

    if (key < S) {
        GT* gK = reinterpret_cast<GT*>(a.gk) + ((long)bh * a.cache_rows + key) * DH;
        GT* gV = reinterpret_cast<GT*>(a.gv) + ((long)bh * a.cache_rows + key) * DH;
        if (key < P) {
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    int dh = db * 32 + 8 * jq + 4 * g;
                    if (DP != DH && dh >= DH) continue;
                    float ok[4] = {0.f, 0.f, 0.f, 0.f}, ov[4] = {0.f, 0.f, 0.f, 0.f};
                    if (a.accumulate_prefix) { load4<GT>(gK + dh, ok); load4<GT>(gV + dh, ov); }
                    store4<GT>(gK + dh, ok[0] + dk[db][4 * jq], ok[1] + dk[db][4 * jq + 1],
                               ok[2] + dk[db][4 * jq + 2], ok[3] + dk[db][4 * jq + 3]);
                    store4<GT>(gV + dh, ov[0] + dv[db][4 * jq], ov[1] + dv[db][4 * jq + 1],
                               ov[2] + dv[db][4 * jq + 2], ov[3] + dv[db][4 * jq + 3]);
                }
        } else {
            const int t = key - P;
            T* dst = reinterpret_cast<T*>(a.dqkv) + ((long)t * a.B + b) * (3 * EE) + (long)h * 3 * DH;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    int dh = db * 32 + 8 * jq + 4 * g;
                    if (DP != DH && dh >= DH) continue;
                    float ok[4] = {0.f, 0.f, 0.f, 0.f}, ov[4] = {0.f, 0.f, 0.f, 0.f};
                    if (a.has_incoming) { load4<GT>(gK + dh, ok); load4<GT>(gV + dh, ov); }
                    store4<T>(dst + DH + dh, ok[0] + dk[db][4 * jq], ok[1] + dk[db][4 * jq + 1],
                              ok[2] + dk[db][4 * jq + 2], ok[3] + dk[db][4 * jq + 3]);
                    store4<T>(dst + 2 * DH + dh, ov[0] + dv[db][4 * jq], ov[1] + dv[db][4 * jq + 1],
                              ov[2] + dv[db][4 * jq + 2], ov[3] + dv[db][4 * jq + 3]);
                    if (a.zero_slice_rows) {
                        store4<GT>(gK + dh, 0.f, 0.f, 0.f, 0.f);
                        store4<GT>(gV + dh, 0.f, 0.f, 0.f, 0.f);
                    }
                }
        }
    }
}

// dQ: each wave owns 32 queries and walks over the key tiles they can see.
template <typename T, int DH, int NW, int BN>
__global__ __launch_bounds__(NW * 64) void attn_bwd_dq_kernel(AttnArgs a) {
    typedef Elem<T> E;
    constexpr int DP = (DH + 31) / 32 * 32;   // LDS tiles and accumulators are padded to whole 32-column blocks
    typedef TileLayout<T, DP> L;
    constexpr int NT = NW * 64, NKB = BN / 32, NDB = DP / 32, NKS = DH / E::KSTEP;
    __shared__ __attribute__((aligned(16))) T sK[L::size(BN)];
    __shared__ __attribute__((aligned(16))) T sV[L::size(BN)];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, li = lane & 31;
    const int bh = blockIdx.y, b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int q0w = (blockIdx.x * NW + wave) * 32;
    const int tq = q0w + li;
    const int q_wg_end = min(T_, (int)(blockIdx.x + 1) * NW * 32);
    const int kv_end = P + q_wg_end;
    const int ntiles = (kv_end + BN - 1) / BN;

    typename E::opnd_t qreg[NKS], doreg[NKS];
    load_row_operands<T, DH>(qreg, reinterpret_cast<const T*>(a.q) + ((long)bh * a.q_bhs + (long)tq * DH), tq < T_, g);
    load_row_operands<T, DH>(doreg, reinterpret_cast<const T*>(a.d_o) + ((long)tq * a.B + b) * EE + (long)h * DH, tq < T_, g);
    const float lse_q = tq < T_ ? a.lse[(long)bh * a.st_bhs + tq] : 0.f;
    const float delta_q = tq < T_ ? a.delta[(long)bh * a.st_bhs + tq] : 0.f;

    float16v dq[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[db][r] = 0.f;

    const T* Kb = reinterpret_cast<const T*>(a.kc) + (long)bh * a.cache_rows * DH;
    const T* Vb = reinterpret_cast<const T*>(a.vc) + (long)bh * a.cache_rows * DH;
    TileCopy<T, BN, DP, NT> ck, cv;
    if (ntiles > 0) {
        ck.load(Kb, DH, 0, 0, S, DH, tid);
        cv.load(Vb, DH, 0, 0, S, DH, tid);
        ck.store(sK, tid);
        cv.store(sV, tid);
    }
    __syncthreads();
    for (int t = 0; t < ntiles; ++t) {
        if (t + 1 < ntiles) {
            ck.load(Kb, DH, (t + 1) * BN, 0, S, DH, tid);
            cv.load(Vb, DH, (t + 1) * BN, 0, S, DH, tid);
        }
        const int key0 = t * BN;
        if (q0w < T_ && key0 <= P + q0w + 31) {
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
                float16v sacc, pacc;
#pragma unroll
                for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    typename E::opnd_t kop = fetch_km<T, DP>(sK, kb * 32 + li, ks * E::KSTEP, lane);
                    sacc = E::mfma(kop, qreg[ks], sacc);
                    typename E::opnd_t vop = fetch_km<T, DP>(sV, kb * 32 + li, ks * E::KSTEP, lane);
                    pacc = E::mfma(vop, doreg[ks], pacc);
                }
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    int key = key0 + kb * 32 + acc_row(j, g);
                    float p = key > P + tq ? 0.f : exp2f((sacc[j] - lse_q) * kLog2e);
                    pacc[j] = p * (pacc[j] - delta_q);
                }
                mfma_acc_as_b<T, DP>(dq, sK, kb * 32, pacc, lane);
            }
        }
        __syncthreads();
        if (t + 1 < ntiles) {
            ck.store(sK, tid);
            cv.store(sV, tid);
        }
        __syncthreads();
    }
    if (tq < T_) {
        T* dst = reinterpret_cast<T*>(a.dqkv) + ((long)tq * a.B + b) * (3 * EE) + (long)h * 3 * DH;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                int dh = db * 32 + 8 * jq + 4 * g;
                if (DP != DH && dh >= DH) continue;
                store4<T>(dst + dh, dq[db][4 * jq] * a.qscale, dq[db][4 * jq + 1] * a.qscale,
                          dq[db][4 * jq + 2] * a.qscale, dq[db][4 * jq + 3] * a.qscale);
            }
    }
}

// ------------------------------------------------------------------------------------------------
// 16-bit kernels: direct global->LDS tile loads, per-wave rings, 32 x 32 MFMA blocks
// ------------------------------------------------------------------------------------------------
// the gradient-cache dK/dV kernel stages the lse / delta vectors of the whole slice in LDS once (T <= kMaxTLds)
static constexpr int kMaxTLds = 4096;

// Workgroups are dealt to the eight XCDs round-robin by linear id.  This maps the linear id to
// (batch*head, block) so that all blocks of one (batch, head) run on the same XCD and its K / V / Q / dO
// rows are fetched into one L2 only.  Launch with xcd_grid(BH, nblocks) workgroups; false = no work.
__device__ __forceinline__ bool xcd_map(int BH, int& bh, int& blk, int id = blockIdx.x) {
    const int xcd = id & 7, slot = id >> 3;
    const int nbh8 = (BH + 7) >> 3;
    bh = xcd + 8 * (slot % nbh8);
    blk = slot / nbh8;
    return bh < BH;
}
static inline unsigned xcd_grid(int BH, int nblocks) { return 8u * ((BH + 7) / 8) * nblocks; }

// ---- shared pieces of the second-generation 16-bit attention kernels -------------------------------

// Wave-private transpose of a [DH x 32] fp32 accumulator set (register j of block db = row db*32 +
// acc_row(j, g), column lane & 31) into row-major [32][DH] through LDS, so that global memory is then
// touched in full rows.  `buf` is the wave's own 32 x (DH + 4) floats.  After the call lane l holds, for
// i in [0, DH / 8): row 2 * i' ... see rows_read.
template <int DH>
__device__ __forceinline__ void acc_to_lds_rows(const float16v* acc, float* buf, int lane) {
    constexpr int NDB = DH / 32, LD = DH + 4;
    const int g = lane >> 5, li = lane & 31;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int jq = 0; jq < 4; ++jq)
            *reinterpret_cast<float4*>(buf + li * LD + db * 32 + 8 * jq + 4 * g) =
                make_float4(acc[db][4 * jq], acc[db][4 * jq + 1], acc[db][4 * jq + 2], acc[db][4 * jq + 3]);
}
// piece i of the row-major read-back: row and first column of the four floats this lane gets
template <int DH> __device__ __forceinline__ void row_piece(int i, int lane, int& row, int& col) {
    constexpr int LPR = DH / 4;            // lanes per row
    const int idx = i * 64 + lane;
    row = idx / LPR;
    col = (idx % LPR) * 4;
}

// dK / dV, second generation: stage-unrolled ring (LDS addresses are lane constants plus immediates),
// scalar-base tile loads, row-contiguous epilogue.
template <typename T, typename GT, int DH, int NW, int STAGES>
__global__ __launch_bounds__(NW * 64) void attn_bwd_dkdv2_kernel(AttnArgs a) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "direct-to-LDS kernels are for fp16 / bf16");
    constexpr int NDB = DH / 32, NKS = DH / 16;
    constexpr int TILE = 32 * DH;                       // elements of one Q or dO tile
    constexpr int CPR = DH / 8;                         // 16-byte chunks per row
    constexpr int NLD = 32 * CPR / (NW * 64);           // loads per thread per tile
    static_assert(32 * CPR % (NW * 64) == 0, "tile must split evenly");
    constexpr int NLOAD = 2 * NLD;
    static_assert(NLOAD * (STAGES - 1) <= 63, "too many loads in flight for vmcnt");
    constexpr int RING_BYTES = STAGES * 2 * TILE * 2;
    constexpr int EPI_LD = DH + 4;
    constexpr int EPI_BYTES = NW * 32 * EPI_LD * 4;
    constexpr int SMEM = RING_BYTES > EPI_BYTES ? RING_BYTES : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM];
    extern __shared__ __attribute__((aligned(16))) float stats[];   // -lse*log2e [Tpad], delta[Tpad]
    T* ring = reinterpret_cast<T*>(smem);
    const unsigned ring_lds = lds_addr(smem);

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5, li = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bh, kblk;
    if (!xcd_map(a.B * a.H, bh, kblk)) return;
    const int b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int key0wg = kblk * NW * 32;
    const int key0w = key0wg + wave * 32;
    const int key = key0w + li;
    const int nqb = (T_ + 31) / 32;
    const int Tpad = nqb * 32;
    float* sLse = stats;
    float* sDelta = stats + Tpad;

    typename E::opnd_t kreg[NKS], vreg[NKS];
    load_row_operands<T, DH>(kreg, reinterpret_cast<const T*>(a.kc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);
    load_row_operands<T, DH>(vreg, reinterpret_cast<const T*>(a.vc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);
    for (int t = tid; t < Tpad; t += NW * 64) {
        sLse[t] = t < T_ ? -a.lse[(long)bh * a.st_bhs + t] * kLog2e : 0.f;
        sDelta[t] = t < T_ ? a.delta[(long)bh * a.st_bhs + t] : 0.f;
    }

    // lane-constant LDS addresses inside stage 0's Q tile (the dO tile and the other stages are
    // compile-time offsets from these)
    const T* pkm[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) pkm[ks] = ring + km_offset<T, DH>(li, ks * 16, lane);
    const T* ptr0[NDB];
    const T* ptr1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        int o0, o1;
        tr_offsets<T, DH, true>(0, db * 32, lane, o0, o1);
        ptr0[db] = ring + o0;
        ptr1[db] = ring + o1;
    }
    // tile loads: per-lane byte offsets from the tile's first row
    unsigned qoff[NLD], dooff[NLD];
    const unsigned ldo_bytes = (unsigned)((long)a.B * EE * 2);
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int p = (i * NW + wave) * 64 + lane;
        const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
        qoff[i] = (unsigned)(r * DH * 2 + lc * 16);
        dooff[i] = (unsigned)(r * ldo_bytes + lc * 16);
    }
    const char* Qb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.q) + (long)bh * a.q_bhs));
    const char* dOb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.d_o) + (long)b * EE + (long)h * DH));
    const int qb_start = key0wg > P ? (key0wg - P) / 32 : 0;
    const int nt = nqb - qb_start;

    wait_vmcnt<0>();
    __syncthreads();

    auto issue = [&](int stage, int it) {
        // query rows past T are clamped to row T-1: finite data whose P and dS are forced to zero
        const unsigned dq_ = ring_lds + (unsigned)(stage * 2 * TILE * 2 + wave * 1024);   // this wave's 1 KB of load 0
        const int row0 = (qb_start + it) * 32;
        if (row0 + 32 <= T_) {
            const char* sq = Qb + (long)row0 * (DH * 2);
            const char* sd = dOb + (long)row0 * ldo_bytes;
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(qoff[i], sq, dq_ + i * NW * 1024);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(dooff[i], sd, dq_ + TILE * 2 + i * NW * 1024);
        } else {
            const int last = T_ - 1;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = (i * NW + wave) * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const int rr = min(row0 + r, last);
                dma16_saddr_lds((unsigned)(rr * DH * 2 + lc * 16), Qb, dq_ + i * NW * 1024);
            }
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = (i * NW + wave) * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const int rr = min(row0 + r, last);
                dma16_saddr_lds((unsigned)(rr * ldo_bytes + lc * 16), dOb, dq_ + TILE * 2 + i * NW * 1024);
            }
        }
    };

    float16v dk[NDB], dv[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[db][r] = 0.f; dv[db][r] = 0.f; }

#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s, s);

    for (int it0 = 0; it0 < nt; it0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {
            const int it = it0 + s;
            if (it < nt) {
                wait_vmcnt<NLOAD * (STAGES - 2)>();
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                issue((s + STAGES - 1) % STAGES, it + STAGES - 1);
                const int so = s * 2 * TILE;              // compile-time after unrolling
                const int qb = qb_start + it;
                if (key0w < S && key0w <= P + qb * 32 + 31) {
                    typename E::opnd_t qop[NKS], doop[NKS];
#pragma unroll
                    for (int ks = 0; ks < NKS; ++ks) {
                        qop[ks] = load_km<T>(pkm[ks] + so);
                        doop[ks] = load_km<T>(pkm[ks] + so + TILE);
                    }
                    float4 l4[4], d4[4];
#pragma unroll
                    for (int jq = 0; jq < 4; ++jq) {
                        l4[jq] = *reinterpret_cast<const float4*>(sLse + qb * 32 + 8 * jq + 4 * g);
                        d4[jq] = *reinterpret_cast<const float4*>(sDelta + qb * 32 + 8 * jq + 4 * g);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    float16v sacc, pacc;
#pragma unroll
                    for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
                    for (int ks = 0; ks < NKS; ++ks) {
                        sacc = E::mfma(qop[ks], kreg[ks], sacc);
                        pacc = E::mfma(doop[ks], vreg[ks], pacc);
                    }
                    // wave-uniform: every (query, key) pair of the block is visible and in range
                    const bool all_visible = (qb * 32 + 32 <= T_) && (key0w + 31 <= P + qb * 32) && (key0w + 32 <= S);
                    float pv[16], dsv[16];
                    if (all_visible) {
#pragma unroll
                        for (int jq = 0; jq < 4; ++jq) {
                            const float lv[4] = {l4[jq].x, l4[jq].y, l4[jq].z, l4[jq].w};
                            const float dl[4] = {d4[jq].x, d4[jq].y, d4[jq].z, d4[jq].w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int j = 4 * jq + e;
                                const float p = fast_exp2(fmaf(sacc[j], kLog2e, lv[e]));
                                pv[j] = p;
                                dsv[j] = p * (pacc[j] - dl[e]);
                            }
                        }
                    } else {
#pragma unroll
                        for (int jq = 0; jq < 4; ++jq) {
                            const float lv[4] = {l4[jq].x, l4[jq].y, l4[jq].z, l4[jq].w};
                            const float dl[4] = {d4[jq].x, d4[jq].y, d4[jq].z, d4[jq].w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const int j = 4 * jq + e;
                                const int t = qb * 32 + 8 * jq + 4 * g + e;
                                const bool vis = (t < T_) && (key <= P + t) && (key < S);
                                const float p = vis ? fast_exp2(fmaf(sacc[j], kLog2e, lv[e])) : 0.f;
                                pv[j] = p;
                                dsv[j] = p * (pacc[j] - dl[e]);
                            }
                        }
                    }
                    uint4 pop[2], dsop[2];
                    pop[0] = pack8<T>(pv); pop[1] = pack8<T>(pv + 8);
                    dsop[0] = pack8<T>(dsv); dsop[1] = pack8<T>(dsv + 8);
                    // dV^T += dO^T P, dK^T += Q^T dS: all sixteen transposed operand fetches first
                    uint4 ado[2][NDB], aq[2][NDB];
#pragma unroll
                    for (int hs = 0; hs < 2; ++hs)
#pragma unroll
                        for (int db = 0; db < NDB; ++db) {
                            ado[hs][db] = load_tr<T>(ptr0[db] + so + TILE + hs * 16 * DH, ptr1[db] + so + TILE + hs * 16 * DH);
                            aq[hs][db] = load_tr<T>(ptr0[db] + so + hs * 16 * DH, ptr1[db] + so + hs * 16 * DH);
                        }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int hs = 0; hs < 2; ++hs)
#pragma unroll
                        for (int db = 0; db < NDB; ++db) {
                            dv[db] = E::mfma(ado[hs][db], pop[hs], dv[db]);
                            dk[db] = E::mfma(aq[hs][db], dsop[hs], dk[db]);
                        }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            }
        }
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();      // every wave is done with the ring: reuse it for the epilogue
    asm volatile("" ::: "memory");

    float* ebuf = reinterpret_cast<float*>(smem) + wave * 32 * EPI_LD;
    GT* gKb = reinterpret_cast<GT*>(a.gk) + ((long)bh * a.cache_rows + key0w) * DH;
    GT* gVb = reinterpret_cast<GT*>(a.gv) + ((long)bh * a.cache_rows + key0w) * DH;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        acc_to_lds_rows<DH>(which == 0 ? dk : dv, ebuf, lane);
        GT* gb = which == 0 ? gKb : gVb;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        constexpr int NP = 32 * DH / 256;
        float4 val[NP];
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            int row, col;
            row_piece<DH>(i, lane, row, col);
            val[i] = *reinterpret_cast<const float4*>(ebuf + row * EPI_LD + col);
        }
        // incoming gradient of these rows (prefix rows: the accumulator itself; slice rows: what the later
        // slices left in the gradient cache)
        float old[NP][4];
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            int row, col;
            row_piece<DH>(i, lane, row, col);
            const int kk = key0w + row;
            old[i][0] = old[i][1] = old[i][2] = old[i][3] = 0.f;
            const bool rd = kk < S && (kk < P ? a.accumulate_prefix != 0 : a.has_incoming != 0);
            if (rd) load4<GT>(gb + (long)row * DH + col, old[i]);
        }
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            int row, col;
            row_piece<DH>(i, lane, row, col);
            const int kk = key0w + row;
            if (kk < S) {
                const float r0 = old[i][0] + val[i].x, r1 = old[i][1] + val[i].y, r2 = old[i][2] + val[i].z,
                            r3 = old[i][3] + val[i].w;
                if (kk < P) {
                    store4<GT>(gb + (long)row * DH + col, r0, r1, r2, r3);
                } else {
                    T* dst = reinterpret_cast<T*>(a.dqkv) + ((long)(kk - P) * a.B + b) * (3 * EE) + (long)h * 3 * DH +
                             (which + 1) * DH + col;
                    store4<T>(dst, r0, r1, r2, r3);
                    if (a.zero_slice_rows) store4<GT>(gb + (long)row * DH + col, 0.f, 0.f, 0.f, 0.f);
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the buffer is rewritten by the next pass
    }
}

// dQ, second generation.  A workgroup owns 32 queries of one (batch, head); its NW waves split the key
// range, each streaming its own K / V tiles of 32 keys through a private two-stage LDS ring (no
// workgroup barrier inside the loop), and the NW partial dQ blocks are summed through LDS at the end.
// The kernel also computes delta = rowsum(dO * O) for its queries and leaves it in a.delta for the
// dK/dV kernel that follows on the stream.
// LDS bytes of the dQ workgroup: NW private rings of two stages of K + V, reused for the reduction
template <int DH, int NW> constexpr int dq2_smem_bytes() {
    constexpr int ring = NW * 2 * 2 * 32 * DH * 2, epi = NW * 32 * (DH + 4) * 4;
    return ring > epi ? ring : epi;
}

// The work of workgroup `wg_id` of xcd_grid(B*H, ceil(T/32)); `smem` = dq2_smem_bytes<DH, NW>() bytes, 16-byte aligned.
template <typename T, int DH, int NW>
__device__ __forceinline__ void attn_bwd_dq2_body(const AttnArgs& a, unsigned char* smem, int wg_id) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "direct-to-LDS kernels are for fp16 / bf16");
    constexpr int NDB = DH / 32, NKS = DH / 16;
    constexpr int TILE = 32 * DH;                       // elements of one K or V tile
    constexpr int CPR = DH / 8;
    constexpr int NLD = 32 * CPR / 64;                  // loads per lane per tile (one wave loads a whole tile)
    constexpr int NLOAD = 2 * NLD;
    static_assert(NLOAD <= 63, "too many loads in flight for vmcnt");
    constexpr int WAVE_RING = 2 * 2 * TILE * 2;         // bytes: two stages of K + V
    constexpr int EPI_LD = DH + 4;

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5, li = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bh, qblk;
    if (!xcd_map(a.B * a.H, bh, qblk, wg_id)) return;
    const int b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int q0 = ((T_ + 31) / 32 - 1 - qblk) * 32;     // the blocks with the longest key range start first
    const int tq = q0 + li;
    const bool qok = tq < T_;
    const int kv_end = P + min(T_, q0 + 32);
    const int ntiles = (kv_end + 31) / 32;
    const int tpw = (ntiles + NW - 1) / NW;
    const int t_beg = wave * tpw, t_end = min(ntiles, t_beg + tpw);
    const int nt = max(t_end - t_beg, 0);

    T* ring = reinterpret_cast<T*>(smem) + wave * (WAVE_RING / 2);
    const unsigned ring_lds = lds_addr(smem) + wave * WAVE_RING;

    // lane-constant LDS addresses inside stage 0's K tile
    const T* pkm[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) pkm[ks] = ring + km_offset<T, DH>(li, ks * 16, lane);
    const T* ptr0[NDB];
    const T* ptr1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        int o0, o1;
        tr_offsets<T, DH, true>(0, db * 32, lane, o0, o1);
        ptr0[db] = ring + o0;
        ptr1[db] = ring + o1;
    }
    unsigned koff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int p = i * 64 + lane;
        const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
        koff[i] = (unsigned)(r * DH * 2 + lc * 16);
    }
    const char* Kb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.kc) + (long)bh * a.cache_rows * DH));
    const char* Vb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.vc) + (long)bh * a.cache_rows * DH));

    auto issue = [&](int stage, int tile) {
        // rows at or past S are clamped to row S-1: finite data, and every such key is masked
        const unsigned dst = ring_lds + (unsigned)(stage * 2 * TILE * 2);
        const int row0 = tile * 32;
        if (row0 + 32 <= S) {
            const char* sk = Kb + (long)row0 * (DH * 2);
            const char* sv = Vb + (long)row0 * (DH * 2);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(koff[i], sk, dst + i * 1024);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(koff[i], sv, dst + TILE * 2 + i * 1024);
        } else {
            const int last = S - 1;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const unsigned off = (unsigned)(min(row0 + r, last) * DH * 2 + lc * 16);
                dma16_saddr_lds(off, Kb, dst + i * 1024);
            }
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const unsigned off = (unsigned)(min(row0 + r, last) * DH * 2 + lc * 16);
                dma16_saddr_lds(off, Vb, dst + TILE * 2 + i * 1024);
            }
        }
    };

    float16v dq[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[db][r] = 0.f;

    // the first tile's loads go out before the query-side rows are asked for, so that the two round trips overlap
    // (vector-memory operations complete in issue order: the first wait in the loop covers both)
    if (nt > 0) issue(0, t_beg);
    typename E::opnd_t qreg[NKS], doreg[NKS];
    const long orow = ((long)tq * a.B + b) * EE + (long)h * DH;
    load_row_operands<T, DH>(qreg, reinterpret_cast<const T*>(a.q) + ((long)bh * a.q_bhs + (long)tq * DH), qok, g);
    load_row_operands<T, DH>(doreg, reinterpret_cast<const T*>(a.d_o) + orow, qok, g);
    float delta_q;
    {
        typename E::opnd_t oreg[NKS];
        load_row_operands<T, DH>(oreg, reinterpret_cast<const T*>(a.o) + orow, qok, g);
        float s = 0.f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const T* x = reinterpret_cast<const T*>(&oreg[ks]);
            const T* y = reinterpret_cast<const T*>(&doreg[ks]);
#pragma unroll
            for (int e = 0; e < 8; ++e) s = fmaf(E::to_float(x[e]), E::to_float(y[e]), s);
        }
        delta_q = s + __shfl_xor(s, 32, 64);
    }
    if (wave == 0 && g == 0 && qok) a.delta[(long)bh * a.st_bhs + tq] = delta_q;
    const float lse_neg = qok ? -a.lse[(long)bh * a.st_bhs + tq] * kLog2e : 0.f;


    auto step = [&](auto stage_c, int it) {
        constexpr int s = decltype(stage_c)::value;
        // the other stage was last read one iteration ago (lgkmcnt(0) below): refill it, then wait
        // for this iteration's tile (all but the NLOAD loads just issued)
        if (it + 1 < nt) {
            issue(s ^ 1, t_beg + it + 1);
            wait_vmcnt<NLOAD>();
        } else {
            wait_vmcnt<0>();
        }
        const int so = s * 2 * TILE;
        const int key0 = (t_beg + it) * 32;
        typename E::opnd_t kop[NKS], vop[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            kop[ks] = load_km<T>(pkm[ks] + so);
            vop[ks] = load_km<T>(pkm[ks] + so + TILE);
        }
        __builtin_amdgcn_sched_barrier(0);
        float16v sacc, pacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            sacc = E::mfma(kop[ks], qreg[ks], sacc);
            pacc = E::mfma(vop[ks], doreg[ks], pacc);
        }
        float dsv[16];
        if (key0 + 31 > P + q0) {        // wave-uniform: the tile touches the causal boundary
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int key = key0 + acc_row(j, g);
                const float p = key > P + tq ? 0.f : fast_exp2(fmaf(sacc[j], kLog2e, lse_neg));
                dsv[j] = p * (pacc[j] - delta_q);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float p = fast_exp2(fmaf(sacc[j], kLog2e, lse_neg));
                dsv[j] = p * (pacc[j] - delta_q);
            }
        }
        uint4 dsop[2];
        dsop[0] = pack8<T>(dsv);
        dsop[1] = pack8<T>(dsv + 8);
        uint4 ak[2][NDB];
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                ak[hs][db] = load_tr<T>(ptr0[db] + so + hs * 16 * DH, ptr1[db] + so + hs * 16 * DH);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) dq[db] = E::mfma(ak[hs][db], dsop[hs], dq[db]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    {
        int it = 0;
        for (; it + 1 < nt; it += 2) {
            step(std::integral_constant<int, 0>(), it);
            step(std::integral_constant<int, 1>(), it + 1);
        }
        if (it < nt) step(std::integral_constant<int, 0>(), it);
    }
    wait_vmcnt<0>();
    __syncthreads();       // every wave is done with its ring: the space is reused for the reduction

    float* ebuf = reinterpret_cast<float*>(smem);
    acc_to_lds_rows<DH>(dq, ebuf + wave * 32 * EPI_LD, lane);
    __syncthreads();
    // thread -> (row, 16 consecutive columns) for DH = 128 with 256 threads; generally 32*DH/(NW*64) columns
    constexpr int CPT = 32 * DH / (NW * 64);             // columns per thread
    static_assert(CPT % 4 == 0 && DH % CPT == 0, "bad reduction split");
    const int row = tid / (DH / CPT), c0 = (tid % (DH / CPT)) * CPT;
    if (q0 + row < T_) {
        T* dst = reinterpret_cast<T*>(a.dqkv) + ((long)(q0 + row) * a.B + b) * (3 * EE) + (long)h * 3 * DH + c0;
#pragma unroll
        for (int c = 0; c < CPT; c += 4) {
            float4 acc4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float4 v = *reinterpret_cast<const float4*>(ebuf + (w * 32 + row) * EPI_LD + c0 + c);
                acc4.x += v.x; acc4.y += v.y; acc4.z += v.z; acc4.w += v.w;
            }
            store4<T>(dst + c, acc4.x * a.qscale, acc4.y * a.qscale, acc4.z * a.qscale, acc4.w * a.qscale);
        }
    }
}

template <typename T, int DH, int NW>
__global__ __launch_bounds__(NW * 64) void attn_bwd_dq2_kernel(AttnArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char smem[dq2_smem_bytes<DH, NW>()];
    attn_bwd_dq2_body<T, DH, NW>(a, smem, blockIdx.x);
}

// Forward, second generation.  A workgroup owns 32 queries of one (batch, head); its NW waves split the
// key range, each streaming its own K / V tiles of 32 keys through a private two-stage LDS ring and
// keeping its own online-softmax state; the NW partial (m, l, O) are merged through LDS at the end.
// STG = 1 gives a wave a single tile buffer (it loads, waits, computes) and is meant for eight waves: two
// per SIMD take turns, which hides the load latency as the second stage does for four, and the key range
// of a query block is split eight ways instead of four -- for the cases where (batch, head) x query blocks
// leave CUs without a workgroup and the length of a wave's key loop is what the call takes.
template <typename T, int DH, int NW, int STG = 2>
__global__ __launch_bounds__(NW * 64) void attn_fwd2_kernel(AttnArgs a) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "direct-to-LDS kernels are for fp16 / bf16");
    constexpr int NDB = DH / 32, NKS = DH / 16;
    constexpr int TILE = 32 * DH;
    constexpr int CPR = DH / 8;
    constexpr int NLD = 32 * CPR / 64;
    constexpr int NLOAD = 2 * NLD;
    static_assert(NLOAD <= 63, "too many loads in flight for vmcnt");
    constexpr int WAVE_RING = STG * 2 * TILE * 2;        // bytes: STG stages of K + V
    constexpr int EPI_LD = DH + 4;
    constexpr int STAT_FLOATS = 2 * NW * 32;
    constexpr int EPI_BYTES = (STAT_FLOATS + NW * 32 * EPI_LD) * 4;
    constexpr int SMEM = NW * WAVE_RING > EPI_BYTES ? NW * WAVE_RING : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM];

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5, li = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bh, qblk;
    if (!xcd_map(a.B * a.H, bh, qblk)) return;
    const int b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int q0 = ((T_ + 31) / 32 - 1 - qblk) * 32;     // the blocks with the longest key range start first
    const int tq = q0 + li;
    const bool qok = tq < T_;
    const int kv_end = P + min(T_, q0 + 32);
    const int ntiles = (kv_end + 31) / 32;
    // the key tiles of this workgroup: all of them, or its share when gridDim.y workgroups split a block's keys
    // (the grid's x extent is a multiple of eight, so they all stay on the XCD that xcd_map gives the block)
    int wg_beg = 0, wg_end = ntiles;
    if (a.nsplit > 1) {
        const int per = (ntiles + a.nsplit - 1) / a.nsplit;
        wg_beg = min(ntiles, (int)blockIdx.y * per);
        wg_end = min(ntiles, wg_beg + per);
    }
    const int tpw = (wg_end - wg_beg + NW - 1) / NW;
    const int t_beg = wg_beg + wave * tpw, t_end = min(wg_end, t_beg + tpw);
    const int nt = max(t_end - t_beg, 0);

    T* ring = reinterpret_cast<T*>(smem) + wave * (WAVE_RING / 2);
    const unsigned ring_lds = lds_addr(smem) + wave * WAVE_RING;

    const T* pkm[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) pkm[ks] = ring + km_offset<T, DH>(li, ks * 16, lane);
    const T* ptr0[NDB];
    const T* ptr1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        int o0, o1;
        tr_offsets<T, DH, true>(0, db * 32, lane, o0, o1);
        ptr0[db] = ring + TILE + o0;          // inside the V tile
        ptr1[db] = ring + TILE + o1;
    }
    unsigned koff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int p = i * 64 + lane;
        const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
        koff[i] = (unsigned)(r * DH * 2 + lc * 16);
    }
    const char* Kb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.kc) + (long)bh * a.cache_rows * DH));
    const char* Vb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.vc) + (long)bh * a.cache_rows * DH));

    auto issue = [&](int stage, int tile) {
        // rows at or past S are clamped to row S-1: finite data, and every such key is masked
        const unsigned dst = ring_lds + (unsigned)(stage * 2 * TILE * 2);
        const int row0 = tile * 32;
        if (row0 + 32 <= S) {
            const char* sk = Kb + (long)row0 * (DH * 2);
            const char* sv = Vb + (long)row0 * (DH * 2);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(koff[i], sk, dst + i * 1024);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(koff[i], sv, dst + TILE * 2 + i * 1024);
        } else {
            const int last = S - 1;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const unsigned off = (unsigned)(min(row0 + r, last) * DH * 2 + lc * 16);
                dma16_saddr_lds(off, Kb, dst + i * 1024);
            }
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const unsigned off = (unsigned)(min(row0 + r, last) * DH * 2 + lc * 16);
                dma16_saddr_lds(off, Vb, dst + TILE * 2 + i * 1024);
            }
        }
    };

    float16v oacc[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m = -INFINITY, lsum = 0.f;

    // the first tile's loads go out before the query rows are asked for, so that the two round trips overlap
    // (vector-memory operations complete in issue order: the first wait in the loop covers both)
    if (nt > 0) issue(0, t_beg);
    typename E::opnd_t qreg[NKS];
    load_row_operands<T, DH>(qreg, reinterpret_cast<const T*>(a.q) + ((long)bh * a.q_bhs + (long)tq * DH), qok, g);

    auto step = [&](auto stage_c, int it) {
        constexpr int s = decltype(stage_c)::value;
        if constexpr (STG == 1) {
            if (it > 0) issue(0, t_beg + it);   // the wave's reads of the previous tile are complete (lgkmcnt below)
            wait_vmcnt<0>();
        } else if (it + 1 < nt) {
            issue(s ^ 1, t_beg + it + 1);
            wait_vmcnt<NLOAD>();
        } else {
            wait_vmcnt<0>();
        }
        constexpr int so = s * 2 * TILE;
        const int key0 = (t_beg + it) * 32;
        typename E::opnd_t kop[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) kop[ks] = load_km<T>(pkm[ks] + so);
        // the V^T operands do not depend on the scores: fetch them now, use them after the softmax
        uint4 av[2][NDB];
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                av[hs][db] = load_tr<T>(ptr0[db] + so + hs * 16 * DH, ptr1[db] + so + hs * 16 * DH);
        __builtin_amdgcn_sched_barrier(0);
        float16v sacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) sacc = E::mfma(kop[ks], qreg[ks], sacc);
        float sv[16];
        float mt = -INFINITY;
        if (key0 + 31 > P + q0) {            // wave-uniform: the tile touches the causal boundary
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int key = key0 + acc_row(j, g);
                sv[j] = key > P + tq ? -INFINITY : sacc[j];
                mt = fmaxf(mt, sv[j]);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) { sv[j] = sacc[j]; mt = fmaxf(mt, sv[j]); }
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        // m is the row's REFERENCE value of the exponentials, not its running maximum: a row keeps it while its
        // scores stay below m + kSlack (exponentials up to e^kSlack = 148, well inside fp16 and the fp32 sums), so
        // the accumulators are rescaled only when some row of the wave outgrows that -- on the first tile and hardly
        // ever again, where a running maximum moves for some of 32 rows on most tiles of a 2048-key range.  The
        // row's log-sum-exp is m + log(sum) either way.
        constexpr float kSlack = 5.0f;
        if (__builtin_amdgcn_ballot_w64(mt > m + kSlack) != 0) {   // wave-uniform
            const float m_new = fmaxf(m, mt);
            const float alpha = m_new == -INFINITY ? 1.0f : fast_exp2((m - m_new) * kLog2e);
            m = m_new;
            lsum *= alpha;
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
        }
        const float mneg = m == -INFINITY ? 0.f : -m * kLog2e;
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            sv[j] = fast_exp2(fmaf(sv[j], kLog2e, mneg));   // exp(s - m); -inf -> 0
            psum += sv[j];
        }
        lsum += psum;
        uint4 pop[2];
        pop[0] = pack8<T>(sv);
        pop[1] = pack8<T>(sv + 8);
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) oacc[db] = E::mfma(av[hs][db], pop[hs], oacc[db]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    if constexpr (STG == 1) {
        for (int it = 0; it < nt; ++it) step(std::integral_constant<int, 0>(), it);
    } else {
        int it = 0;
        for (; it + 1 < nt; it += 2) {
            step(std::integral_constant<int, 0>(), it);
            step(std::integral_constant<int, 1>(), it + 1);
        }
        if (it < nt) step(std::integral_constant<int, 0>(), it);
    }
    wait_vmcnt<0>();
    __syncthreads();       // every wave is done with its ring: the space is reused for the merge

    float* sM = reinterpret_cast<float*>(smem);
    float* sL = sM + NW * 32;
    float* ebuf = sL + NW * 32;
    const float lw = lsum + __shfl_xor(lsum, 32, 64);
    if (g == 0) { sM[wave * 32 + li] = m; sL[wave * 32 + li] = lw; }
    __syncthreads();
    float m_tot = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) m_tot = fmaxf(m_tot, sM[w * 32 + li]);
    const float m_ts = m_tot == -INFINITY ? 0.f : m_tot;
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) L += sL[w * 32 + li] * fast_exp2((sM[w * 32 + li] - m_ts) * kLog2e);
    const float f = L > 0.f ? fast_exp2((m - m_ts) * kLog2e) / L : 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= f;
    acc_to_lds_rows<DH>(oacc, ebuf + wave * 32 * EPI_LD, lane);
    // a workgroup that has a share of the keys only leaves its normalised output and its log-sum-exp as fp32
    // partials; attn_fwd_merge_kernel weighs the shares together
    const bool partial = a.nsplit > 1;
    const long prow0 = ((long)blockIdx.y * (a.B * a.H) + bh) * T_;
    if (wave == 0 && g == 0 && qok) {
        const float lse_wg = L > 0.f ? m_tot + logf(L) : -INFINITY;
        if (partial) a.part_lse[prow0 + tq] = lse_wg;
        else a.lse[(long)bh * a.st_bhs + tq] = lse_wg;
    }
    __syncthreads();
    constexpr int CPT = 32 * DH / (NW * 64);
    static_assert(CPT % 4 == 0 && DH % CPT == 0, "bad reduction split");
    const int row = tid / (DH / CPT), c0 = (tid % (DH / CPT)) * CPT;
    if (q0 + row < T_) {
        T* dst = reinterpret_cast<T*>(a.o) + ((long)(q0 + row) * a.B + b) * EE + (long)h * DH + c0;
        float* pdst = a.part_o + (prow0 + q0 + row) * DH + c0;
#pragma unroll
        for (int c = 0; c < CPT; c += 4) {
            float4 acc4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const float4 v = *reinterpret_cast<const float4*>(ebuf + (w * 32 + row) * EPI_LD + c0 + c);
                acc4.x += v.x; acc4.y += v.y; acc4.z += v.z; acc4.w += v.w;
            }
            if (partial) *reinterpret_cast<float4*>(pdst + c) = acc4;
            else store4<T>(dst + c, acc4.x, acc4.y, acc4.z, acc4.w);
        }
    }
}

// Forward for slices of 64 queries and more.  A workgroup owns 64 queries of one (batch, head) -- two blocks of 32 --
// and, as in attn_fwd2_kernel, its NW waves split the key range, each streaming its own K / V tiles through a
// private two-stage ring.  Every wave works on BOTH query blocks against each tile it has fetched: a K / V byte
// enters LDS once per 64 queries instead of once per 32 (the global -> LDS path is what bounds the 32-query form
// from 128-token slices on), the K and V^T operands are read from LDS once for two blocks, and the two blocks are
// independent instruction chains.  The loop is software-pipelined so that one straight-line block holds the
// exponentials of tile t, its output MFMAs and the score MFMAs of tile t + 1 -- vector ALU and MFMA work with no
// dependency between them, for the scheduler to interleave (one wave per SIMD: two blocks' accumulators and query
// operands take more than half of the register file).  What has to sit between two such blocks is short: the row
// maxima of the new scores, and the rescaling of the accumulators on the rare tile that moves a row's maximum.
// A pair whose second block lies beyond the slice computes it on zero queries and stores nothing of it.
template <typename T, int DH, int NW>
__global__ __launch_bounds__(NW * 64) void attn_fwd3_kernel(AttnArgs a) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "direct-to-LDS kernels are for fp16 / bf16");
    constexpr int NDB = DH / 32, NKS = DH / 16;
    constexpr int TILE = 32 * DH;
    constexpr int CPR = DH / 8;
    constexpr int NLD = 32 * CPR / 64;                   // loads per K or V tile and lane
    static_assert(3 * NLD <= 63, "too many loads in flight for vmcnt");
    constexpr int WAVE_RING = 2 * 2 * TILE * 2;          // bytes: two stages of K + V
    constexpr int EPI_LD = DH + 4;
    constexpr int STAT_FLOATS = 2 * NW * 32;
    constexpr int EPI_BYTES = (STAT_FLOATS + NW * 32 * EPI_LD) * 4;
    constexpr int SMEM = NW * WAVE_RING > EPI_BYTES ? NW * WAVE_RING : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM];

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5, li = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bh, qblk;
    if (!xcd_map(a.B * a.H, bh, qblk)) return;
    const int b = bh / a.H, h = bh - b * a.H;
    const int T_ = a.T, P = a.P, S = a.P + a.T;
    const long EE = (long)a.H * DH;
    const int q0 = ((T_ + 63) / 64 - 1 - qblk) * 64;     // the pairs with the longest key range start first
    const bool two = q0 + 32 < T_;                       // workgroup-uniform: the pair's second block exists
    const int tq0 = q0 + li, tq1 = q0 + 32 + li;
    const bool qok0 = tq0 < T_, qok1 = tq1 < T_;
    const int kv_end = P + min(T_, q0 + 64);
    const int ntiles = (kv_end + 31) / 32;
    int wg_beg = 0, wg_end = ntiles;
    if (a.nsplit > 1) {
        const int per = (ntiles + a.nsplit - 1) / a.nsplit;
        wg_beg = min(ntiles, (int)blockIdx.y * per);
        wg_end = min(ntiles, wg_beg + per);
    }
    const int tpw = (wg_end - wg_beg + NW - 1) / NW;
    const int t_beg = wg_beg + wave * tpw, t_end = min(wg_end, t_beg + tpw);
    const int nt = max(t_end - t_beg, 0);

    T* ring = reinterpret_cast<T*>(smem) + wave * (WAVE_RING / 2);
    const unsigned ring_lds = lds_addr(smem) + wave * WAVE_RING;

    const T* pkm[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) pkm[ks] = ring + km_offset<T, DH>(li, ks * 16, lane);
    const T* ptr0[NDB];
    const T* ptr1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        int o0, o1;
        tr_offsets<T, DH, true>(0, db * 32, lane, o0, o1);
        ptr0[db] = ring + TILE + o0;          // inside the V tile
        ptr1[db] = ring + TILE + o1;
    }
    unsigned koff[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int p = i * 64 + lane;
        const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
        koff[i] = (unsigned)(r * DH * 2 + lc * 16);
    }
    const char* Kb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.kc) + (long)bh * a.cache_rows * DH));
    const char* Vb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.vc) + (long)bh * a.cache_rows * DH));

    // one tile (K: which = 0, V: which = 1) of 32 keys into its half of a stage; rows at or past S are clamped to
    // row S - 1: finite data, and every such key is masked
    auto issue = [&](int stage, int which, int tile) {
        const unsigned dst = ring_lds + (unsigned)((stage * 2 + which) * TILE * 2);
        const char* base = which ? Vb : Kb;
        const int row0 = tile * 32;
        if (row0 + 32 <= S) {
            const char* sb = base + (long)row0 * (DH * 2);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(koff[i], sb, dst + i * 1024);
        } else {
            const int last = S - 1;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                const unsigned off = (unsigned)(min(row0 + r, last) * DH * 2 + lc * 16);
                dma16_saddr_lds(off, base, dst + i * 1024);
            }
        }
    };

    float16v oacc0[NDB], oacc1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { oacc0[db][r] = 0.f; oacc1[db][r] = 0.f; }
    float m0 = -INFINITY, l0 = 0.f, m1 = -INFINITY, l1 = 0.f;

    // loads go out in the order K(0) V(0) K(1) V(1), then per tile t: K(t + 2) when its body starts, V(t + 2) when
    // it ends (vector-memory operations complete in issue order)
    if (nt > 0) { issue(0, 0, t_beg); issue(0, 1, t_beg); }
    if (nt > 1) { issue(1, 0, t_beg + 1); issue(1, 1, t_beg + 1); }
    typename E::opnd_t qreg0[NKS], qreg1[NKS];
    const T* qbase = reinterpret_cast<const T*>(a.q) + (long)bh * a.q_bhs;
    load_row_operands<T, DH>(qreg0, qbase + (long)tq0 * DH, qok0, g);
    load_row_operands<T, DH>(qreg1, qbase + (long)(qok1 ? tq1 : 0) * DH, qok1, g);

    // score blocks of both query blocks against the K tile in stage `so`
    auto scores = [&](int so, float16v& s0, float16v& s1) {
#pragma unroll
        for (int r = 0; r < 16; ++r) { s0[r] = 0.f; s1[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const typename E::opnd_t kop = load_km<T>(pkm[ks] + so);
            s0 = E::mfma(kop, qreg0[ks], s0);
            s1 = E::mfma(kop, qreg1[ks], s1);
        }
    };
    // causal mask (tiles at a block's boundary only) and the row maxima of one block's scores
    auto tile_max = [&](float16v& sc, int key0, int tq, int qb0) {
        if (key0 + 31 > P + qb0) {           // wave-uniform
#pragma unroll
            for (int j = 0; j < 16; ++j)
                if (key0 + acc_row(j, g) > P + tq) sc[j] = -INFINITY;
        }
        float mt = sc[0];
#pragma unroll
        for (int j = 1; j < 16; ++j) mt = fmaxf(mt, sc[j]);
        return fmaxf(mt, __shfl_xor(mt, 32, 64));
    };
    // exp(s - m) of one block, packed as the two MFMA operands; returns the lane's share of the row sums
    auto exps = [&](const float16v& sc, float mneg, uint4* pop) {
        float sv[16];
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            sv[j] = fast_exp2(fmaf(sc[j], kLog2e, mneg));   // -inf -> 0
            psum += sv[j];
        }
        pop[0] = pack8<T>(sv);
        pop[1] = pack8<T>(sv + 8);
        return psum;
    };

    float16v s0, s1;
    if (nt > 0) {
        if (nt > 1) wait_vmcnt<3 * NLD>(); else wait_vmcnt<NLD>();
        scores(0, s0, s1);
    }
    // (the score MFMAs of "the next tile" also run behind a wave's last tile, on whatever the other stage holds:
    // nothing reads their result, and the loop body stays one piece of code per stage)
    auto body = [&](auto stage_c, int it) {
        constexpr int st = decltype(stage_c)::value;
        constexpr int so = st * 2 * TILE, son = (st ^ 1) * 2 * TILE;
        const int key0 = (t_beg + it) * 32;
        // -- between the straight-line blocks: row maxima, and the rare move of the reference --
        // m0 / m1 are the rows' REFERENCE values of the exponentials, not their running maxima: a row keeps its
        // reference while its scores stay below reference + kSlack (exponentials up to e^kSlack = 148, well inside
        // fp16 and the fp32 sums), so that the accumulators are rescaled only when some row of the wave outgrows
        // that -- on the first tile, and hardly ever again (a running maximum moves for some row of 64 on nearly
        // every tile of a 2048-key range).  The row's log-sum-exp is reference + log(sum) either way.
        constexpr float kSlack = 5.0f;
        const float mt0 = tile_max(s0, key0, tq0, q0), mt1 = tile_max(s1, key0, tq1, q0 + 32);
        float al0 = 1.0f, al1 = 1.0f;
        if (__builtin_amdgcn_ballot_w64(mt0 > m0 + kSlack || mt1 > m1 + kSlack) != 0) {
            const float mn0 = fmaxf(m0, mt0), mn1 = fmaxf(m1, mt1);
            al0 = mn0 == -INFINITY ? 1.0f : fast_exp2((m0 - mn0) * kLog2e);
            al1 = mn1 == -INFINITY ? 1.0f : fast_exp2((m1 - mn1) * kLog2e);
            m0 = mn0; m1 = mn1;
            // The accumulators stay in accumulation registers for the whole loop: a plain multiply here would make
            // them vector registers everywhere (the vector ALU cannot address the other file) and the loop would
            // spill.  The copies are explicit, with the wait states an MFMA result needs before it is read and a
            // written register before an MFMA takes it as its addend.
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float t0, t1;
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t0) : "a"(oacc0[db][r]));
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t1) : "a"(oacc1[db][r]));
                    t0 *= al0; t1 *= al1;
                    asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(oacc0[db][r]) : "v"(t0));
                    asm volatile("v_accvgpr_write_b32 %0, %1" : "=a"(oacc1[db][r]) : "v"(t1));
                }
            asm volatile("s_nop 7" ::: "memory");
            l0 *= al0; l1 *= al1;
        }
        const float ms0 = m0 == -INFINITY ? 0.f : m0, ms1 = m1 == -INFINITY ? 0.f : m1;
        if (it + 2 < nt) { issue(st, 0, t_beg + it + 2); wait_vmcnt<2 * NLD>(); }   // K(it) was read one body ago
        else wait_vmcnt<0>();
        // -- the block: exponentials and output MFMAs of this tile, score MFMAs of the next --
        uint4 av[2][NDB];
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db)
                av[hs][db] = load_tr<T>(ptr0[db] + so + hs * 16 * DH, ptr1[db] + so + hs * 16 * DH);
        float16v n0, n1;
        scores(son, n0, n1);
        uint4 p0[2], p1[2];
        l0 += exps(s0, -ms0 * kLog2e, p0);
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) oacc0[db] = E::mfma(av[hs][db], p0[hs], oacc0[db]);
        l1 += exps(s1, -ms1 * kLog2e, p1);
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) oacc1[db] = E::mfma(av[hs][db], p1[hs], oacc1[db]);
        s0 = n0; s1 = n1;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the stage's V tile is in registers
        if (it + 2 < nt) issue(st, 1, t_beg + it + 2);
    };
    for (int it = 0; it < nt; it += 2) {
        body(std::integral_constant<int, 0>(), it);
        if (it + 1 < nt) body(std::integral_constant<int, 1>(), it + 1);
    }
    wait_vmcnt<0>();

    // merge of the NW partial (m, l, O) of a block through LDS, one block after the other in the same space
    float* sM = reinterpret_cast<float*>(smem);
    float* sL = sM + NW * 32;
    float* ebuf = sL + NW * 32;
    const bool partial = a.nsplit > 1;
    constexpr int CPT = 32 * DH / (NW * 64);
    static_assert(CPT % 4 == 0 && DH % CPT == 0, "bad reduction split");
    auto finish = [&](float16v* oacc, float m, float lsum, int qb0, int tq, bool qok) {
        __syncthreads();       // every wave is done with its ring (or with the previous block's merge)
        const float lw = lsum + __shfl_xor(lsum, 32, 64);
        if (g == 0) { sM[wave * 32 + li] = m; sL[wave * 32 + li] = lw; }
        __syncthreads();
        float m_tot = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) m_tot = fmaxf(m_tot, sM[w * 32 + li]);
        const float m_ts = m_tot == -INFINITY ? 0.f : m_tot;
        float L = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) L += sL[w * 32 + li] * fast_exp2((sM[w * 32 + li] - m_ts) * kLog2e);
        const float f = L > 0.f ? fast_exp2((m - m_ts) * kLog2e) / L : 0.f;
        // (the accumulators are read out of their accumulation registers explicitly, see the loop; layout as
        // acc_to_lds_rows)
        {
            float* wbuf = ebuf + wave * 32 * EPI_LD;
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
            for (int db = 0; db < NDB; ++db)
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    float t[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t[e]) : "a"(oacc[db][4 * jq + e]));
                        t[e] *= f;
                    }
                    *reinterpret_cast<float4*>(wbuf + li * EPI_LD + db * 32 + 8 * jq + 4 * g) = make_float4(t[0], t[1], t[2], t[3]);
                }
        }
        const long prow0 = ((long)blockIdx.y * (a.B * a.H) + bh) * T_;
        if (wave == 0 && g == 0 && qok) {
            const float lse_wg = L > 0.f ? m_tot + logf(L) : -INFINITY;
            if (partial) a.part_lse[prow0 + tq] = lse_wg;
            else a.lse[(long)bh * a.st_bhs + tq] = lse_wg;
        }
        __syncthreads();
        const int row = tid / (DH / CPT), c0 = (tid % (DH / CPT)) * CPT;
        if (qb0 + row < T_) {
            T* dst = reinterpret_cast<T*>(a.o) + ((long)(qb0 + row) * a.B + b) * EE + (long)h * DH + c0;
            float* pdst = a.part_o + (prow0 + qb0 + row) * DH + c0;
#pragma unroll
            for (int c = 0; c < CPT; c += 4) {
                float4 acc4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float4 v = *reinterpret_cast<const float4*>(ebuf + (w * 32 + row) * EPI_LD + c0 + c);
                    acc4.x += v.x; acc4.y += v.y; acc4.z += v.z; acc4.w += v.w;
                }
                if (partial) *reinterpret_cast<float4*>(pdst + c) = acc4;
                else store4<T>(dst + c, acc4.x, acc4.y, acc4.z, acc4.w);
            }
        }
    };
    finish(oacc0, m0, l0, q0, tq0, qok0);
    if (two) finish(oacc1, m1, l1, q0 + 32, tq1, qok1);
}

// ------------------------------------------------------------------------------------------------
// dK / dV of one slice's keys against every query position that can see them (tp_attn_suffix_dkdv).
// A workgroup owns 32 keys of one (batch, head); its NW waves split the query blocks [key .. q_end),
// each streaming its own Q / dO tiles of 32 positions (plus their lse and delta) through a private
// two-stage LDS ring, and the NW partial dK / dV blocks are summed through LDS at the end.
// ------------------------------------------------------------------------------------------------
struct SuffixArgs {
    const void* kc; const void* vc; const void* q; const void* d_o;
    const float* lse; const float* delta; void* dqkv;
    const void* o_all;      // OWN_DELTA only: the attention output [.., B, H*Dh], row = position
    int own_end;            // OWN_DELTA only: delta of the positions [P, own_end) is computed here
    int B, H, P, T, Lq;
    long cache_rows, q_bhs, st_bhs;
};

// LDS bytes of the dK/dV workgroup: NW private rings of two stages of Q + dO and of (lse, delta) rows
template <int DH, int NW> constexpr int suffix_smem_bytes() {
    constexpr int ring = NW * (2 * 2 * 32 * DH * 2 + 2 * 256), epi = NW * 32 * (DH + 4) * 4;
    return ring > epi ? ring : epi;
}

// The work of workgroup `wg_id` of xcd_grid(B*H, ceil(T/32)); `smem` = suffix_smem_bytes<DH, NW>() bytes.
// OWN_DELTA: delta of the positions [P, own_end) -- the slice's own and those of the slices whose dQ launch may still
// be running -- is not read from a.delta but taken here from dO and the attention output, into `own`
// (ceil((own_end - P) / 32) * 32 floats of LDS).
template <typename T, int DH, int NW, bool OWN_DELTA>
__device__ __forceinline__ void attn_suffix_dkdv_body(const SuffixArgs& a, unsigned char* smem, float* own, int wg_id) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "direct-to-LDS kernels are for fp16 / bf16");
    constexpr int NDB = DH / 32, NKS = DH / 16;
    constexpr int TILE = 32 * DH;                       // elements of one Q or dO tile
    constexpr int CPR = DH / 8;
    constexpr int NLD = 32 * CPR / 64;
    constexpr int NLOAD = 2 * NLD + 1;                  // Q, dO and the stats row
    static_assert(NLOAD <= 63, "too many loads in flight for vmcnt");
    constexpr int WAVE_RING = 2 * 2 * TILE * 2;         // bytes: two stages of Q + dO
    constexpr int STAT_BYTES = 2 * 256;                 // per wave: two stages of 32 lse + 32 delta
    constexpr int EPI_LD = DH + 4;

    const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5, li = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int bh, kblk;
    if (!xcd_map(a.B * a.H, bh, kblk, wg_id)) return;
    const int b = bh / a.H, h = bh - b * a.H;
    const int P = a.P, S = a.P + a.T, Lq = a.Lq;
    const long EE = (long)a.H * DH;
    const int key0 = P + kblk * 32;
    const int key = key0 + li;
    const int nqb = (Lq - key0 + 31) / 32;              // query blocks start at the key block's position
    const int tpw = (nqb + NW - 1) / NW;
    const int j_beg = wave * tpw, j_end = min(nqb, j_beg + tpw);
    const int nt = max(j_end - j_beg, 0);

    T* ring = reinterpret_cast<T*>(smem) + wave * (WAVE_RING / 2);
    const unsigned ring_lds = lds_addr(smem) + wave * WAVE_RING;
    const float* sstat = reinterpret_cast<const float*>(smem + NW * WAVE_RING + wave * STAT_BYTES);
    const unsigned stat_lds = lds_addr(smem) + NW * WAVE_RING + wave * STAT_BYTES;

    const T* pkm[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) pkm[ks] = ring + km_offset<T, DH>(li, ks * 16, lane);
    const T* ptr0[NDB];
    const T* ptr1[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        int o0, o1;
        tr_offsets<T, DH, true>(0, db * 32, lane, o0, o1);
        ptr0[db] = ring + o0;
        ptr1[db] = ring + o1;
    }
    unsigned qoff[NLD], dooff[NLD];
    const unsigned ldo_bytes = (unsigned)((long)a.B * EE * 2);
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int p = i * 64 + lane;
        const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
        qoff[i] = (unsigned)(r * DH * 2 + lc * 16);
        dooff[i] = (unsigned)(r * ldo_bytes + lc * 16);
    }
    const char* Qb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.q) + (long)bh * a.q_bhs));
    const char* dOb = uniform_ptr(reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.d_o) + (long)b * EE + (long)h * DH));
    const float* statb = (g == 0 ? a.lse : a.delta) + (long)bh * a.st_bhs;   // lanes 0-31 fetch lse, 32-63 delta

    auto issue = [&](int stage, int j) {
        // positions at or past q_end are clamped to q_end - 1: finite data whose P and dS are forced to zero
        const unsigned dst = ring_lds + (unsigned)(stage * 2 * TILE * 2);
        const int row0 = key0 + j * 32;
        if (row0 + 32 <= Lq) {
            const char* sq = Qb + (long)row0 * (DH * 2);
            const char* sd = dOb + (long)row0 * ldo_bytes;
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(qoff[i], sq, dst + i * 1024);
#pragma unroll
            for (int i = 0; i < NLD; ++i) dma16_saddr_lds(dooff[i], sd, dst + TILE * 2 + i * 1024);
        } else {
            const int last = Lq - 1;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                dma16_saddr_lds((unsigned)(min(row0 + r, last) * DH * 2 + lc * 16), Qb, dst + i * 1024);
            }
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int p = i * 64 + lane;
                const int r = p / CPR, lc = (p % CPR) ^ swz16<DH>(r);
                dma16_saddr_lds((unsigned)(min(row0 + r, last) * ldo_bytes + lc * 16), dOb, dst + TILE * 2 + i * 1024);
            }
        }
        dma4(statb + min(row0 + li, Lq - 1), stat_lds + stage * 256);
    };

    float16v dk[NDB], dv[NDB];
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[db][r] = 0.f; dv[db][r] = 0.f; }

    // the first tile's loads go out before the key rows are asked for, so that the two round trips overlap
    // (vector-memory operations complete in issue order: the first wait in the loop covers both)
    if (nt > 0) issue(0, j_beg);
    typename E::opnd_t kreg[NKS], vreg[NKS];
    load_row_operands<T, DH>(kreg, reinterpret_cast<const T*>(a.kc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);
    load_row_operands<T, DH>(vreg, reinterpret_cast<const T*>(a.vc) + ((long)bh * a.cache_rows + key) * DH, key < S, g);
    if constexpr (OWN_DELTA) {
        // delta = rowsum(dO * O) of the positions [key0, own_end), 32 positions per wave and pass: lane (li, g)
        // takes half g of position li's row, as the dQ kernel does for its own rows
        for (int blk = wave; key0 + blk * 32 < a.own_end; blk += NW) {
            const int t = key0 + blk * 32 + li;
            typename E::opnd_t oreg[NKS], doreg[NKS];
            load_row_operands<T, DH>(oreg, reinterpret_cast<const T*>(a.o_all) + ((long)t * a.B + b) * EE + (long)h * DH, t < a.own_end, g);
            load_row_operands<T, DH>(doreg, reinterpret_cast<const T*>(a.d_o) + ((long)t * a.B + b) * EE + (long)h * DH, t < a.own_end, g);
            float sum = 0.f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const T* x = reinterpret_cast<const T*>(&oreg[ks]);
                const T* y = reinterpret_cast<const T*>(&doreg[ks]);
#pragma unroll
                for (int e = 0; e < 8; ++e) sum = fmaf(E::to_float(x[e]), E::to_float(y[e]), sum);
            }
            sum += __shfl_xor(sum, 32, 64);
            if (g == 0) own[blk * 32 + li] = sum;
        }
        __syncthreads();
    }

    auto step = [&](auto stage_c, int it) {
        constexpr int s = decltype(stage_c)::value;
        if (it + 1 < nt) {
            issue(s ^ 1, j_beg + it + 1);
            wait_vmcnt<NLOAD>();
        } else {
            wait_vmcnt<0>();
        }
        constexpr int so = s * 2 * TILE;
        const int t0 = key0 + (j_beg + it) * 32;        // first query position of the block
        typename E::opnd_t qop[NKS], doop[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            qop[ks] = load_km<T>(pkm[ks] + so);
            doop[ks] = load_km<T>(pkm[ks] + so + TILE);
        }
        float4 l4[4], d4[4];
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
            l4[jq] = *reinterpret_cast<const float4*>(sstat + s * 64 + 8 * jq + 4 * g);
            d4[jq] = *reinterpret_cast<const float4*>(sstat + s * 64 + 32 + 8 * jq + 4 * g);
        }
        if constexpr (OWN_DELTA) {
            if (t0 < a.own_end) {           // wave-uniform: the block has positions whose delta is taken here
#pragma unroll
                for (int jq = 0; jq < 4; ++jq) {
                    const int rel = t0 - key0 + 8 * jq + 4 * g;     // position - key0 of the float4's first entry
                    if (t0 + 8 * jq + 4 * g + 0 < a.own_end) d4[jq].x = own[rel + 0];
                    if (t0 + 8 * jq + 4 * g + 1 < a.own_end) d4[jq].y = own[rel + 1];
                    if (t0 + 8 * jq + 4 * g + 2 < a.own_end) d4[jq].z = own[rel + 2];
                    if (t0 + 8 * jq + 4 * g + 3 < a.own_end) d4[jq].w = own[rel + 3];
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        float16v sacc, pacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; pacc[r] = 0.f; }
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            sacc = E::mfma(qop[ks], kreg[ks], sacc);
            pacc = E::mfma(doop[ks], vreg[ks], pacc);
        }
        // wave-uniform: every (query, key) pair of the block is visible and in range
        const bool all_visible = (t0 + 32 <= Lq) && (key0 + 31 <= t0) && (key0 + 32 <= S);
        float pv[16], dsv[16];
        if (all_visible) {
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const float lv[4] = {l4[jq].x, l4[jq].y, l4[jq].z, l4[jq].w};
                const float dl[4] = {d4[jq].x, d4[jq].y, d4[jq].z, d4[jq].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 4 * jq + e;
                    const float p = fast_exp2((sacc[j] - lv[e]) * kLog2e);
                    pv[j] = p;
                    dsv[j] = p * (pacc[j] - dl[e]);
                }
            }
        } else {
#pragma unroll
            for (int jq = 0; jq < 4; ++jq) {
                const float lv[4] = {l4[jq].x, l4[jq].y, l4[jq].z, l4[jq].w};
                const float dl[4] = {d4[jq].x, d4[jq].y, d4[jq].z, d4[jq].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 4 * jq + e;
                    const int t = t0 + 8 * jq + 4 * g + e;
                    const bool vis = (t < Lq) && (key <= t) && (key < S);
                    const float p = vis ? fast_exp2((sacc[j] - lv[e]) * kLog2e) : 0.f;
                    pv[j] = p;
                    dsv[j] = vis ? p * (pacc[j] - dl[e]) : 0.f;
                }
            }
        }
        uint4 pop[2], dsop[2];
        pop[0] = pack8<T>(pv); pop[1] = pack8<T>(pv + 8);
        dsop[0] = pack8<T>(dsv); dsop[1] = pack8<T>(dsv + 8);
        uint4 ado[2][NDB], aq[2][NDB];
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                ado[hs][db] = load_tr<T>(ptr0[db] + so + TILE + hs * 16 * DH, ptr1[db] + so + TILE + hs * 16 * DH);
                aq[hs][db] = load_tr<T>(ptr0[db] + so + hs * 16 * DH, ptr1[db] + so + hs * 16 * DH);
            }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                dv[db] = E::mfma(ado[hs][db], pop[hs], dv[db]);
                dk[db] = E::mfma(aq[hs][db], dsop[hs], dk[db]);
            }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    {
        int it = 0;
        for (; it + 1 < nt; it += 2) {
            step(std::integral_constant<int, 0>(), it);
            step(std::integral_constant<int, 1>(), it + 1);
        }
        if (it < nt) step(std::integral_constant<int, 0>(), it);
    }
    wait_vmcnt<0>();
    __syncthreads();       // every wave is done with its ring: the space is reused for the reduction

    float* ebuf = reinterpret_cast<float*>(smem);
    constexpr int CPT = 32 * DH / (NW * 64);
    static_assert(CPT % 4 == 0 && DH % CPT == 0, "bad reduction split");
    const int row = tid / (DH / CPT), c0 = (tid % (DH / CPT)) * CPT;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        acc_to_lds_rows<DH>(which == 0 ? dk : dv, ebuf + wave * 32 * EPI_LD, lane);
        __syncthreads();
        if (key0 + row < S) {
            T* dst = reinterpret_cast<T*>(a.dqkv) + ((long)(key0 + row - P) * a.B + b) * (3 * EE) + (long)h * 3 * DH +
                     (which + 1) * DH + c0;
#pragma unroll
            for (int c = 0; c < CPT; c += 4) {
                float4 acc4 = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    const float4 v = *reinterpret_cast<const float4*>(ebuf + (w * 32 + row) * EPI_LD + c0 + c);
                    acc4.x += v.x; acc4.y += v.y; acc4.z += v.z; acc4.w += v.w;
                }
                store4<T>(dst + c, acc4.x, acc4.y, acc4.z, acc4.w);
            }
        }
        __syncthreads();   // the buffer is rewritten by the next pass
    }
}

template <typename T, int DH, int NW>
__global__ __launch_bounds__(NW * 64) void attn_suffix_dkdv_kernel(SuffixArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char smem[suffix_smem_bytes<DH, NW>()];
    attn_suffix_dkdv_body<T, DH, NW, false>(a, smem, nullptr, blockIdx.x);
}

// dQ (+ delta) of a slice and the one-pass dK / dV of the same slice as ONE launch: workgroups [0, n_dq) do the
// work of attn_bwd_dq2_kernel, the others that of attn_suffix_dkdv_kernel, side by side on different CUs -- the dQ
// side streams the keys before the slice, the dK/dV side the queries after it, so the two loads are complementary
// and a call with few (batch, head) pairs fills twice as many CUs.  The dK/dV side does not wait for the delta
// that the dQ side writes: it takes delta of the positions [P, own_end) from dO and O itself (dynamic LDS:
// ceil((own_end - P) / 32) * 32 floats).  n_dq is a multiple of eight, so both sides keep the XCD placement of xcd_map.
template <typename T, int DH>
__global__ __launch_bounds__(256) void attn_bwd_fused_kernel(AttnArgs a, SuffixArgs sa, int n_dq) {
    constexpr int SM = dq2_smem_bytes<DH, 4>() > suffix_smem_bytes<DH, 4>() ? dq2_smem_bytes<DH, 4>() : suffix_smem_bytes<DH, 4>();
    __shared__ __attribute__((aligned(16))) unsigned char smem[SM];
    extern __shared__ __attribute__((aligned(16))) float own_delta[];
    if ((int)blockIdx.x < n_dq) attn_bwd_dq2_body<T, DH, 4>(a, smem, blockIdx.x);
    else attn_suffix_dkdv_body<T, DH, 4, true>(sa, smem, own_delta, (int)blockIdx.x - n_dq);
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
static constexpr int kNumCU = 256;

// head dimensions of the 16-bit kernels with direct global->LDS loads; the others run, in every dtype, on the
// register-staged kernels, whose LDS tiles pad the head dimension to whole 32-column blocks
static inline bool tiled16(int head_dim) { return head_dim == 64 || head_dim == 128; }
static inline bool known_head_dim(int hd) { return hd == 16 || hd == 32 || hd == 64 || hd == 80 || hd == 96 || hd == 128; }

// calls f(std::integral_constant<int, hd>) for a known head dimension
template <typename F> static void for_head_dim(int hd, F&& f) {
    switch (hd) {
    case 16: f(std::integral_constant<int, 16>()); break;
    case 32: f(std::integral_constant<int, 32>()); break;
    case 64: f(std::integral_constant<int, 64>()); break;
    case 80: f(std::integral_constant<int, 80>()); break;
    case 96: f(std::integral_constant<int, 96>()); break;
    default: f(std::integral_constant<int, 128>()); break;
    }
}

static int validate_attn(const tp_attn_desc* d, bool bwd) {
    const char* who = bwd ? "tp_attn_prefix_bwd" : "tp_attn_prefix_fwd";
    if (!d) { set_error("%s: null descriptor", who); return TP_ERR_ARG; }
    if (d->dtype < TP_F32 || d->dtype > TP_BF16) { set_error("%s: bad dtype %d", who, d->dtype); return TP_ERR_ARG; }
    if (!known_head_dim(d->head_dim)) { set_error("%s: head_dim %d not supported (16, 32, 64, 80, 96 or 128)", who, d->head_dim); return TP_ERR_UNSUPPORTED; }
    if (d->batch <= 0 || d->heads <= 0 || d->T <= 0 || d->cache_len < 0) { set_error("%s: bad geometry B=%d H=%d T=%d P=%d", who, d->batch, d->heads, d->T, d->cache_len); return TP_ERR_ARG; }
    if ((long)d->cache_len + d->T > d->cache_rows) { set_error("%s: slice [%d, %d) does not fit a cache of %ld rows", who, d->cache_len, d->cache_len + d->T, (long)d->cache_rows); return TP_ERR_ARG; }
    if (!d->q || !d->k_cache || !d->v_cache || !d->o || !d->lse) { set_error("%s: null tensor", who); return TP_ERR_ARG; }
    if (((uintptr_t)d->q | (uintptr_t)d->k_cache | (uintptr_t)d->v_cache | (uintptr_t)d->o) & 15) { set_error("%s: tensors must be 16-byte aligned", who); return TP_ERR_ARG; }
    if (bwd) {
        if (!d->d_o || !d->delta || !d->dqkv) { set_error("%s: null gradient tensor", who); return TP_ERR_ARG; }
        if (((uintptr_t)d->d_o | (uintptr_t)d->dqkv | (uintptr_t)d->dk_cache | (uintptr_t)d->dv_cache) & 15) { set_error("%s: tensors must be 16-byte aligned", who); return TP_ERR_ARG; }
        if (!d->dq_only && (d->cache_len > 0 || d->has_incoming || d->zero_slice_rows) && (!d->dk_cache || !d->dv_cache)) { set_error("%s: gradient caches required", who); return TP_ERR_ARG; }
        if (d->grad_cache_dtype != d->dtype && d->grad_cache_dtype != TP_F32) { set_error("%s: grad_cache_dtype must be dtype or fp32", who); return TP_ERR_ARG; }
    }
    return TP_OK;
}

struct FwdPlan { int nw, bn, nsplit, qblocks; };

static FwdPlan plan_fwd(const tp_attn_desc* d) {
    FwdPlan p;
    if (d->dtype != TP_F32 && tiled16(d->head_dim)) {
        // 16-bit: one workgroup per 32 queries whose four waves split the key range and merge in LDS
        // slices of 64 queries and more: workgroups of 64 queries (attn_fwd3_kernel; p.bn = 64); reserved2 bit 3
        // forces the 32-query workgroups
        // -- when the pairs still give the chip enough workgroups (measured: ahead from 160 on, 5 to 20 %; behind
        // at 64 to 120, where the 32-query form has twice the workgroups and eight waves each); bit 4 forces them
        const bool pairs = d->T >= 64 && !(d->reserved2 & 8) &&
                           ((long)d->batch * d->heads * ((d->T + 63) / 64) >= 160 || (d->reserved2 & 16));
        p.nw = 0; p.bn = 32; p.nsplit = 1; p.qblocks = pairs ? (d->T + 63) / 64 : (d->T + 31) / 32;
        // A call with so few query blocks that over half of the CUs would get no workgroup, and a key range long
        // enough to share (16 tiles of 32 keys per share), spreads each block's keys over as many workgroups as fit
        // the chip; they leave fp32 partials in the workspace and the merge launch weighs them together.  Measured
        // at 96 (batch, head) pairs of 32 queries: 28.4 against 31.1 us at 2048 keys, nothing gained below 1024.
        const long wgs = (long)d->batch * d->heads * p.qblocks;
        const int ntiles = (d->cache_len + d->T + 31) / 32;
        if (d->reserved & 0xff) {
            p.nsplit = (d->reserved & 0xff) > 16 ? 16 : (d->reserved & 0xff);
        } else if (wgs * 5 <= kNumCU * 2) {
            int ns = (int)(kNumCU / wgs);
            if (ns > ntiles / 16) ns = ntiles / 16;
            if (ns > 8) ns = 8;
            if (ns >= 2) p.nsplit = ns;
        }
        // bn doubles as the wave count of this kernel: 8 = eight waves with one tile buffer each, faster
        // from about twenty key tiles on (measured: 19 against 24 us at 2048 keys, 7.9 against 7.6 us at 256);
        // reserved2 bit 1 forces it, bit 2 forces four waves
        if (((long)d->cache_len + d->T >= 640 || (d->reserved2 & 2)) && !(d->reserved2 & 4)) p.bn = 8;
        if (pairs) p.bn = 64;
        return p;
    }
    p.nw = d->T > 64 ? 4 : (d->T > 32 ? 2 : 1);
    // few (batch, head) pairs: 64-row workgroups give twice as many of them
    if (p.nw == 4 && (long)((d->T + 127) / 128) * d->batch * d->heads < kNumCU / 2) p.nw = 2;
    p.bn = p.nw == 1 ? 32 : 64;
    p.qblocks = (d->T + 32 * p.nw - 1) / (32 * p.nw);
    long waves = (long)p.qblocks * d->batch * d->heads * p.nw;
    int ntiles_min = (d->cache_len + (d->T < 32 * p.nw ? d->T : 32 * p.nw) + p.bn - 1) / p.bn;  // first q block
    int ns = 1;
    if (waves < 4L * kNumCU) {
        ns = (int)((4L * kNumCU + waves - 1) / waves);
        int cap = ntiles_min / 2;  // at least two tiles per split
        if (ns > cap) ns = cap;
        if (ns > 32) ns = 32;
        if (ns < 1) ns = 1;
    }
    if (d->reserved & 0xff) ns = d->reserved & 0xff;
    p.nsplit = ns;
    return p;
}

static AttnArgs make_args(const tp_attn_desc* d) {
    AttnArgs a;
    a.q = d->q; a.kc = d->k_cache; a.vc = d->v_cache; a.o = d->o; a.lse = d->lse;
    a.d_o = d->d_o; a.delta = d->delta; a.dqkv = d->dqkv; a.gk = d->dk_cache; a.gv = d->dv_cache;
    a.B = d->batch; a.H = d->heads; a.T = d->T; a.P = d->cache_len; a.cache_rows = d->cache_rows;
    a.nsplit = 1; a.part_o = nullptr; a.part_lse = nullptr;
    a.accumulate_prefix = d->accumulate_prefix; a.has_incoming = d->has_incoming;
    a.zero_slice_rows = d->zero_slice_rows; a.qscale = d->q_scale;
    a.dq_only = d->dq_only;
    a.q_bhs = (d->q_bh_rows > 0 ? d->q_bh_rows : (long)d->T) * d->head_dim;
    a.st_bhs = d->stat_bh_rows > 0 ? d->stat_bh_rows : (long)d->T;
    return a;
}

template <typename T, int DH>
static void launch_fwd(const FwdPlan& p, const AttnArgs& a, hipStream_t s) {
    dim3 grid(p.qblocks, a.B * a.H, p.nsplit);
    if constexpr (sizeof(T) == 2 && (DH == 64 || DH == 128)) {
        const dim3 g2(xcd_grid(a.B * a.H, (a.T + 31) / 32), p.nsplit);
        if (p.bn == 64) attn_fwd3_kernel<T, DH, 4><<<dim3(xcd_grid(a.B * a.H, (a.T + 63) / 64), p.nsplit), 256, 0, s>>>(a);
        else if (p.bn == 8) attn_fwd2_kernel<T, DH, 8, 1><<<g2, 512, 0, s>>>(a);
        else attn_fwd2_kernel<T, DH, 4><<<g2, 256, 0, s>>>(a);
    } else {
        if (p.nw == 4) attn_fwd_kernel<T, DH, 4, 64><<<grid, 256, 0, s>>>(a);
        else if (p.nw == 2) attn_fwd_kernel<T, DH, 2, 64><<<grid, 128, 0, s>>>(a);
        else attn_fwd_kernel<T, DH, 1, 32><<<grid, 64, 0, s>>>(a);
    }
    if (p.nsplit > 1) {
        long rows = (long)a.B * a.H * a.T;
        attn_fwd_merge_kernel<T, DH><<<(unsigned)((rows + 3) / 4), 256, 0, s>>>(a);
    }
}

template <typename T, typename GT, int DH>
static void launch_bwd(const AttnArgs& a, hipStream_t s) {
    const int S = a.P + a.T;
    long rows = (long)a.T * a.B * a.H;
    constexpr bool kTiled16 = sizeof(T) == 2 && (DH == 64 || DH == 128);
    if constexpr (kTiled16) {
        // dQ first: it also leaves delta for the dK/dV kernel
        attn_bwd_dq2_kernel<T, DH, 4><<<xcd_grid(a.B * a.H, (a.T + 31) / 32), 256, 0, s>>>(a);
    } else {
        attn_bwd_delta_kernel<T, DH><<<(unsigned)((rows + 3) / 4), 256, 0, s>>>(a);
    }
    if (!a.dq_only) {
        // dK/dV: 4 waves x 32 keys per workgroup when that still fills the chip, else 2 or 1
        long bh = (long)a.B * a.H;
        int nw = 4;
        if (((S + 127) / 128) * bh < 2L * kNumCU) nw = 2;
        if (((S + 63) / 64) * bh < 2L * kNumCU) nw = 1;
        dim3 grid((S + 32 * nw - 1) / (32 * nw), (unsigned)bh);
        if (kTiled16 && a.T <= kMaxTLds) {
            if constexpr (kTiled16) {
                const size_t dyn = (size_t)2 * ((a.T + 31) / 32) * 32 * sizeof(float);
                const unsigned g2 = xcd_grid((int)bh, (int)grid.x);
                if (nw == 4) attn_bwd_dkdv2_kernel<T, GT, DH, 4, 3><<<g2, 256, dyn, s>>>(a);
                else if (nw == 2) attn_bwd_dkdv2_kernel<T, GT, DH, 2, 3><<<g2, 128, dyn, s>>>(a);
                else attn_bwd_dkdv2_kernel<T, GT, DH, 1, 3><<<g2, 64, dyn, s>>>(a);
            }
        } else {
            if (nw == 4) attn_bwd_dkdv_kernel<T, GT, DH, 4><<<grid, 256, 0, s>>>(a);
            else if (nw == 2) attn_bwd_dkdv_kernel<T, GT, DH, 2><<<grid, 128, 0, s>>>(a);
            else attn_bwd_dkdv_kernel<T, GT, DH, 1><<<grid, 64, 0, s>>>(a);
        }
    }
    if constexpr (!kTiled16) {
        int nw = a.T > 64 ? 4 : (a.T > 32 ? 2 : 1);
        if (nw == 4 && (long)((a.T + 127) / 128) * a.B * a.H < kNumCU / 2) nw = 2;
        dim3 grid((a.T + 32 * nw - 1) / (32 * nw), a.B * a.H);
        {
            if (nw == 4) attn_bwd_dq_kernel<T, DH, 4, 64><<<grid, 256, 0, s>>>(a);
            else if (nw == 2) attn_bwd_dq_kernel<T, DH, 2, 64><<<grid, 128, 0, s>>>(a);
            else attn_bwd_dq_kernel<T, DH, 1, 32><<<grid, 64, 0, s>>>(a);
        }
    }
}

template <typename T>
static void dispatch_fwd(int hd, const FwdPlan& p, const AttnArgs& a, hipStream_t s) {
    for_head_dim(hd, [&](auto dh) { launch_fwd<T, decltype(dh)::value>(p, a, s); });
}

template <typename T>
static void dispatch_bwd(int hd, bool f32grad, const AttnArgs& a, hipStream_t s) {
    if (sizeof(T) == 4 || f32grad) for_head_dim(hd, [&](auto dh) { launch_bwd<T, float, decltype(dh)::value>(a, s); });
    else for_head_dim(hd, [&](auto dh) { launch_bwd<T, T, decltype(dh)::value>(a, s); });
}

}  // namespace tp

extern "C" size_t tp_attn_fwd_workspace_bytes(const tp_attn_desc* d) {
    if (!d || d->T <= 0 || d->batch <= 0 || d->heads <= 0) return 0;
    tp::FwdPlan p = tp::plan_fwd(d);
    if (p.nsplit <= 1) return 0;
    size_t rows = (size_t)p.nsplit * d->batch * d->heads * d->T;
    return rows * d->head_dim * sizeof(float) + rows * sizeof(float);
}

extern "C" int tp_attn_prefix_fwd(const tp_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace tp;
    int rc = validate_attn(d, false);
    if (rc != TP_OK) return rc;
    FwdPlan p = plan_fwd(d);
    AttnArgs a = make_args(d);
    if (p.nsplit > 1) {
        size_t need = tp_attn_fwd_workspace_bytes(d);
        if (!workspace || workspace_bytes < need) { set_error("tp_attn_prefix_fwd: workspace of %zu bytes needed, %zu given", need, workspace_bytes); return TP_ERR_WORKSPACE; }
        if ((uintptr_t)workspace & 15) { set_error("tp_attn_prefix_fwd: workspace must be 16-byte aligned"); return TP_ERR_ARG; }
        size_t rows = (size_t)p.nsplit * d->batch * d->heads * d->T;
        a.nsplit = p.nsplit;
        a.part_o = reinterpret_cast<float*>(workspace);
        a.part_lse = a.part_o + rows * d->head_dim;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (d->dtype) {
    case TP_F32: dispatch_fwd<float>(d->head_dim, p, a, s); break;
    case TP_F16: dispatch_fwd<f16>(d->head_dim, p, a, s); break;
    default: dispatch_fwd<bf16>(d->head_dim, p, a, s); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("tp_attn_prefix_fwd: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

extern "C" size_t tp_attn_bwd_workspace_bytes(const tp_attn_desc* d) { (void)d; return 0; }

extern "C" int tp_attn_prefix_bwd(const tp_attn_desc* d, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace tp;
    (void)workspace; (void)workspace_bytes;
    int rc = validate_attn(d, true);
    if (rc != TP_OK) return rc;
    AttnArgs a = make_args(d);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool f32grad = d->grad_cache_dtype == TP_F32;
    switch (d->dtype) {
    case TP_F32: dispatch_bwd<float>(d->head_dim, true, a, s); break;
    case TP_F16: dispatch_bwd<f16>(d->head_dim, f32grad, a, s); break;
    default: dispatch_bwd<bf16>(d->head_dim, f32grad, a, s); break;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("tp_attn_prefix_bwd: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    if (d->colsum_dqkv_acc && !d->dq_only) {
        return tp_colsum_acc(d->dqkv, 3L * d->heads * d->head_dim, d->colsum_dqkv_acc, d->T * d->batch,
                             3 * d->heads * d->head_dim, d->dtype, stream);
    }
    return TP_OK;
}

static int validate_suffix(const tp_attn_suffix_desc* d, const char* who);
static tp::SuffixArgs make_suffix_args(const tp_attn_suffix_desc* d);

extern "C" int tp_attn_suffix_dkdv(const tp_attn_suffix_desc* d, void* stream) {
    using namespace tp;
    const char* who = "tp_attn_suffix_dkdv";
    int rc = validate_suffix(d, who);
    if (rc != TP_OK) return rc;
    SuffixArgs a = make_suffix_args(d);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const unsigned grid = xcd_grid(d->batch * d->heads, (d->key_count + 31) / 32);
    if (d->dtype == TP_F16) {
        if (d->head_dim == 64) attn_suffix_dkdv_kernel<f16, 64, 4><<<grid, 256, 0, s>>>(a);
        else attn_suffix_dkdv_kernel<f16, 128, 4><<<grid, 256, 0, s>>>(a);
    } else {
        if (d->head_dim == 64) attn_suffix_dkdv_kernel<bf16, 64, 4><<<grid, 256, 0, s>>>(a);
        else attn_suffix_dkdv_kernel<bf16, 128, 4><<<grid, 256, 0, s>>>(a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", who, hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

extern "C" int tp_attn_bwd_fused(const tp_attn_desc* d, const tp_attn_suffix_desc* sd, const void* o_all, int own_delta_end,
                                 void* stream) {
    using namespace tp;
    const char* who = "tp_attn_bwd_fused";
    int rc = validate_attn(d, true);
    if (rc != TP_OK) return rc;
    rc = validate_suffix(sd, who);
    if (rc != TP_OK) return rc;
    if (!d->dq_only) { set_error("%s: the backward descriptor must have dq_only set (no gradient caches on this path)", who); return TP_ERR_ARG; }
    if (d->dtype != sd->dtype || d->batch != sd->batch || d->heads != sd->heads || d->head_dim != sd->head_dim ||
        d->cache_len != sd->key_begin || d->T != sd->key_count || d->dqkv != sd->dqkv || d->k_cache != sd->k_cache ||
        d->v_cache != sd->v_cache || (long)d->cache_rows != (long)sd->cache_rows) {
        set_error("%s: the two descriptors do not describe the same slice (dtype, batch, heads, head_dim, cache_len = key_begin, "
                  "T = key_count, dqkv, caches)", who);
        return TP_ERR_ARG;
    }
    if (!o_all || ((uintptr_t)o_all & 15)) { set_error("%s: o_all must be a 16-byte aligned device pointer", who); return TP_ERR_ARG; }
    if (own_delta_end < sd->key_begin + sd->key_count || own_delta_end > sd->q_end) {
        set_error("%s: own_delta_end %d outside [key_begin + key_count, q_end] = [%d, %d]", who, own_delta_end,
                  sd->key_begin + sd->key_count, sd->q_end);
        return TP_ERR_ARG;
    }
    const int own_len = own_delta_end - sd->key_begin;
    if (own_len > kMaxTLds) { set_error("%s: delta of up to %d positions is taken in the launch (got %d); use the two separate calls", who, kMaxTLds, own_len); return TP_ERR_UNSUPPORTED; }
    AttnArgs a = make_args(d);
    SuffixArgs sa = make_suffix_args(sd);
    sa.o_all = o_all;
    sa.own_end = own_delta_end;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const int n_dq = (int)xcd_grid(d->batch * d->heads, (d->T + 31) / 32);
    const unsigned grid = (unsigned)n_dq + xcd_grid(d->batch * d->heads, (d->T + 31) / 32);
    const size_t dyn = (size_t)((own_len + 31) / 32) * 32 * sizeof(float);
    if (d->dtype == TP_F16) {
        if (d->head_dim == 64) attn_bwd_fused_kernel<f16, 64><<<grid, 256, dyn, s>>>(a, sa, n_dq);
        else attn_bwd_fused_kernel<f16, 128><<<grid, 256, dyn, s>>>(a, sa, n_dq);
    } else {
        if (d->head_dim == 64) attn_bwd_fused_kernel<bf16, 64><<<grid, 256, dyn, s>>>(a, sa, n_dq);
        else attn_bwd_fused_kernel<bf16, 128><<<grid, 256, dyn, s>>>(a, sa, n_dq);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", who, hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

static int validate_suffix(const tp_attn_suffix_desc* d, const char* who) {
    using namespace tp;
    if (!d) { set_error("%s: null descriptor", who); return TP_ERR_ARG; }
    if (d->dtype != TP_F16 && d->dtype != TP_BF16) { set_error("%s: dtype %d not supported (fp16 / bf16)", who, d->dtype); return TP_ERR_UNSUPPORTED; }
    if (d->head_dim != 64 && d->head_dim != 128) { set_error("%s: head_dim %d not supported (64 or 128)", who, d->head_dim); return TP_ERR_UNSUPPORTED; }
    if (d->batch <= 0 || d->heads <= 0 || d->key_begin < 0 || d->key_count <= 0 || d->q_end < d->key_begin + d->key_count) {
        set_error("%s: bad geometry B=%d H=%d keys [%d, +%d) q_end=%d", who, d->batch, d->heads, d->key_begin, d->key_count, d->q_end);
        return TP_ERR_ARG;
    }
    if ((long)d->key_begin + d->key_count > d->cache_rows || d->q_end > d->q_bh_rows || d->q_end > d->stat_bh_rows) {
        set_error("%s: positions up to %d do not fit cache_rows %ld / q_bh_rows %ld / stat_bh_rows %ld", who, d->q_end,
                  (long)d->cache_rows, (long)d->q_bh_rows, (long)d->stat_bh_rows);
        return TP_ERR_ARG;
    }
    if (!d->k_cache || !d->v_cache || !d->q_all || !d->d_o_all || !d->lse_all || !d->delta_all || !d->dqkv) { set_error("%s: null tensor", who); return TP_ERR_ARG; }
    if (((uintptr_t)d->k_cache | (uintptr_t)d->v_cache | (uintptr_t)d->q_all | (uintptr_t)d->d_o_all | (uintptr_t)d->dqkv) & 15) { set_error("%s: tensors must be 16-byte aligned", who); return TP_ERR_ARG; }
    return TP_OK;
}

static tp::SuffixArgs make_suffix_args(const tp_attn_suffix_desc* d) {
    tp::SuffixArgs a;
    a.kc = d->k_cache; a.vc = d->v_cache; a.q = d->q_all; a.d_o = d->d_o_all;
    a.lse = d->lse_all; a.delta = d->delta_all; a.dqkv = d->dqkv; a.o_all = nullptr; a.own_end = 0;
    a.B = d->batch; a.H = d->heads; a.P = d->key_begin; a.T = d->key_count; a.Lq = d->q_end;
    a.cache_rows = d->cache_rows; a.q_bhs = d->q_bh_rows * d->head_dim; a.st_bhs = d->stat_bh_rows;
    return a;
}
