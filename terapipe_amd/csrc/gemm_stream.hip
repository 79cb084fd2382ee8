// Weight-streaming GEMM for the slice linears whose activation has few rows (NT forward Y = X W^T and NN data
// gradient dX = dY W, 16-bit, M up to a few hundred): such a product is bound by how fast the weight streams
// from HBM, and a CU streams only as fast as (bytes it has in flight) / (memory latency).
//
// A workgroup owns ALL rows of a row tile (BM = 64 * RB, up to 256: the whole slice) and BN columns, so the
// weight passes through exactly one workgroup per row tile, and it keeps two rings of LDS tiles of DIFFERENT
// depth: a shallow one for the activation tile (BM x 64, re-read by every workgroup, served by L2) and a deep one
// for the weight tile (BN x 64, from HBM) -- a uniform ring would spend most of the 160 KB on activation
// stages.  A wave's vector-memory operations complete in issue order, so the two rings are fed by different
// waves: the first half of the waves issues only activation tiles, the second half only weight tiles, each
// with its own prefetch distance and its own s_waitcnt count; one s_barrier per k-tile joins them.
//
// Compute: v_mfma_f32_16x16x32 (16-row granularity: 160 = 10 blocks, no padding to 32).  Wave w owns rows
// [(w % 4) * RB * 16, +RB * 16) and the (w / 4)-th share of the column blocks; per 32 of k it fetches RB + CBW
// operand fragments for RB * CBW MFMAs.
#include "gemm_args.h"

namespace tp {

template <typename T, bool BKM, int RB, int CB, int WN, int AS, int BS>
__global__ __launch_bounds__(256 * WN) void gemm_stream_kernel(GemmArgs a) {
    static_assert(sizeof(T) == 2, "16-bit only");
    static_assert(CB % WN == 0, "column blocks split evenly over the wave columns");
    constexpr int NW = 4 * WN;                 // waves
    constexpr int NLA = NW / 2;                // waves that load activation tiles; the others load weight tiles
    constexpr int BM = 64 * RB, BN = 16 * CB, BK = 64;
    constexpr int CBW = CB / WN, BNW = 16 * CBW;
    constexpr int A_ELEMS = BM * BK, B_ELEMS = BN * BK;
    constexpr int BR = BKM ? BN : BK, BC = BKM ? BK : BN;
    typedef ClampTileDma<T, BM, BK, NLA * 64, true, true> DA;
    typedef ClampTileDma<T, BR, BC, (NW - NLA) * 64, BKM, BKM> DB;
    constexpr int NA = DA::N, NB = DB::N;
    static_assert(NA * (AS - 1) <= 63 && NB * (BS - 1) <= 63, "too many loads in flight for vmcnt");
    constexpr int TILE_BYTES = (AS * A_ELEMS + BS * B_ELEMS) * 2;
    constexpr int SP = BNW + 4;                // fp32 pitch of a wave's 16-row epilogue strip
    constexpr int EPI_BYTES = NW * 16 * SP * 4;
    constexpr int SMEM_BYTES = TILE_BYTES > EPI_BYTES ? TILE_BYTES : EPI_BYTES;
    static_assert(SMEM_BYTES <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    T* tilesA = reinterpret_cast<T*>(smem);
    T* tilesB = tilesA + AS * A_ELEMS;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave & 3, wn = wave >> 2;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int kbeg = blockIdx.z * a.kper;
    const int kend = min(a.K, kbeg + a.kper);
    const int nk = (kend - kbeg) / BK;         // whole tiles only (the plan guarantees it)
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const bool role_a = wave_u < NLA;          // wave-uniform

    DA da;
    DB db;
    da.init(reinterpret_cast<const T*>(a.A), a.lda, m0, a.M, kbeg, BK, tid & (NLA * 64 - 1));
    db.init(reinterpret_cast<const T*>(a.B), a.ldb, n0, a.N, kbeg, BK, (tid - NLA * 64) & ((NW - NLA) * 64 - 1));
    const unsigned ldsA = lds_addr(tilesA), ldsB = lds_addr(tilesB);

    float4v acc[RB][CBW];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < CBW; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    // this lane's operand fetch offsets inside a tile (elements); a row block further down / another k-step of a
    // k-major tile is a compile-time distance away (the swizzle only looks at the low row bits)
    const int r16 = lane & 15, g4 = lane >> 4;
    int oa[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) oa[ks] = TileLayout<T, BK, true>::off(wm * RB * 16 + r16, ks * 32 + 8 * g4);
    int ob[BKM ? 2 : 2 * CBW];
    if constexpr (BKM) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) ob[ks] = TileLayout<T, BK, true>::off(wn * BNW + r16, ks * 32 + 8 * g4);
    } else {
        // k runs down the rows of the weight tile: two transpose reads per fragment, rows 8 * g4 + (p >> 2) and
        // four below, the 16 lanes of a group covering 4 rows x 16 columns
#pragma unroll
        for (int j = 0; j < CBW; ++j) {
            const int col = wn * BNW + j * 16 + 4 * (r16 & 3);
            const int row = 8 * g4 + (r16 >> 2);
            ob[2 * j] = TileLayout<T, BN>::off(row, col);
            ob[2 * j + 1] = TileLayout<T, BN>::off(row + 4, col);
        }
    }

    // prologue: each role fills its ring
    if (role_a) {
#pragma unroll
        for (int s = 0; s < AS - 1; ++s)
            if (s < nk) da.issue(ldsA + (unsigned)(s * A_ELEMS * 2), wave_u);
    } else {
#pragma unroll
        for (int s = 0; s < BS - 1; ++s)
            if (s < nk) db.issue(ldsB + (unsigned)(s * B_ELEMS * 2), wave_u - NLA);
    }

    int sa = 0, sb = 0;                         // ring slots of the current tile (wave-uniform)
    int fa = AS - 1, fb = BS - 1;               // ring slots the next issued tiles go to
    uint4 fra[2][RB], frb[2][CBW];
    for (int kt = 0; kt < nk; ++kt) {
        const bool more_a = kt + AS - 1 < nk, more_b = kt + BS - 1 < nk;
        if (role_a) {
            if (more_a) wait_vmcnt<NA * (AS - 2)>();
            else wait_vmcnt<0>();
        } else {
            if (more_b) wait_vmcnt<NB * (BS - 2)>();
            else wait_vmcnt<0>();
        }
        __builtin_amdgcn_s_barrier();           // tile kt is in LDS; nobody reads tile kt - 1 any more
        asm volatile("" ::: "memory");
        if (role_a) {
            if (more_a) da.issue(ldsA + (unsigned)(fa * A_ELEMS * 2), wave_u);
        } else {
            if (more_b) db.issue(ldsB + (unsigned)(fb * B_ELEMS * 2), wave_u - NLA);
        }
        const T* tA = tilesA + sa * A_ELEMS;
        const T* tB = tilesB + sb * B_ELEMS;
        auto fetch = [&](int ks, int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < RB; ++i) fra[buf][i] = load_km<T>(tA + oa[ks] + i * 16 * BK);
#pragma unroll
            for (int j = 0; j < CBW; ++j) {
                if constexpr (BKM) frb[buf][j] = load_km<T>(tB + ob[ks] + j * 16 * BK);
                else frb[buf][j] = load_tr<T>(tB + ob[2 * j] + ks * 32 * BN, tB + ob[2 * j + 1] + ks * 32 * BN);
            }
        };
        fetch(0, 0);
        __builtin_amdgcn_sched_barrier(0);
        fetch(1, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CBW; ++j) acc[i][j] = Mfma16x16x32<T>::run(fra[0][i], frb[0][j], acc[i][j]);
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int j = 0; j < CBW; ++j) acc[i][j] = Mfma16x16x32<T>::run(fra[1][i], frb[1][j], acc[i][j]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave's LDS reads of the tile are done
        sa = sa + 1 == AS ? 0 : sa + 1;
        sb = sb + 1 == BS ? 0 : sb + 1;
        fa = fa + 1 == AS ? 0 : fa + 1;
        fb = fb + 1 == BS ? 0 : fb + 1;
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // Epilogue: a wave passes its 16-row strips through LDS (rows 4 * g4 + r of a block sit in register r) so that a
    // lane ends up with 8 consecutive columns of a row: 16-byte stores and the vector epilogue.
    float* stage = reinterpret_cast<float*>(smem) + wave * 16 * SP;
    constexpr int CG = BNW / 8;                 // 8-column groups per strip row
    constexpr int ITEMS = 16 * CG;
    constexpr int NI = (ITEMS + 63) / 64;
    float csum[NI][8];
#pragma unroll
    for (int it = 0; it < NI; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) csum[it][e] = 0.f;
    static_for<RB>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
#pragma unroll
        for (int j = 0; j < CBW; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) stage[(4 * g4 + r) * SP + j * 16 + r16] = acc[i][j][r];
        __builtin_amdgcn_s_waitcnt(0xc07f);     // lgkmcnt(0): the strip is private to the wave
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < NI; ++it) {
            const int item = lane + 64 * it;
            if (ITEMS % 64 == 0 || item < ITEMS) {
                const int rr = item / CG, cg = item - rr * CG;
                const int row = m0 + (wm * RB + i) * 16 + rr;
                const int col0 = n0 + wn * BNW + cg * 8;
                float4 v0 = *reinterpret_cast<const float4*>(stage + rr * SP + cg * 8);
                float4 v1 = *reinterpret_cast<const float4*>(stage + rr * SP + cg * 8 + 4);
                if (row < a.M && col0 < a.N) {
                    if (a.nsplit > 1) {
                        float* dst = a.partial + ((long)blockIdx.z * a.M + row) * a.N + col0;
                        *reinterpret_cast<float4*>(dst) = v0;
                        *reinterpret_cast<float4*>(dst + 4) = v1;
                    } else {
                        float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                        epilogue_vec8<T>(a, row, col0, v);
#pragma unroll
                        for (int e = 0; e < 8; ++e) csum[it][e] += v[e];
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    });
    if (a.nsplit == 1 && a.colsum) {
#pragma unroll
        for (int it = 0; it < NI; ++it) {
            const int item = lane + 64 * it;
            const int cg = item % CG;
            const int col0 = n0 + wn * BNW + cg * 8;
            if ((ITEMS % 64 == 0 || item < ITEMS) && col0 < a.N) {
#pragma unroll
                for (int e = 0; e < 8; ++e) atomicAdd(a.colsum + col0 + e, csum[it][e]);
            }
        }
    }
}

// id -> (RB, CB, WN, AS, BS); ids are the tile-configuration numbers of the plan (gemm.hip kCfgs)
template <typename T, bool BKM>
static bool launch_stream_cfg(int cfg, dim3 grid, const GemmArgs& a, hipStream_t s) {
    switch (cfg) {
    case 21: gemm_stream_kernel<T, BKM, 3, 8, 1, 3, 5><<<grid, 256, 0, s>>>(a); return true;
    case 22: gemm_stream_kernel<T, BKM, 4, 8, 1, 3, 4><<<grid, 256, 0, s>>>(a); return true;
    case 23: gemm_stream_kernel<T, BKM, 4, 8, 1, 2, 6><<<grid, 256, 0, s>>>(a); return true;
    case 24: if constexpr (BKM) { gemm_stream_kernel<T, BKM, 3, 5, 1, 3, 8><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 25: if constexpr (BKM) { gemm_stream_kernel<T, BKM, 4, 5, 1, 3, 6><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 26: gemm_stream_kernel<T, BKM, 2, 8, 1, 3, 7><<<grid, 256, 0, s>>>(a); return true;
    case 27: gemm_stream_kernel<T, BKM, 4, 4, 1, 3, 8><<<grid, 256, 0, s>>>(a); return true;
    case 28: gemm_stream_kernel<T, BKM, 3, 4, 1, 3, 10><<<grid, 256, 0, s>>>(a); return true;
    case 29: gemm_stream_kernel<T, BKM, 4, 8, 2, 3, 4><<<grid, 512, 0, s>>>(a); return true;
    case 30: gemm_stream_kernel<T, BKM, 3, 8, 2, 3, 5><<<grid, 512, 0, s>>>(a); return true;
    case 31: gemm_stream_kernel<T, BKM, 3, 8, 4, 3, 5><<<grid, 1024, 0, s>>>(a); return true;
    case 32: gemm_stream_kernel<T, BKM, 4, 8, 4, 3, 4><<<grid, 1024, 0, s>>>(a); return true;
    case 33: gemm_stream_kernel<T, BKM, 3, 16, 4, 2, 3><<<grid, 1024, 0, s>>>(a); return true;
    case 34: gemm_stream_kernel<T, BKM, 4, 16, 4, 2, 3><<<grid, 1024, 0, s>>>(a); return true;
    case 35: gemm_stream_kernel<T, BKM, 2, 16, 4, 3, 3><<<grid, 1024, 0, s>>>(a); return true;
    case 36: gemm_stream_kernel<T, BKM, 1, 16, 4, 3, 4><<<grid, 1024, 0, s>>>(a); return true;
    case 37: gemm_stream_kernel<T, BKM, 2, 8, 4, 3, 7><<<grid, 1024, 0, s>>>(a); return true;
    case 38: gemm_stream_kernel<T, BKM, 1, 8, 4, 3, 8><<<grid, 1024, 0, s>>>(a); return true;
    case 39: gemm_stream_kernel<T, BKM, 2, 16, 2, 3, 3><<<grid, 512, 0, s>>>(a); return true;
    case 40: gemm_stream_kernel<T, BKM, 1, 16, 2, 3, 4><<<grid, 512, 0, s>>>(a); return true;
    default: return false;
    }
}

bool launch_gemm_stream(int cfg, int op, int dtype, dim3 grid, const GemmArgs& a, hipStream_t s) {
    if (dtype == TP_F32 || op == TP_GEMM_TN) return false;
    if (dtype == TP_F16) {
        return op == TP_GEMM_NT ? launch_stream_cfg<f16, true>(cfg, grid, a, s) : launch_stream_cfg<f16, false>(cfg, grid, a, s);
    }
    return op == TP_GEMM_NT ? launch_stream_cfg<bf16, true>(cfg, grid, a, s) : launch_stream_cfg<bf16, false>(cfg, grid, a, s);
}

}  // namespace tp
