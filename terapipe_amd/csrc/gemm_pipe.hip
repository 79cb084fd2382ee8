// The software-pipelined GEMM tiles (16 x 16 x 32 MFMA blocks, one wave per SIMD) and their launchers; a translation
// unit of its own so that it compiles beside gemm.hip.
#include "gemm_epilogue.h"

namespace tp {

// ---------------------------------------------------------------------------------------------
// Software-pipelined tall tile on 16 x 16 x 32 MFMA blocks, one wave per SIMD (four waves, accumulators in AGPRs).
// A k-tile of 64 is two sub-steps of 32.  While the MFMAs of a sub-step run, the operand fragments of the NEXT
// sub-step are fetched from LDS into the other register set, one fetch between every few MFMAs, front-loaded so
// that they have landed when the sub-step ends; the workgroup barrier sits in the MIDDLE of a k-tile: by then
// every wave has read the tile's second half into registers, so its buffer is free and the loads of the tile
// STAGES ahead are issued into it, spread over the second sub-step's MFMAs, and the next tile (which the barrier
// also proves landed) is fetched from during that sub-step.  No LDS or barrier latency stands between two MFMAs
// of a wave except the barrier itself.
// The blocks are 16 x 16 x 32 rather than 32 x 32 x 16: the same flops per cycle and, for a wave's tile, the same
// operand bytes from LDS per flop, but on operands with random bits the chip sustains more of them -- a loop of
// nothing but MFMAs runs at 2.0 against 1.6 PFLOP/s (2.4 for both on zeros).  They also cut a tile at 16 rows
// (192 = 2 x 96 rows).  Measured on the 13B slice shapes: 4 to 12 % under the 32 x 32 tiles' times.
// ---------------------------------------------------------------------------------------------
template <typename T, bool AKM, bool BKM, int BM, int BN, int WM, int WN, int STAGES, bool GROUPED = false>
__global__ __launch_bounds__(WM * WN * 64)
void gemm_pipe_kernel(typename std::conditional<GROUPED, GemmGroupArgs, GemmArgs>::type args) {
    int prob = 0, tile_x = blockIdx.x, tile_y = blockIdx.y, tile_z = blockIdx.z;
    if constexpr (GROUPED) {
        static_assert(kGroupMax == 4, "the selects below are written out for four problems");
        int first = 0, tx = args.tiles_x[0], ty = args.tiles_y[0];
        if (1 < args.n && (int)blockIdx.x >= args.first_tile[1]) { prob = 1; first = args.first_tile[1]; tx = args.tiles_x[1]; ty = args.tiles_y[1]; }
        if (2 < args.n && (int)blockIdx.x >= args.first_tile[2]) { prob = 2; first = args.first_tile[2]; tx = args.tiles_x[2]; ty = args.tiles_y[2]; }
        if (3 < args.n && (int)blockIdx.x >= args.first_tile[3]) { prob = 3; first = args.first_tile[3]; tx = args.tiles_x[3]; ty = args.tiles_y[3]; }
        xcd_tile((int)blockIdx.x - first, tx, ty, tile_x, tile_y);
    } else if (gridDim.z == 1) {
        xcd_tile((int)(blockIdx.y * gridDim.x + blockIdx.x), (int)gridDim.x, (int)gridDim.y, tile_x, tile_y);
    } else {
        xcd_tile3((int)((blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x), (int)gridDim.x, (int)gridDim.y,
                  (int)gridDim.z, tile_x, tile_y, tile_z);
    }
    const GemmArgs a = [&]() -> GemmArgs {
        if constexpr (GROUPED) {
            if (prob == 1) return args.g[1];
            if (prob == 2) return args.g[2];
            if (prob == 3) return args.g[3];
            return args.g[0];
        } else {
            return args;
        }
    }();
    static_assert(sizeof(T) == 2, "16-bit only");
    static_assert(WM * WN == 4, "one wave per SIMD");
    constexpr int NT = WM * WN * 64, BK = 64, KS = 32;
    constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
    static_assert(BM % (WM * 16) == 0 && BN % (WN * 16) == 0, "a wave's tile is whole 16 x 16 blocks");
    constexpr int NF = TM + TN, NM = TM * TN;
    constexpr int AR = AKM ? BM : BK, AC = AKM ? BK : BM;
    constexpr int BR = BKM ? BN : BK, BC = BKM ? BK : BN;
    constexpr int A_ELEMS = AR * AC, B_ELEMS = BR * BC;
    constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
    typedef ClampTileDma<T, AR, AC, NT, AKM, AKM> DA;
    typedef ClampTileDma<T, BR, BC, NT, BKM, BKM> DB;
    constexpr int NLOAD = DA::N + DB::N;
    static_assert(NLOAD * STAGES <= 63, "too many loads in flight for vmcnt (every buffer has a tile under way)");
    constexpr int TILE_BYTES = STAGES * STAGE_ELEMS * 2;
    constexpr int EPI_BYTES = WM * WN * 32 * 36 * 4;
    constexpr int SMEM_BYTES = TILE_BYTES > EPI_BYTES ? TILE_BYTES : EPI_BYTES;
    static_assert(SMEM_BYTES <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    T* tiles = reinterpret_cast<T*>(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int m0 = tile_y * BM, n0 = tile_x * BN;
    const int kbeg = tile_z * a.kper;
    const int kend = min(a.K, kbeg + a.kper);
    const int nk = (kend - kbeg) / BK;          // whole tiles only (the plan guarantees it)
    DA da;
    DB db;
    da.init(reinterpret_cast<const T*>(a.A), a.lda, m0, a.M, kbeg, BK, tid);
    db.init(reinterpret_cast<const T*>(a.B), a.ldb, n0, a.N, kbeg, BK, tid);
    const unsigned lds0 = lds_addr(smem);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);

    float4v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    constexpr int NPA = AKM ? 1 : 2, NPB = BKM ? 1 : 2;
    int oa[2][TM][NPA], ob[2][TN][NPB];        // [sub-step][block][piece]: element offsets inside stage 0
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int mb = (wm * TM + i) * 16;
            if constexpr (AKM) oa[ks][i][0] = TileLayout<T, AC, true>::off(mb + (lane & 15), ks * KS + 8 * (lane >> 4));
            else tr_offsets16<T, AC>(ks * KS, mb, lane, oa[ks][i][0], oa[ks][i][NPA - 1]);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nb = (wn * TN + j) * 16;
            if constexpr (BKM) ob[ks][j][0] = A_ELEMS + TileLayout<T, BC, true>::off(nb + (lane & 15), ks * KS + 8 * (lane >> 4));
            else {
                tr_offsets16<T, BC>(ks * KS, nb, lane, ob[ks][j][0], ob[ks][j][NPB - 1]);
                ob[ks][j][0] += A_ELEMS;
                ob[ks][j][NPB - 1] += A_ELEMS;
            }
        }
    }

    uint4 fa[2][TM], fb[2][TN];
    // fetch number f of sub-step `sub` of the tile in stage s, into register set `set`
    auto fetch_one = [&](auto fc, auto subc, auto sc, auto setc) __attribute__((always_inline)) {
        constexpr int f = decltype(fc)::value, sub = decltype(subc)::value, s = decltype(sc)::value, set = decltype(setc)::value;
        const T* st = tiles + s * STAGE_ELEMS;
        if constexpr (f < TM) {
            if constexpr (AKM) fa[set][f] = load_km<T>(st + oa[sub][f][0]);
            else fa[set][f] = load_tr<T>(st + oa[sub][f][0], st + oa[sub][f][NPA - 1]);
        } else {
            constexpr int j = f - TM;
            if constexpr (BKM) fb[set][j] = load_km<T>(st + ob[sub][j][0]);
            else fb[set][j] = load_tr<T>(st + ob[sub][j][0], st + ob[sub][j][NPB - 1]);
        }
    };
    // One sub-step: the NM MFMAs on register set SET, with the NF fetches of (stage FS, sub-step FSUB) into the
    // other set after MFMAs 0, RF, 2 RF, ... (the first three quarters of the sub-step) and, if DMA, the NLOAD tile loads into
    // stage DS after MFMAs at an even spacing.
    auto substep = [&](auto setc, auto fetchc, auto fsc, auto fsubc, auto dmac, auto dsc) __attribute__((always_inline)) {
        constexpr int set = decltype(setc)::value;
        constexpr bool FETCH = decltype(fetchc)::value, DMA = decltype(dmac)::value;
        constexpr int fs = decltype(fsc)::value, fsub = decltype(fsubc)::value, ds = decltype(dsc)::value;
        constexpr int RF = (NM - NM / 4) / NF > 0 ? (NM - NM / 4) / NF : 1;
        constexpr int RD = NM / NLOAD > 0 ? NM / NLOAD : 1;
        const unsigned sA = lds0 + (unsigned)(ds * STAGE_ELEMS * 2);
        static_for<NM>([&](auto mc) __attribute__((always_inline)) {
            constexpr int m = decltype(mc)::value;
            constexpr int i = m / TN, j = m % TN;
            acc[i][j] = Mfma16x16x32<T>::run(fa[set][i], fb[set][j], acc[i][j]);
            if constexpr (FETCH && m % RF == 0 && m / RF < NF)
                fetch_one(std::integral_constant<int, m / RF>{}, fsubc, fsc, std::integral_constant<int, set ^ 1>{});
            if constexpr (DMA && m % RD == RD - 1 && m / RD < NLOAD) {
                constexpr int d = m / RD;
                if constexpr (d < DA::N) da.issue_one(d, sA, wave_u);
                else db.issue_one(d - DA::N, sA + (unsigned)(A_ELEMS * 2), wave_u);
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        (void)fs; (void)fsub; (void)ds;
    };

    // prologue: every buffer gets a tile; tile 0 is waited for and its first sub-step fetched
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
        if (s < nk) {
            const unsigned sA = lds0 + (unsigned)(s * STAGE_ELEMS * 2);
            da.issue(sA, wave_u);
            db.issue(sA + (unsigned)(A_ELEMS * 2), wave_u);
        }
    if (nk >= STAGES) wait_vmcnt<NLOAD * (STAGES - 1)>();
    else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    static_for<NF>([&](auto fc) __attribute__((always_inline)) {
        fetch_one(fc, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    });

    auto tile = [&](auto sc, int kt) __attribute__((always_inline)) {
        constexpr int s = decltype(sc)::value, sn = (s + 1) % STAGES;
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<bool, true> Yes;
        typedef std::integral_constant<bool, false> No;
        // first half: its operands were asked for during the previous sub-step
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_sched_barrier(0);
        substep(I0{}, Yes{}, sc, I1{}, No{}, sc);
        // middle: this wave has read all of the tile; the next tile has landed once every wave says so
        __builtin_amdgcn_s_waitcnt(0xc07f);
        const bool next = kt + 1 < nk;               // uniform
        const bool refill = kt + STAGES < nk;        // uniform
        if (next) {
            if (kt + STAGES - 1 < nk) wait_vmcnt<NLOAD * (STAGES - 2)>();
            else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
        if (refill) {
            substep(I1{}, Yes{}, std::integral_constant<int, sn>{}, I0{}, Yes{}, sc);
            da.advance();
            db.advance();
        } else if (next) {
            substep(I1{}, Yes{}, std::integral_constant<int, sn>{}, I0{}, No{}, sc);
        } else {
            substep(I1{}, No{}, sc, I0{}, No{}, sc);
        }
    };
    // a tile in the steady state: the next tile exists and the one STAGES ahead is loaded into this tile's buffer
    auto tile_steady = [&](auto sc) __attribute__((always_inline)) {
        constexpr int s = decltype(sc)::value, sn = (s + 1) % STAGES;
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 1> I1;
        typedef std::integral_constant<bool, true> Yes;
        typedef std::integral_constant<bool, false> No;
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_sched_barrier(0);
        substep(I0{}, Yes{}, sc, I1{}, No{}, sc);
        __builtin_amdgcn_s_waitcnt(0xc07f);
        wait_vmcnt<NLOAD * (STAGES - 2)>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        substep(I1{}, Yes{}, std::integral_constant<int, sn>{}, I0{}, Yes{}, sc);
        da.advance();
        db.advance();
    };
    // one straight-line loop body of STAGES tiles while every one of them refills its buffer (no branches and no
    // copies of accumulators between its tiles), then the last tiles one by one
    int kt0 = 0;
    for (; kt0 + 2 * STAGES <= nk; kt0 += STAGES) {
        tile_steady(std::integral_constant<int, 0>{});
        if constexpr (STAGES > 1) tile_steady(std::integral_constant<int, 1>{});
        if constexpr (STAGES > 2) tile_steady(std::integral_constant<int, 2>{});
        if constexpr (STAGES > 3) tile_steady(std::integral_constant<int, 3>{});
        if constexpr (STAGES > 4) tile_steady(std::integral_constant<int, 4>{});
    }
    for (; kt0 < nk; kt0 += STAGES) {
        if (kt0 + 0 < nk) tile(std::integral_constant<int, 0>{}, kt0);
        if constexpr (STAGES > 1) { if (kt0 + 1 < nk) tile(std::integral_constant<int, 1>{}, kt0 + 1); }
        if constexpr (STAGES > 2) { if (kt0 + 2 < nk) tile(std::integral_constant<int, 2>{}, kt0 + 2); }
        if constexpr (STAGES > 3) { if (kt0 + 3 < nk) tile(std::integral_constant<int, 3>{}, kt0 + 3); }
        if constexpr (STAGES > 4) { if (kt0 + 4 < nk) tile(std::integral_constant<int, 4>{}, kt0 + 4); }
        static_assert(STAGES <= 5, "at most five stages");
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    gemm_epilogue16<T, TM, TN, WM, WN>(a, acc, reinterpret_cast<float*>(smem), m0, n0, tile_z);
}

template <typename T, bool AKM, bool BKM>
static bool launch_pipe_cfg(int cfg, dim3 grid, const GemmArgs& a, hipStream_t s) {
    switch (cfg) {
    case 6: if constexpr (AKM && BKM) { gemm_pipe_kernel<T, AKM, BKM, 192, 160, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 7: if constexpr (AKM && BKM) { gemm_pipe_kernel<T, AKM, BKM, 160, 160, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 14: if constexpr (AKM) { gemm_pipe_kernel<T, AKM, BKM, 192, 128, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 15: gemm_pipe_kernel<T, AKM, BKM, 256, 128, 4, 1, 3><<<grid, 256, 0, s>>>(a); return true;
    case 16: gemm_pipe_kernel<T, AKM, BKM, 128, 128, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true;
    case 41: if constexpr (AKM) { gemm_pipe_kernel<T, AKM, BKM, 224, 128, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 42: if constexpr (AKM) { gemm_pipe_kernel<T, AKM, BKM, 160, 128, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    case 43: if constexpr (AKM && BKM) { gemm_pipe_kernel<T, AKM, BKM, 224, 160, 2, 2, 3><<<grid, 256, 0, s>>>(a); return true; } return false;
    default: return false;
    }
}

template <typename T>
static bool launch_pipe_op(int cfg, int op, dim3 grid, const GemmArgs& a, hipStream_t s) {
    switch (op) {
    case TP_GEMM_NT: return launch_pipe_cfg<T, true, true>(cfg, grid, a, s);
    case TP_GEMM_NN: return launch_pipe_cfg<T, true, false>(cfg, grid, a, s);
    default: return launch_pipe_cfg<T, false, false>(cfg, grid, a, s);
    }
}

bool launch_gemm_pipe(int cfg, int op, int dtype, dim3 grid, const GemmArgs& a, hipStream_t s) {
    if (dtype == TP_F16) return launch_pipe_op<f16>(cfg, op, grid, a, s);
    if (dtype == TP_BF16) return launch_pipe_op<bf16>(cfg, op, grid, a, s);
    return false;
}

bool launch_gemm_pipe_group(int cfg, int dtype, int tiles, const GemmGroupArgs& ga, hipStream_t s) {
    if (cfg != 15) return false;
    if (dtype == TP_F16) gemm_pipe_kernel<f16, false, false, 256, 128, 4, 1, 3, true><<<dim3(tiles), 256, 0, s>>>(ga);
    else if (dtype == TP_BF16) gemm_pipe_kernel<bf16, false, false, 256, 128, 4, 1, 3, true><<<dim3(tiles), 256, 0, s>>>(ga);
    else return false;
    return true;
}

}  // namespace tp
