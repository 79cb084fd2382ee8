// MFMA GEMMs (NT / NN / TN) with fused epilogues for the linears of the GPT layer at tensor-parallel
// size 1.  One templated kernel covers the three operand layouts and the three dtypes: an operand is
// either "k-major" (k contiguous in memory: fetched from LDS with ds_read_b128) or "mn-major"
// (k is the slow dimension: fetched with the gfx950 LDS transpose read), see common.h.
#include "gemm_epilogue.h"

#include <mutex>

namespace tp {

// ---------------------------------------------------------------------------------------------
// 16-bit kernel with direct global->LDS loads (global_load_lds_dwordx4) and a STAGES-deep ring of
// LDS tiles.  A wave instruction writes 64 consecutive 16-byte chunks of LDS, so the XOR swizzle of the
// tile layout is applied on the global side: the lane that fills LDS chunk (row, pc) loads the global
// chunk (row, pc ^ swz(row)).  Chunks outside the matrix are loaded from a zero buffer so that every
// lane issues every load and the per-tile vmcnt accounting is exact.  The loads are inline asm: the
// compiler does not see them as LDS writes (it would otherwise force vmcnt(0) before every ds_read),
// and the kernel waits with explicit s_waitcnt vmcnt(n) + s_barrier once per k-tile.
// ---------------------------------------------------------------------------------------------
template <typename T, bool AKM, bool BKM, int BM, int BN, int BK, int WM, int WN, int STAGES>
__global__ __launch_bounds__(WM * WN * 64) void gemm_dma_kernel(GemmArgs a) {
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "the direct-to-LDS kernel is for fp16 / bf16");
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int AR = AKM ? BM : BK, AC = AKM ? BK : BM;
    constexpr int BR = BKM ? BN : BK, BC = BKM ? BK : BN;
    constexpr int A_ELEMS = AR * AC, B_ELEMS = BR * BC;
    constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
    typedef SlidingTileDma<T, AR, AC, NT, AKM> DA;
    typedef SlidingTileDma<T, BR, BC, NT, BKM> DB;
    constexpr int NLOAD = DA::N + DB::N;                 // DMA instructions per thread per k-tile
    static_assert(NLOAD * (STAGES - 1) <= 63, "too many loads in flight for vmcnt");
    constexpr int TILE_BYTES = STAGES * STAGE_ELEMS * 2;
    constexpr int EPI_BYTES = WM * WN * 32 * 36 * 4;
    constexpr int SMEM_BYTES = TILE_BYTES > EPI_BYTES ? TILE_BYTES : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    T* tiles = reinterpret_cast<T*>(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int kbeg = blockIdx.z * a.kper;
    const int kend = min(a.K, kbeg + a.kper);
    const T* A = reinterpret_cast<const T*>(a.A);
    const T* B = reinterpret_cast<const T*>(a.B);

    DA da;
    DB db;
    da.init(A, a.lda, m0, a.M, kbeg, BK, tid);
    db.init(B, a.ldb, n0, a.N, kbeg, BK, tid);
    const int klen = kend - kbeg;
    auto issue = [&](int stage) {      // tiles are issued in k order; tiles past the end load zeros
        T* sA = tiles + stage * STAGE_ELEMS;
        da.issue(sA, klen, BK, tid);
        db.issue(sA + A_ELEMS, klen, BK, tid);
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // LDS addresses of this lane's operand fetches inside stage 0 (they do not depend on the k-tile;
    // with the stage loop unrolled the stage base folds into the instruction's immediate offset)
    constexpr int NKSTEP = BK / E::KSTEP;
    constexpr int NPA = AKM ? 1 : 2, NPB = BKM ? 1 : 2;
    const T* pa[NKSTEP][TM][NPA];
    const T* pb[NKSTEP][TN][NPB];
#pragma unroll
    for (int ks = 0; ks < NKSTEP; ++ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int mb = (wm * TM + i) * 32;
            if constexpr (AKM) {
                pa[ks][i][0] = tiles + km_offset<T, AC>(mb + (lane & 31), ks * E::KSTEP, lane);
            } else {
                int o0, o1;
                tr_offsets<T, AC, false>(ks * E::KSTEP, mb, lane, o0, o1);
                pa[ks][i][0] = tiles + o0;
                pa[ks][i][NPA - 1] = tiles + o1;
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nb = (wn * TN + j) * 32;
            if constexpr (BKM) {
                pb[ks][j][0] = tiles + A_ELEMS + km_offset<T, BC>(nb + (lane & 31), ks * E::KSTEP, lane);
            } else {
                int o0, o1;
                tr_offsets<T, BC, false>(ks * E::KSTEP, nb, lane, o0, o1);
                pb[ks][j][0] = tiles + A_ELEMS + o0;
                pb[ks][j][NPB - 1] = tiles + A_ELEMS + o1;
            }
        }
    }

    const int nk = (kend - kbeg + BK - 1) / BK;
    // prologue: tiles 0 .. STAGES-2 in flight (tiles past the end load zeros; keeps the counts uniform)
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s);

    for (int kt0 = 0; kt0 < nk; kt0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {        // stage index is a compile-time constant in here
            if (kt0 + s < nk) {
                // tile kt has landed once at most the loads of the STAGES-2 younger tiles are outstanding
                wait_vmcnt<NLOAD * (STAGES - 2)>();
                __builtin_amdgcn_s_barrier();   // every wave's part of the tile is in LDS; the previous tile is no longer read
                asm volatile("" ::: "memory");
                issue((s + STAGES - 1) % STAGES);   // tile kt + STAGES - 1 refills the buffer of tile kt - 1
                // all operand fetches of the tile are issued before the first MFMA, so their LDS latency
                // overlaps instead of being paid once per k-step (one wave per SIMD has nothing else to hide it)
                typename E::opnd_t fa[NKSTEP][TM], fb[NKSTEP][TN];
#pragma unroll
                for (int ks = 0; ks < NKSTEP; ++ks) {
#pragma unroll
                    for (int i = 0; i < TM; ++i) {
                        if constexpr (AKM) fa[ks][i] = load_km<T>(pa[ks][i][0] + s * STAGE_ELEMS);
                        else fa[ks][i] = load_tr<T>(pa[ks][i][0] + s * STAGE_ELEMS, pa[ks][i][NPA - 1] + s * STAGE_ELEMS);
                    }
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if constexpr (BKM) fb[ks][j] = load_km<T>(pb[ks][j][0] + s * STAGE_ELEMS);
                        else fb[ks][j] = load_tr<T>(pb[ks][j][0] + s * STAGE_ELEMS, pb[ks][j][NPB - 1] + s * STAGE_ELEMS);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);   // keep the scheduler from sinking the fetches to their uses
#pragma unroll
                for (int ks = 0; ks < NKSTEP; ++ks)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) acc[i][j] = E::mfma(fa[ks][i], fb[ks][j], acc[i][j]);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave's LDS reads of the tile are done
            }
        }
    }
    // drain the zero-tile loads still in flight before LDS is reused for the epilogue
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    gemm_epilogue<T, TM, TN, WM, WN>(a, acc, reinterpret_cast<float*>(smem), m0, n0, (int)blockIdx.z);
}

// ---------------------------------------------------------------------------------------------
// Tall-tile variant for long activations (M >= 256): BM = 256 rows by four waves stacked in M, each
// holding a 64 x BN block of the output in accumulator registers (BN up to 192 -> 192 AGPRs; one wave per
// SIMD).  A 256 x 160 x 64 tile moves 52 KB for 5.2 MFLOP, 1.5 times the flops per byte of a 128 x 128 tile:
// the vector-memory path into LDS (64 B/clk per CU) stops being the limit.  BN is any multiple of 32, so
// the tile count can be matched to the 256 CUs (N = 20480: BN = 160 gives exactly 256 tiles for M = 512).
// Tiles are loaded with ClampTileDma (whole k-tiles only) and the operand fetches of k-step s+1 are issued
// before the MFMAs of k-step s.
// MI16: 16 x 16 x 32 MFMA blocks and ONE set of operand registers per wave (two waves share a SIMD: one computes
// while the other fetches; two sets of the twice as many operand registers do not fit beside the accumulators).
template <typename T, bool AKM, bool BKM, int BM, int BN, int BK, int WM, int WN, int STAGES, bool GROUPED = false,
          bool MI16 = false>
__global__ __launch_bounds__(WM * WN * 64)
void gemm_tall_kernel(typename std::conditional<GROUPED, GemmGroupArgs, GemmArgs>::type args) {
    // which problem and which of its tiles (wave-uniform)
    int prob = 0, tile_x = blockIdx.x, tile_y = blockIdx.y;
    if constexpr (GROUPED) {
        static_assert(kGroupMax == 4, "the selects below are written out for four problems");
        int first = 0, tx = args.tiles_x[0], ty = args.tiles_y[0];
        if (1 < args.n && (int)blockIdx.x >= args.first_tile[1]) { prob = 1; first = args.first_tile[1]; tx = args.tiles_x[1]; ty = args.tiles_y[1]; }
        if (2 < args.n && (int)blockIdx.x >= args.first_tile[2]) { prob = 2; first = args.first_tile[2]; tx = args.tiles_x[2]; ty = args.tiles_y[2]; }
        if (3 < args.n && (int)blockIdx.x >= args.first_tile[3]) { prob = 3; first = args.first_tile[3]; tx = args.tiles_x[3]; ty = args.tiles_y[3]; }
        xcd_tile((int)blockIdx.x - first, tx, ty, tile_x, tile_y);
    } else if (gridDim.z == 1) {
        xcd_tile((int)(blockIdx.y * gridDim.x + blockIdx.x), (int)gridDim.x, (int)gridDim.y, tile_x, tile_y);
    }
    // (constant indices only: a dynamically indexed kernel argument would be copied to scratch memory)
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
    typedef Elem<T> E;
    static_assert(sizeof(T) == 2, "16-bit only");
    constexpr int NT = WM * WN * 64;
    constexpr int BLK = MI16 ? 16 : 32;                  // rows / columns of an MFMA block
    constexpr int KS = MI16 ? 32 : E::KSTEP;             // k of one MFMA
    static_assert(!MI16 || WM * WN == 8, "the 16 x 16 blocks are written for two waves per SIMD");
    constexpr int TM = BM / WM / BLK, TN = BN / WN / BLK;
    constexpr int AR = AKM ? BM : BK, AC = AKM ? BK : BM;
    constexpr int BR = BKM ? BN : BK, BC = BKM ? BK : BN;
    constexpr int A_ELEMS = AR * AC, B_ELEMS = BR * BC;
    constexpr int STAGE_ELEMS = A_ELEMS + B_ELEMS;
    typedef ClampTileDma<T, AR, AC, NT, AKM, MI16 && AKM> DA;
    typedef ClampTileDma<T, BR, BC, NT, BKM, MI16 && BKM> DB;
    constexpr int NLOAD = DA::N + DB::N;
    static_assert(NLOAD * (STAGES - 1) <= 63, "too many loads in flight for vmcnt");
    constexpr int TILE_BYTES = STAGES * STAGE_ELEMS * 2;
    constexpr int EPI_BYTES = WM * WN * 32 * 36 * 4;
    constexpr int SMEM_BYTES = TILE_BYTES > EPI_BYTES ? TILE_BYTES : EPI_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
    T* tiles = reinterpret_cast<T*>(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int m0 = tile_y * BM, n0 = tile_x * BN;
    const int kbeg = blockIdx.z * a.kper;
    const int kend = min(a.K, kbeg + a.kper);
    DA da;
    DB db;
    da.init(reinterpret_cast<const T*>(a.A), a.lda, m0, a.M, kbeg, BK, tid);
    db.init(reinterpret_cast<const T*>(a.B), a.ldb, n0, a.N, kbeg, BK, tid);
    const unsigned lds0 = lds_addr(smem);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto issue = [&](int stage) {
        const unsigned sA = lds0 + (unsigned)(stage * STAGE_ELEMS * (int)sizeof(T));
        da.issue(sA, wave_u);
        db.issue(sA + (unsigned)(A_ELEMS * (int)sizeof(T)), wave_u);
    };

    typedef typename std::conditional<MI16, float4v, float16v>::type acc_t;
    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < (MI16 ? 4 : 16); ++r) acc[i][j][r] = 0.f;

    constexpr int NKSTEP = BK / KS;
    constexpr int NPA = AKM ? 1 : 2, NPB = BKM ? 1 : 2;
    // lane's fetch offsets for k-step 0 of stage 0; k-steps and stages are compile-time byte offsets for
    // k-major operands (a k-step is two (four) chunks further along the row)
    int oa[NKSTEP][TM][NPA], ob[NKSTEP][TN][NPB];
    auto operand_offsets = [&](auto km_c, auto cols_c, int row0, int k0, int& o0, int& o1) {
        constexpr bool KM = decltype(km_c)::value;
        constexpr int COLS = decltype(cols_c)::value;
        if constexpr (MI16) {
            if constexpr (KM) o0 = o1 = TileLayout<T, COLS, true>::off(row0 + (lane & 15), k0 + 8 * (lane >> 4));
            else tr_offsets16<T, COLS>(k0, row0, lane, o0, o1);
        } else {
            if constexpr (KM) o0 = o1 = km_offset<T, COLS>(row0 + (lane & 31), k0, lane);
            else tr_offsets<T, COLS, false>(k0, row0, lane, o0, o1);
        }
    };
#pragma unroll
    for (int ks = 0; ks < NKSTEP; ++ks) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
            operand_offsets(std::integral_constant<bool, AKM>{}, std::integral_constant<int, AC>{}, (wm * TM + i) * BLK,
                            ks * KS, oa[ks][i][0], oa[ks][i][NPA - 1]);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            int o0, o1;
            operand_offsets(std::integral_constant<bool, BKM>{}, std::integral_constant<int, BC>{}, (wn * TN + j) * BLK,
                            ks * KS, o0, o1);
            ob[ks][j][0] = A_ELEMS + o0;
            ob[ks][j][NPB - 1] = A_ELEMS + o1;
        }
    }

    const int nk = (kend - kbeg) / BK;          // whole tiles only (the plan guarantees it)
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < nk) issue(s);

    constexpr int NSET = MI16 ? 1 : 2;
    typename E::opnd_t fa[NSET][TM], fb[NSET][TN];
    auto fetch = [&](auto ksc, auto sc, int buf) {
        constexpr int ks = decltype(ksc)::value, s = decltype(sc)::value;
        const T* st = tiles + s * STAGE_ELEMS;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if constexpr (AKM) fa[buf][i] = load_km<T>(st + oa[ks][i][0]);
            else fa[buf][i] = load_tr<T>(st + oa[ks][i][0], st + oa[ks][i][NPA - 1]);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if constexpr (BKM) fb[buf][j] = load_km<T>(st + ob[ks][j][0]);
            else fb[buf][j] = load_tr<T>(st + ob[ks][j][0], st + ob[ks][j][NPB - 1]);
        }
    };
    // No tile is loaded past the end of k (ClampTileDma does not bound the sliding axis): the last STAGES - 1
    // tiles issue nothing and wait for every outstanding load instead of all but the younger tiles'.
    auto tile = [&](auto sc, int kt) {
        constexpr int s = decltype(sc)::value;
        const bool more = kt + STAGES - 1 < nk;      // uniform
        if (more) wait_vmcnt<NLOAD * (STAGES - 2)>();
        else wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        fetch(std::integral_constant<int, 0>{}, sc, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (more) issue((s + STAGES - 1) % STAGES);   // issued while the fetch above is in flight
        auto step = [&](auto ksc) {
            constexpr int ks = decltype(ksc)::value;
            constexpr int set = MI16 ? 0 : (ks & 1);
            if constexpr (MI16) {
                if constexpr (ks > 0) fetch(ksc, sc, 0);
            } else if constexpr (ks + 1 < NKSTEP) {
                fetch(std::integral_constant<int, ks + 1>{}, sc, (ks + 1) & 1);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (MI16) acc[i][j] = Mfma16x16x32<T>::run(fa[set][i], fb[set][j], acc[i][j]);
                    else acc[i][j] = E::mfma(fa[set][i], fb[set][j], acc[i][j]);
                }
            if constexpr (MI16) __builtin_amdgcn_sched_barrier(0);
        };
        step(std::integral_constant<int, 0>{});
        if constexpr (NKSTEP > 1) step(std::integral_constant<int, 1>{});
        if constexpr (NKSTEP > 2) step(std::integral_constant<int, 2>{});
        if constexpr (NKSTEP > 3) step(std::integral_constant<int, 3>{});
        static_assert(NKSTEP <= 4, "k-tile of at most four k-steps");
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    for (int kt0 = 0; kt0 < nk; kt0 += STAGES) {
        if (kt0 + 0 < nk) tile(std::integral_constant<int, 0>{}, kt0);
        if constexpr (STAGES > 1) { if (kt0 + 1 < nk) tile(std::integral_constant<int, 1>{}, kt0 + 1); }
        if constexpr (STAGES > 2) { if (kt0 + 2 < nk) tile(std::integral_constant<int, 2>{}, kt0 + 2); }
        if constexpr (STAGES > 3) { if (kt0 + 3 < nk) tile(std::integral_constant<int, 3>{}, kt0 + 3); }
        static_assert(STAGES <= 4, "at most four stages");
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (MI16) gemm_epilogue16<T, TM, TN, WM, WN>(a, acc, reinterpret_cast<float*>(smem), m0, n0, (int)blockIdx.z);
    else gemm_epilogue<T, TM, TN, WM, WN>(a, acc, reinterpret_cast<float*>(smem), m0, n0, (int)blockIdx.z);
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

    gemm_epilogue<T, TM, TN, WM, WN>(a, acc, reinterpret_cast<float*>(smem), m0, n0, (int)blockIdx.z);
}

// Sums the split-K partials and applies the epilogue.  A block of 256 threads covers 256 columns
// (32 threads x 8 columns) by 32 rows (8 row lanes x 4 rows); column sums are combined across the
// row lanes in LDS so that they cost one atomic per column per block.
template <typename T>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmArgs a) {
    __shared__ float cs[8][256];
    const int cl = threadIdx.x & 31, rl = threadIdx.x >> 5;
    const int col0 = (blockIdx.x * 32 + cl) * 8;
    const int rbase = blockIdx.y * 32;
    float csum[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) csum[e] = 0.f;
    if (col0 < a.N) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int row = rbase + rr * 8 + rl;
            if (row < a.M) {
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
        }
    }
    if (a.colsum) {
#pragma unroll
        for (int e = 0; e < 8; ++e) cs[rl][cl * 8 + e] = csum[e];
        __syncthreads();
        const int c = threadIdx.x;
        const int col = blockIdx.x * 256 + c;
        if (col < a.N) {
            float t = 0.f;
#pragma unroll
            for (int r = 0; r < 8; ++r) t += cs[r][c];
            atomicAdd(a.colsum + col, t);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static constexpr int kNumCU = 256;  // MI355X

// Tile configurations of the 16-bit kernels by number (the numbers are what the measured plan table, the
// `reserved` field of tp_gemm_desc and the tuning script refer to; numbers not listed do not exist).
struct TileCfg { int bm, bn, bk, stages; };
static bool tile_cfg(int id, TileCfg& c) {
    switch (id) {
    case 0: c = {64, 64, 64, 2}; return true;      // gemm_kernel, register-staged (fp32 runs it with 64 x 64 x 16 tiles)
    // gemm_dma_kernel: four waves 2 x 2 (configuration 3: eight waves of 64 x 64)
    case 3: c = {128, 256, 64, 3}; return true;
    case 5: c = {128, 128, 64, 2}; return true;
    case 8: c = {64, 64, 64, 4}; return true;
    case 10: c = {128, 128, 32, 4}; return true;
    case 11: c = {64, 256, 64, 3}; return true;
    case 12: c = {64, 64, 128, 4}; return true;
    case 13: c = {128, 128, 64, 3}; return true;
    // gemm_tall_kernel: 256-row tiles
    case 2: c = {256, 256, 32, 4}; return true;    // gemm_tall_kernel, 20 on 16 x 16 x 32 MFMA blocks
    // gemm_pipe_kernel: four waves, 16 x 16 x 32 MFMA blocks, software-pipelined k-loop
    case 6: c = {192, 160, 64, 3}; return true;    // 2 x 2 waves of 96 x 80 (NT only, like 7)
    case 7: c = {160, 160, 64, 3}; return true;    // 2 x 2 waves of 80 x 80
    case 14: c = {192, 128, 64, 3}; return true;   // 2 x 2 waves of 96 x 64
    case 15: c = {256, 128, 64, 3}; return true;   // 4 x 1 waves of 64 x 128
    case 16: c = {128, 128, 64, 3}; return true;   // 2 x 2 waves of 64 x 64
    case 17: c = {256, 160, 64, 3}; return true;   // 4 waves stacked in M, 64 x 160 each (NT only)
    case 18: c = {256, 128, 64, 3}; return true;   // 64 x 128 each
    case 19: c = {256, 256, 64, 2}; return true;   // 8 waves (4 x 2) of 64 x 128
    case 20: c = {256, 256, 32, 4}; return true;   // the same with half the k-tile and twice the stages
    // gemm_stream_kernel (gemm_stream.hip; NT and NN): whole-slice row tiles of 64 * RB rows, separate activation /
    // weight rings (stages = the weight ring's); 4 waves unless noted
    case 21: c = {192, 128, 64, 5}; return true;
    case 22: c = {256, 128, 64, 4}; return true;
    case 23: c = {256, 128, 64, 6}; return true;   // two activation stages
    case 24: c = {192, 80, 64, 8}; return true;    // NT only
    case 25: c = {256, 80, 64, 6}; return true;    // NT only
    case 26: c = {128, 128, 64, 7}; return true;
    case 27: c = {256, 64, 64, 8}; return true;
    case 28: c = {192, 64, 64, 10}; return true;
    case 29: c = {256, 128, 64, 4}; return true;   // 8 waves
    case 30: c = {192, 128, 64, 5}; return true;   // 8 waves
    case 31: c = {192, 128, 64, 5}; return true;   // 16 waves
    case 32: c = {256, 128, 64, 4}; return true;   // 16 waves
    case 33: c = {192, 256, 64, 3}; return true;   // 16 waves
    case 34: c = {256, 256, 64, 3}; return true;   // 16 waves
    case 35: c = {128, 256, 64, 3}; return true;   // 16 waves
    case 36: c = {64, 256, 64, 4}; return true;    // 16 waves
    case 37: c = {128, 128, 64, 7}; return true;   // 16 waves
    case 38: c = {64, 128, 64, 8}; return true;    // 16 waves
    case 39: c = {128, 256, 64, 3}; return true;   // 8 waves
    case 40: c = {64, 256, 64, 4}; return true;    // 8 waves
    // gemm_pipe_kernel again: row tiles that fit slices of 224 and of 160 / 320 rows (whole 16-row blocks, so
    // nothing of a tile lies beyond the slice)
    case 41: c = {224, 128, 64, 3}; return true;   // 2 x 2 waves of 112 x 64
    case 42: c = {160, 128, 64, 3}; return true;   // 2 x 2 waves of 80 x 64
    case 43: c = {224, 160, 64, 3}; return true;   // 2 x 2 waves of 112 x 80 (NT only, like 6 and 7)
    default: return false;
    }
}
static constexpr int kFirstStreamCfg = 21, kLastStreamCfg = 40;

// Measured plans: for NT / NN the weight extents (N, K) match exactly and M (tokens of the slice) picks the
// nearest measured M at or above it (at least half of it, so that a much shorter slice falls through to the
// heuristics); TN (parameter gradients) matches all three extents.
struct TunedPlan { int op, M, N, K, cfg, nsplit; };
static const TunedPlan kTuned[] = {
#include "gemm_tuned.inc"
    {-1, 0, 0, 0, 0, 0},
};

static const TunedPlan* find_tuned(const tp_gemm_desc* d) {
    const TunedPlan* best = nullptr;
    for (const TunedPlan* t = kTuned; t->op >= 0; ++t) {
        if (t->op != d->op || t->N != d->N || t->K != d->K) continue;
        if (d->op == TP_GEMM_TN) {
            if (t->M == d->M) return t;
            continue;
        }
        if (t->M >= d->M && t->M <= 2 * d->M && (!best || t->M < best->M)) best = t;
    }
    return best;
}

struct GemmPlan {
    int cfg;
    int nsplit;
    int kper;
    int gx, gy;
};

static void finish_plan(const tp_gemm_desc* d, GemmPlan& p, int bk, int nsplit) {
    long kt = (d->K + bk - 1) / bk;
    if (nsplit > kt) nsplit = (int)kt;
    if (nsplit < 1) nsplit = 1;
    long per = (kt + nsplit - 1) / nsplit;
    p.kper = (int)(per * bk);
    p.nsplit = (int)((d->K + p.kper - 1) / p.kper);
}

static GemmPlan plan_gemm(const tp_gemm_desc* d) {
    GemmPlan p;
    if (d->dtype == TP_F32) {
        p.cfg = 0;
        p.gx = (d->N + 63) / 64; p.gy = (d->M + 63) / 64;
        long tiles = (long)p.gx * p.gy;
        int nsplit = 1;
        if (tiles < 2 * kNumCU) {
            long want = (2 * kNumCU + tiles - 1) / tiles;
            long kt = (d->K + 15) / 16;
            long maxs = kt / 8 > 0 ? kt / 8 : 1;
            nsplit = (int)(want < maxs ? want : maxs);
            if (nsplit > 16) nsplit = 16;
        }
        finish_plan(d, p, 16, nsplit);
        return p;
    }
    // reserved: bits 0-7 force a tile configuration (1-based index + 1 so that 0 means automatic),
    // bits 8-15 force the number of k splits.  For tuning and tests.
    int forced_cfg = (d->reserved & 0xff) - 1;
    int forced_split = (d->reserved >> 8) & 0xff;
    const long t128 = (long)((d->M + 127) / 128) * ((d->N + 127) / 128);
    const long t64 = (long)((d->M + 63) / 64) * ((d->N + 63) / 64);
    int cfg, ns = 1;
    const long t256n = (d->N + 255) / 256;
    const long t256 = (long)((d->M + 255) / 256) * t256n;
    // k splits that bring `tiles` workgroups as near to one per CU as they get without exceeding it (a second, partly
    // filled round costs more than the idle CUs) while every split keeps at least min_k of k
    auto splits_for = [&](long tiles, int min_k) {
        int v = (int)(kNumCU / tiles);
        const int maxs = d->K / min_k;
        if (v > maxs) v = maxs;
        if (v > 8) v = 8;
        return v < 1 ? 1 : v;
    };
    if (d->op != TP_GEMM_TN && d->M <= 512) {
        // A slice's linears, forward (NT) and data gradient (NN): up to 512 rows against a weight.  The rules are the
        // common ground of sweeps over every tile configuration and split on layer geometries that have no entry in
        // the measured table (hidden 3072 to 10240, 64 to 512 rows): about one workgroup per CU is the target -- fewer
        // leave CUs without a share of the weight stream, every extra split adds a round of fp32 partial sums and
        // does not pay below 1536-2048 of k per split -- and the tile grows with the slice so that the activation,
        // which every column tile re-reads, stays the smaller part of what a CU has to fill.
        const long t3 = (long)((d->M + 127) / 128) * t256n;          // 128 x 256 tiles
        const bool small_weight = (long)d->N * d->K <= (16L << 20);  // 4096 x 4096 and below
        if (d->M <= 64) {
            // one row of tiles: 64 x 64 until they come to more than two per CU, then 64 x 256
            if (t64 >= 2 * kNumCU) { cfg = 11; ns = splits_for(t256n, 2048); }
            else { cfg = 8; ns = splits_for(t64, 2048); }
        } else if (small_weight) {
            // 64 x 64 tiles reach the CU count without splitting k
            cfg = (d->M <= 256 && d->K % 128 == 0) ? 12 : 8;
            ns = t64 >= 96 ? 1 : splits_for(t64, 2048);
        } else if (d->M <= 128) {
            const int ns13 = splits_for(t128, 1536);
            if (t128 > kNumCU) { cfg = 3; ns = splits_for(t3, 2048); }                      // many column tiles: 128 x 256
            else if (t128 * ns13 < 192 && t64 >= 192 && t64 <= 2 * kNumCU) { cfg = 8; }     // too few 128 x 128 tiles for the chip
            else { cfg = 13; ns = ns13; }
        } else if (d->M > 448 && d->K % 64 == 0 && t256 >= 160) {
            cfg = 19;               // two full rows of 256 x 256 tiles for most of the CUs
        } else if (d->M > 256 && d->M <= 384 && d->K % 64 == 0 && t3 > kNumCU) {
            cfg = 33;               // two row tiles of 192 x 256 (the weight-streaming kernel) where 128 x 256 tiles are too many
            ns = splits_for(2 * t256n, 2048);
        } else {
            // 128 x 256 tiles when a split still keeps 4096 of k, to amortise the larger tile's prologue; else 128 x 128
            const int ns3 = splits_for(t3, 2048);
            if (d->K / ns3 >= 4096 || t128 > kNumCU) { cfg = 3; ns = ns3; }
            else { cfg = 13; ns = splits_for(t128, 2048); }
        }
    } else if ((d->op == TP_GEMM_TN || d->M >= 512) && d->K % 64 == 0 && t256 >= 192) {
        // parameter gradients of a whole step, and any product of 512 rows or more with that many tiles (the LM
        // head): 256 x 256 tiles by eight waves (half the bytes per flop of a 128 x 128 tile through the
        // 64 B/clk vector-memory path into LDS); the parameter gradients on 16 x 16 x 32 blocks with the 32-wide
        // k-tile in four stages (timed inside steps of four geometries: 1 to 5 % under the 32 x 32 blocks)
        cfg = d->op == TP_GEMM_TN ? 2 : 19;
    } else if (d->op != TP_GEMM_TN && d->M >= 512 && d->K % 64 == 0 && t256 >= 48 && d->K >= 8192) {
        // the same tiles on a long k with too few of them for the chip (the LM head's data gradient, k =
        // vocabulary): k is split to about one workgroup per CU
        cfg = 19;
        ns = (int)((256 + t256 - 1) / t256);
        int maxs = d->K / 2048;
        if (ns > maxs) ns = maxs;
        if (ns > 8) ns = 8;
    } else if (t128 >= 144) {
        // short activations: the deeper ring keeps the weight stream going; parameter gradients (both
        // operands fetched with transpose reads): 128 x 128 x 32, four stages, two workgroups per CU
        cfg = d->op == TP_GEMM_TN ? 10 : (d->M <= 256 ? 13 : 5);
        if (t128 < 224) {
            ns = (int)(448 / t128);
            int maxs = d->K / 1024;
            if (ns > maxs) ns = maxs;
        }
    } else {
        cfg = 8;
        if (t64 < 384) {
            ns = (int)(512 / t64);
            int maxs = d->K / 3072;
            if (ns > maxs) ns = maxs;
        }
    }
    // The pipelined 16 x 16 x 32 tiles in place of the 32 x 32 ones the rules above name, where a sweep over other
    // geometries (hidden 3072, 4096, 8192; 128 to 512 rows; 144 slice products) has them ahead: 128 x 128 for
    // 128 x 128 (0.94 to 0.99 of the time), 192 x 128 for 128 x 256 at 129 to 192 rows and at 257 to 384 (0.83 to 0.91),
    // 256 x 128 above 384 rows (0.92), and the 160- and 224-row tiles where they end with the slice (0.95 to 1.0 of
    // the padded tile's time on the 13B shapes); a k-split stays within one round of workgroups of the new tile.
    if (d->op != TP_GEMM_TN && d->K % 64 == 0 && (cfg == 13 || cfg == 3)) {
        int bm = 128, bn = 128, to = 16;
        if (cfg == 3) {
            // row tiles that end with the slice where whole 16-row blocks allow it: 160 (one or two tiles), 192 (one
            // or two), 224 (one or two), else 256
            if ((d->M > 128 && d->M <= 160) || (d->M > 256 && d->M <= 320)) { to = 42; bm = 160; }
            else if ((d->M > 160 && d->M <= 192) || (d->M > 320 && d->M <= 384)) { to = 14; bm = 192; }
            else if ((d->M > 192 && d->M <= 224) || (d->M > 384 && d->M <= 448)) { to = 41; bm = 224; }
            else if (d->M > 448) { to = 15; bm = 256; }
            else to = 3;
        }
        if (to != 3) {
            cfg = to;
            const long tiles = (long)((d->M + bm - 1) / bm) * ((d->N + bn - 1) / bn);
            const int cap = (int)(kNumCU / tiles);
            if (ns > 1 && ns > cap) ns = cap < 1 ? 1 : cap;
        }
    }
    if (const TunedPlan* t = find_tuned(d)) { cfg = t->cfg; ns = t->nsplit; }
    if (ns < 1) ns = 1;
    if (ns > 16) ns = 16;
    TileCfg tc;
    if (forced_cfg >= 0 && tile_cfg(forced_cfg, tc)) cfg = forced_cfg;
    if (forced_split) ns = forced_split;
    // the tall tiles load whole k-tiles only, and the 160 / 192 wide ones exist for the k-major weight (NT)
    // (a token-major tile 160 or 192 wide has no XOR swizzle: the chunk index would leave the row)
    if ((cfg == 6 || cfg == 7 || cfg == 43) && (d->K % 64 || d->op != TP_GEMM_NT)) cfg = 5;
    if ((cfg == 41 || cfg == 42) && (d->K % 64 || d->op == TP_GEMM_TN)) cfg = 5;
    if (((cfg >= 14 && cfg <= 20) || cfg == 2) && (d->K % 64 || (cfg == 17 && d->op != TP_GEMM_NT) || (cfg == 14 && d->op == TP_GEMM_TN))) cfg = 5;
    // the streaming kernel: NT and NN only, whole 64-wide k-tiles only; tiles whose width is not a power of two need
    // the k-major weight (NT)
    if (cfg >= kFirstStreamCfg && cfg <= kLastStreamCfg &&
        (d->op == TP_GEMM_TN || d->K % 64 || ((cfg == 24 || cfg == 25) && d->op != TP_GEMM_NT))) cfg = 5;
    p.cfg = cfg;
    tile_cfg(cfg, tc);
    p.gx = (d->N + tc.bn - 1) / tc.bn;
    p.gy = (d->M + tc.bm - 1) / tc.bm;
    finish_plan(d, p, tc.bk, ns);
    return p;
}

// the tile configurations of gemm_pipe.hip
static inline bool is_pipe_cfg(int cfg) { return cfg == 6 || cfg == 7 || (cfg >= 14 && cfg <= 16) || (cfg >= 41 && cfg <= 43); }

template <typename T, bool AKM, bool BKM>
static void launch_cfg(const GemmPlan& p, const GemmArgs& a, hipStream_t s) {
    dim3 grid(p.gx, p.gy, p.nsplit);
    if constexpr (sizeof(T) == 4) {
        gemm_kernel<T, AKM, BKM, 64, 64, 16, 2, 2><<<grid, 256, 0, s>>>(a);
    } else {
        switch (p.cfg) {
        case 2: gemm_tall_kernel<T, AKM, BKM, 256, 256, 32, 4, 2, 4, false, true><<<grid, 512, 0, s>>>(a); break;
        case 3: gemm_dma_kernel<T, AKM, BKM, 128, 256, 64, 2, 4, 3><<<grid, 512, 0, s>>>(a); break;
        case 5: gemm_dma_kernel<T, AKM, BKM, 128, 128, 64, 2, 2, 2><<<grid, 256, 0, s>>>(a); break;
        case 8: gemm_dma_kernel<T, AKM, BKM, 64, 64, 64, 2, 2, 4><<<grid, 256, 0, s>>>(a); break;
        case 11: gemm_dma_kernel<T, AKM, BKM, 64, 256, 64, 2, 2, 3><<<grid, 256, 0, s>>>(a); break;
        case 10: gemm_dma_kernel<T, AKM, BKM, 128, 128, 32, 2, 2, 4><<<grid, 256, 0, s>>>(a); break;
        case 12: gemm_dma_kernel<T, AKM, BKM, 64, 64, 128, 2, 2, 4><<<grid, 256, 0, s>>>(a); break;
        case 13: gemm_dma_kernel<T, AKM, BKM, 128, 128, 64, 2, 2, 3><<<grid, 256, 0, s>>>(a); break;
        case 17: if constexpr (BKM) gemm_tall_kernel<T, AKM, BKM, 256, 160, 64, 4, 1, 3><<<grid, 256, 0, s>>>(a); break;
        case 18: gemm_tall_kernel<T, AKM, BKM, 256, 128, 64, 4, 1, 3><<<grid, 256, 0, s>>>(a); break;
        case 19: gemm_tall_kernel<T, AKM, BKM, 256, 256, 64, 4, 2, 2><<<grid, 512, 0, s>>>(a); break;
        case 20: gemm_tall_kernel<T, AKM, BKM, 256, 256, 32, 4, 2, 4><<<grid, 512, 0, s>>>(a); break;
        default: gemm_kernel<T, AKM, BKM, 64, 64, 64, 2, 2><<<grid, 256, 0, s>>>(a); break;
        }
    }
}

// false: the plan names a (tile configuration, op, dtype) that no kernel is built for -- nothing was launched
template <typename T>
static bool launch_gemm(const tp_gemm_desc* d, const GemmPlan& p, const GemmArgs& a, hipStream_t s) {
    if (p.cfg >= kFirstStreamCfg && p.cfg <= kLastStreamCfg) {
        if (!launch_gemm_stream(p.cfg, d->op, d->dtype, dim3(p.gx, p.gy, p.nsplit), a, s)) return false;
    } else if (is_pipe_cfg(p.cfg) && d->dtype != TP_F32) {
        if (!launch_gemm_pipe(p.cfg, d->op, d->dtype, dim3(p.gx, p.gy, p.nsplit), a, s)) return false;
    } else {
        switch (d->op) {
        case TP_GEMM_NT: launch_cfg<T, true, true>(p, a, s); break;
        case TP_GEMM_NN: launch_cfg<T, true, false>(p, a, s); break;
        default: launch_cfg<T, false, false>(p, a, s); break;
        }
    }
    if (p.nsplit > 1 && !d->defer_reduce) {
        dim3 grid((d->N + 255) / 256, (d->M + 31) / 32);
        gemm_splitk_reduce_kernel<T><<<grid, 256, 0, s>>>(a);
    }
    return true;
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
    if (d->defer_reduce && ((d->epilogue != TP_EPI_STORE && d->epilogue != TP_EPI_BIAS_RESIDUAL) || d->colsum_acc)) {
        set_error("tp_gemm: defer_reduce needs the STORE or BIAS_RESIDUAL epilogue and no colsum_acc");
        return TP_ERR_ARG;
    }
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

extern "C" int tp_gemm_splits(const tp_gemm_desc* d) {
    if (tp::validate_gemm(d) != TP_OK) return 0;
    return tp::plan_gemm(d).nsplit;
}

extern "C" int tp_gemm_plan(const tp_gemm_desc* d, int* tile_cfg, int* nsplit) {
    int rc = tp::validate_gemm(d);
    if (rc != TP_OK) return rc;
    tp::GemmPlan p = tp::plan_gemm(d);
    if (tile_cfg) *tile_cfg = p.cfg;
    if (nsplit) *nsplit = p.nsplit;
    return TP_OK;
}

extern "C" size_t tp_gemm_workspace_bytes(const tp_gemm_desc* d) {
    if (tp::validate_gemm(d) != TP_OK) return 0;
    tp::GemmPlan p = tp::plan_gemm(d);
    return p.nsplit > 1 ? (size_t)p.nsplit * d->M * d->N * sizeof(float) : 0;
}

namespace tp {
static GemmArgs fill_args(const tp_gemm_desc* d, const GemmPlan& p, void* workspace) {
    GemmArgs a;
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
    a.q_rows = d->q_bh_rows > 0 ? d->q_bh_rows : a.T;
    a.P = d->cache_len; a.cache_rows = d->cache_rows; a.qscale = d->q_scale;
    a.kper = p.kper; a.nsplit = p.nsplit; a.partial = reinterpret_cast<float*>(workspace);
    return a;
}

// One launch for the whole group when every member is a 16-bit TN product (parameter gradients) of the same dtype
// whose k is a whole number of 64-wide tiles and the group's largest member plans to a 256 x 256 tile with
// unsplit k.
// The tile configuration of the single launch that runs the group, or 0 when it runs member by member.
static int group_cfg(const tp_gemm_desc* descs, int n) {
    if (n < 2 || n > kGroupMax) return 0;
    int big = 0;
    for (int i = 0; i < n; ++i) {
        const tp_gemm_desc& d = descs[i];
        if (d.op != TP_GEMM_TN || d.dtype != descs[0].dtype || d.dtype == TP_F32 || d.K % 64 != 0 ||
            d.reserved != descs[0].reserved ||      // a forced plan (tuning, tests) must be the same for all members
            d.defer_reduce != 0 || d.epilogue == TP_EPI_QKV_SCATTER)
            return 0;
        if ((double)d.M * d.N > (double)descs[big].M * descs[big].N) big = i;
    }
    const GemmPlan pb = plan_gemm(&descs[big]);
    return ((pb.cfg == 2 || pb.cfg == 15 || pb.cfg == 19 || pb.cfg == 20) && pb.nsplit == 1) ? pb.cfg : 0;
}

template <typename T>
static bool launch_group(const tp_gemm_desc* descs, int n, int cfg, hipStream_t s) {
    constexpr bool AKM = false, BKM = false;     // TN: both operands token-major
    GemmGroupArgs ga;
    int tiles = 0;
    for (int i = 0; i < n; ++i) {
        GemmPlan p;                 // every member on the group's tiles, its whole k in one piece
        p.cfg = cfg;
        TileCfg tc;
        tile_cfg(cfg, tc);
        p.gx = (descs[i].N + tc.bn - 1) / tc.bn;
        p.gy = (descs[i].M + tc.bm - 1) / tc.bm;
        p.kper = descs[i].K; p.nsplit = 1;
        ga.g[i] = fill_args(&descs[i], p, nullptr);
        ga.first_tile[i] = tiles;
        ga.tiles_x[i] = p.gx;
        ga.tiles_y[i] = p.gy;
        tiles += p.gx * p.gy;
    }
    for (int i = n; i < kGroupMax; ++i) { ga.g[i] = ga.g[0]; ga.first_tile[i] = tiles; ga.tiles_x[i] = 1; ga.tiles_y[i] = 1; }
    ga.n = n;
    if (cfg == 2) gemm_tall_kernel<T, AKM, BKM, 256, 256, 32, 4, 2, 4, true, true><<<dim3(tiles), 512, 0, s>>>(ga);
    else if (cfg == 15) return launch_gemm_pipe_group(cfg, descs[0].dtype, tiles, ga, s);
    else if (cfg == 19) gemm_tall_kernel<T, AKM, BKM, 256, 256, 64, 4, 2, 2, true><<<dim3(tiles), 512, 0, s>>>(ga);
    else gemm_tall_kernel<T, AKM, BKM, 256, 256, 32, 4, 2, 4, true><<<dim3(tiles), 512, 0, s>>>(ga);
    return true;
}
}  // namespace tp

// ---------------------------------------------------------------------------------------------
// Workspace for callers that cannot allocate (tp_gemm_static_ws): the k-split partial sums go to a
// file-scope device array instead of a caller's buffer.  In host code the array's name is only a
// stand-in; its device address is asked for once per device and kept.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[TP_GEMM_STATIC_WS_BYTES];

namespace tp {
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the CURRENT device (nullptr + error text on failure)
static void* scratch_on_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("tp_gemm_static_ws: hipGetDevice failed or device index %d out of range: %s", dev, hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("tp_gemm_static_ws: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace tp

// Also looks up the array's address on the current device (a module and symbol lookup that must not happen while a
// stream capture is open): callers that capture tp_gemm_static_ws call this once per device beforehand.
extern "C" size_t tp_gemm_static_ws_capacity(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) == hipSuccess && n > 0) (void)tp::scratch_on_current_device();
    return (size_t)TP_GEMM_STATIC_WS_BYTES;
}

extern "C" int tp_gemm_static_ws(const tp_gemm_desc* d, void* stream) {
    int rc = tp::validate_gemm(d);
    if (rc != TP_OK) return rc;
    if (d->defer_reduce) {
        tp::set_error("tp_gemm_static_ws: defer_reduce hands the workspace to a later call; use tp_gemm");
        return TP_ERR_ARG;
    }
    tp::GemmPlan p = tp::plan_gemm(d);
    const size_t need = p.nsplit > 1 ? (size_t)p.nsplit * d->M * d->N * sizeof(float) : 0;
    if (need > (size_t)TP_GEMM_STATIC_WS_BYTES) {
        tp::set_error("tp_gemm_static_ws: this product needs %zu bytes of k-split workspace, the built-in one holds %zu "
                      "(M=%d N=%d K=%d, %d splits); use tp_gemm with a caller workspace",
                      need, (size_t)TP_GEMM_STATIC_WS_BYTES, d->M, d->N, d->K, p.nsplit);
        return TP_ERR_WORKSPACE;
    }
    void* ws = nullptr;
    if (need > 0) {
        ws = tp::scratch_on_current_device();
        if (!ws) return TP_ERR_LAUNCH;
    }
    return tp_gemm(d, ws, need, stream);
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
    tp::GemmArgs a = tp::fill_args(d, p, workspace);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    bool launched;
    switch (d->dtype) {
    case TP_F32: launched = tp::launch_gemm<float>(d, p, a, s); break;
    case TP_F16: launched = tp::launch_gemm<tp::f16>(d, p, a, s); break;
    default: launched = tp::launch_gemm<tp::bf16>(d, p, a, s); break;
    }
    if (!launched) {
        tp::set_error("tp_gemm: no kernel for tile configuration %d with op %d, dtype %d", p.cfg, d->op, d->dtype);
        return TP_ERR_UNSUPPORTED;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { tp::set_error("tp_gemm: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
    return TP_OK;
}

extern "C" int tp_gemm_group_cfg(const tp_gemm_desc* descs, int n) {
    if (!descs || n < 1) return 0;
    for (int i = 0; i < n; ++i)
        if (tp::validate_gemm(&descs[i]) != TP_OK) return 0;
    return tp::group_cfg(descs, n);
}

extern "C" int tp_gemm_grouped(const tp_gemm_desc* descs, int n, void* workspace, size_t workspace_bytes, void* stream) {
    if (!descs || n < 1) { tp::set_error("tp_gemm_grouped: bad argument"); return TP_ERR_ARG; }
    for (int i = 0; i < n; ++i) {
        int rc = tp::validate_gemm(&descs[i]);
        if (rc != TP_OK) return rc;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (const int cfg = tp::group_cfg(descs, n)) {
        const bool launched = descs[0].dtype == TP_F16 ? tp::launch_group<tp::f16>(descs, n, cfg, s)
                                                       : tp::launch_group<tp::bf16>(descs, n, cfg, s);
        if (!launched) {
            tp::set_error("tp_gemm_grouped: no kernel for tile configuration %d, dtype %d", cfg, descs[0].dtype);
            return TP_ERR_UNSUPPORTED;
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) { tp::set_error("tp_gemm_grouped: launch failed: %s", hipGetErrorString(e)); return TP_ERR_LAUNCH; }
        return TP_OK;
    }
    // any other group: its members one after the other (they share the workspace: same stream, in order)
    for (int i = 0; i < n; ++i) {
        int rc = tp_gemm(&descs[i], workspace, workspace_bytes, stream);
        if (rc != TP_OK) return rc;
    }
    return TP_OK;
}
