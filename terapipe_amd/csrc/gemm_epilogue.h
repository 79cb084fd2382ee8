// Pieces shared by the GEMM kernels of gemm.hip and gemm_pipe.hip: the argument block of a grouped launch, the
// epilogue, and the workgroup -> tile map.
#pragma once
#include "gemm_args.h"

namespace tp {

// Several GEMMs of one tile configuration in one launch (unsplit k): workgroup w works on one of the
// tiles_x[p] x tiles_y[p] tiles of problem p, the last p whose first_tile is <= w.
constexpr int kGroupMax = 4;
struct GemmGroupArgs {
    GemmArgs g[kGroupMax];
    int first_tile[kGroupMax];
    int tiles_x[kGroupMax];
    int tiles_y[kGroupMax];
    int n;
};

// Epilogue shared by the GEMM kernels.  Each wave transposes one 32x32 accumulator block at a time
// through its own LDS staging block so that a lane ends up with 8 consecutive columns of a row: 16-byte
// stores and a vector epilogue.  Lane -> (row = lane / 4 + 16 * pass, columns 8 * (lane % 4) .. + 7).
// `stage_base` must hold 32 * 36 floats per wave and must no longer be read as tile data by any wave.
// `write_block(ic, jc, stage)` puts the wave's 32x32 block (ic, jc) into `stage` (row pitch 36 floats).  A wave's tile
// is WROWS x WCOLS (multiples of 16): its last block row / column may be half a block.
template <typename T, int TM, int TN, int WM, int WN, int WROWS, int WCOLS, typename WriteBlock>
__device__ __forceinline__ void gemm_epilogue_blocks(const GemmArgs& a, WriteBlock&& write_block, float* stage_base,
                                                     int m0, int n0, int zsplit) {
    static_assert(WROWS <= TM * 32 && WROWS > TM * 32 - 32 && WCOLS <= TN * 32 && WCOLS > TN * 32 - 32, "block counts");
    constexpr int SPITCH = 36;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    float* stage = stage_base + wave * 32 * SPITCH;
    const int er = lane >> 2, ec = (lane & 3) * 8;
    static_for<TN>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        const int col0 = n0 + wn * WCOLS + j * 32 + ec;
        const bool col_in = (j + 1) * 32 <= WCOLS || ec < WCOLS - j * 32;      // compile-time true for whole blocks
        float csum[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) csum[e] = 0.f;
        static_for<TM>([&](auto ic) __attribute__((always_inline)) {
            constexpr int i = decltype(ic)::value;
            write_block(ic, jc, stage);
            // the block is private to the wave: LDS operations of one wave complete in order
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                const int rr = er + 16 * pass;
                const int row = m0 + wm * WROWS + i * 32 + rr;
                const bool row_in = (i + 1) * 32 <= WROWS || rr < WROWS - i * 32;
                float v[8];
                float4 v0 = *reinterpret_cast<const float4*>(stage + rr * SPITCH + ec);
                float4 v1 = *reinterpret_cast<const float4*>(stage + rr * SPITCH + ec + 4);
                v[0] = v0.x; v[1] = v0.y; v[2] = v0.z; v[3] = v0.w;
                v[4] = v1.x; v[5] = v1.y; v[6] = v1.z; v[7] = v1.w;
                if (row < a.M && col0 < a.N && row_in && col_in) {
                    if (a.nsplit > 1) {
                        float* dst = a.partial + ((long)zsplit * a.M + row) * a.N + col0;
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
        });
        if (a.nsplit == 1 && a.colsum && col_in) {
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
    });
}

// accumulators of 32x32 MFMA blocks: register r of block (i, j) is row acc_row(r, lane >> 5), column lane & 31
template <typename T, int TM, int TN, int WM, int WN>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, float16v (&acc)[TM][TN], float* stage_base,
                                              int m0, int n0, int zsplit) {
    const int lane = threadIdx.x & 63, g = lane >> 5, li = lane & 31;
    gemm_epilogue_blocks<T, TM, TN, WM, WN, TM * 32, TN * 32>(a, [&](auto ic, auto jc, float* stage) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
#pragma unroll
        for (int r = 0; r < 16; ++r) stage[acc_row(r, g) * 36 + li] = acc[i][j][r];
    }, stage_base, m0, n0, zsplit);
}

// accumulators of 16x16 MFMA blocks (TM x TN of them, either may be odd): register r of a block is row
// 4 * (lane >> 4) + r, column lane & 15
template <typename T, int TM, int TN, int WM, int WN>
__device__ __forceinline__ void gemm_epilogue16(const GemmArgs& a, float4v (&acc)[TM][TN], float* stage_base,
                                                int m0, int n0, int zsplit) {
    const int lane = threadIdx.x & 63, q = lane >> 4, c = lane & 15;
    gemm_epilogue_blocks<T, (TM + 1) / 2, (TN + 1) / 2, WM, WN, TM * 16, TN * 16>(
        a, [&](auto ic, auto jc, float* stage) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value, j = decltype(jc)::value;
        static_for<4>([&](auto dc) __attribute__((always_inline)) {
            constexpr int di = decltype(dc)::value >> 1, dj = decltype(dc)::value & 1;
            if constexpr (2 * i + di < TM && 2 * j + dj < TN) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    stage[(16 * di + 4 * q + r) * 36 + 16 * dj + c] = acc[2 * i + di][2 * j + dj][r];
            }
        });
    }, stage_base, m0, n0, zsplit);
}

// Which tile of a tx x ty tile grid the t-th workgroup of a launch (or of a problem of a grouped launch) takes.
// Workgroups go to the eight XCDs in turn, and each XCD has its own L2.  The tiles are laid out as a sequence
// that sweeps bands of four tile rows column by column, and XCD slot j = t mod 8 takes the j-th eighth of that
// sequence in order: the 32 tiles an XCD works on at a time form a 4 x 8 block that shares 12 operand slabs per
// k-tile, whatever the tile grid's width (with tiles numbered row by row a grid eight tiles wide gives an XCD one
// column: 33 slabs for 32 tiles).  A bijection of [0, tx * ty); every slot gets its share of the tiles to within one.
__device__ __forceinline__ void xcd_tile(int t, int tx, int ty, int& tile_x, int& tile_y) {
    const int n = tx * ty;
    const int j = t & 7, q = n >> 3, r = n & 7;
    const int seq = j * q + min(j, r) + (t >> 3);
    const int band = seq / (4 * tx), within = seq - band * 4 * tx;
    const int hb = min(4, ty - band * 4);
    tile_x = within / hb;
    tile_y = band * 4 + within % hb;
}
// The same over a launch with k splits (grid = tx x ty x tz, workgroup t = (z * ty + y) * tx + x): the sequence
// runs split by split, so an XCD's workgroups of a moment share one or two k ranges of the operands and its L2
// holds those, instead of every XCD reading every k range of the row operand.
__device__ __forceinline__ void xcd_tile3(int t, int tx, int ty, int tz, int& tile_x, int& tile_y, int& tile_z) {
    const int plane = tx * ty, n = plane * tz;
    const int j = t & 7, q = n >> 3, r = n & 7;
    const int seq = j * q + min(j, r) + (t >> 3);
    tile_z = seq / plane;
    const int in_plane = seq - tile_z * plane;
    const int band = in_plane / (4 * tx), within = in_plane - band * 4 * tx;
    const int hb = min(4, ty - band * 4);
    tile_x = within / hb;
    tile_y = band * 4 + within % hb;
}


// The pipelined tiles of gemm_pipe.hip (tile configurations 6, 7, 14, 15, 16, 41, 42, 43 of the plan): launches `cfg` on `grid` =
// (column tiles, row tiles, k splits); false when cfg / op / dtype has no such kernel.
bool launch_gemm_pipe(int cfg, int op, int dtype, dim3 grid, const GemmArgs& a, hipStream_t s);
// A grouped launch (TN, token-major operands) of `tiles` workgroups on the pipelined 256 x 128 tile.
bool launch_gemm_pipe_group(int cfg, int dtype, int tiles, const GemmGroupArgs& ga, hipStream_t s);

}  // namespace tp
