// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of the sliced GPT-layer path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "../../include/terapipe_hip.h"

namespace tp {

typedef _Float16 f16;
typedef __bf16 bf16;

typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));

#define TP_LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// ---------------------------------------------------------------------------------------------
// Element traits.  KP = k-values one lane feeds to one 32x32 MFMA; KSTEP = k covered by one MFMA.
// 16-bit types use v_mfma_f32_32x32x16_{f16,bf16}: lane l holds row/col (l & 31) and the 8
// consecutive k values 8 * (l >> 5) ... + 7.  fp32 uses v_mfma_f32_32x32x2_f32: lane l holds
// row/col (l & 31) and k = (l >> 5).  The 32x32 fp32 accumulator is 16 registers per lane:
// acc[j] is row 8 * (j / 4) + 4 * (l >> 5) + (j % 4), column (l & 31).
// ---------------------------------------------------------------------------------------------
template <typename T> struct Elem;

template <> struct Elem<f16> {
    static constexpr int KP = 8, KSTEP = 16, CH = 8;
    typedef uint4 opnd_t;
    static __device__ __forceinline__ float16v mfma(opnd_t a, opnd_t b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                     __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_float(f16 x) { return (float)x; }
    static __device__ __forceinline__ f16 from_float(float x) { return (f16)x; }
};

template <> struct Elem<bf16> {
    static constexpr int KP = 8, KSTEP = 16, CH = 8;
    typedef uint4 opnd_t;
    static __device__ __forceinline__ float16v mfma(opnd_t a, opnd_t b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                      __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_float(bf16 x) { return (float)x; }
    static __device__ __forceinline__ bf16 from_float(float x) { return (bf16)x; }
};

template <> struct Elem<float> {
    static constexpr int KP = 1, KSTEP = 2, CH = 4;
    typedef float opnd_t;
    static __device__ __forceinline__ float16v mfma(opnd_t a, opnd_t b, float16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_float(float x) { return x; }
    static __device__ __forceinline__ float from_float(float x) { return x; }
};

// Row of accumulator register j for the lane's k-group g = lane >> 5.
__device__ __forceinline__ int acc_row(int j, int g) { return 8 * (j >> 2) + 4 * g + (j & 3); }

// ---------------------------------------------------------------------------------------------
// LDS tiles.  A tile is ROWS x COLS elements, COLS contiguous, exactly as it lies in global memory.
// 16-bit tiles are XOR-swizzled at 16-byte chunk granularity so that both access patterns used by
// the MFMA operand fetches are free of avoidable bank conflicts:
//   (a) "k-major" fetch: 16 consecutive rows, the same 16-byte chunk (ds_read_b128), and
//   (b) "transposed" fetch: ds_read_b64_tr_b16 over 4 consecutive rows x 64 bytes.
// KM16 selects the mask for tiles whose only fetch is the k-major one of the 16x16x32 blocks (16 rows x 4
// chunks a read): the LDS serves a ds_read_b128 in four groups of lanes that the masks of (a) and (b) leave
// two-way conflicted for that shape (SQ_LDS_BANK_CONFLICT / SQ_LDS_IDX_ACTIVE 0.49 against 0.00 with these).
// fp32 tiles are padded by 4 floats per row instead.
// ---------------------------------------------------------------------------------------------
template <int COLS, bool KM16 = false> __device__ __forceinline__ int swz16(int row) {
    // returns the chunk XOR mask for a 16-bit tile with COLS elements per row
    if constexpr (KM16 && COLS == 64) {
        return (row >> 1) & 7;
    } else if constexpr (KM16 && COLS == 32) {
        return (row >> 1) & 3;
    } else if constexpr (COLS >= 128) {
        return ((row & 3) << 2) | ((row >> 2) & 3);
    } else if constexpr (COLS == 64) {
        return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
    } else if constexpr (COLS == 32) {
        return (row >> 2) & 3;
    } else {
        return 0;
    }
}

template <typename T, int COLS, bool KM16 = false> struct TileLayout {
    static constexpr bool kSwz = (sizeof(T) == 2);
    static constexpr int LD = kSwz ? COLS : COLS + 4;   // row pitch in elements
    // element offset of (row, col); for swizzled tiles col's 8-element chunk index is permuted
    static __device__ __forceinline__ int off(int row, int col) {
        if constexpr (kSwz) {
            return row * LD + ((((col >> 3) ^ swz16<COLS, KM16>(row)) << 3) | (col & 7));
        } else {
            return row * LD + col;
        }
    }
    static constexpr int size(int rows) { return rows * LD; }
};

// Cooperative global -> register -> LDS copy of a ROWS x COLS tile by NT threads, 16 bytes a chunk.
// Chunks wholly outside [0, rmax) x [0, cmax) are zero-filled (cmax and the leading dimension must be
// multiples of the chunk length, which the host checks).
template <typename T, int ROWS, int COLS, int NT> struct TileCopy {
    static constexpr int CH = 16 / sizeof(T);
    static constexpr int CPR = COLS / CH;
    static constexpr int TOTAL = ROWS * CPR;
    static constexpr int N = (TOTAL + NT - 1) / NT;
    uint4 r[N];

    __device__ __forceinline__ void load(const T* __restrict__ base, long ld, int r0, int c0, int rmax,
                                         int cmax, int tid) {
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int c = tid + i * NT;
            int row = c / CPR, cc = c % CPR;
            int gr = r0 + row, gc = c0 + cc * CH;
            uint4 v = make_uint4(0, 0, 0, 0);
            if ((TOTAL % NT == 0 || c < TOTAL) && gr < rmax && gc < cmax)
                v = *reinterpret_cast<const uint4*>(base + (long)gr * ld + gc);
            r[i] = v;
        }
    }
    __device__ __forceinline__ void store(T* lds, int tid) const {
        typedef TileLayout<T, COLS> L;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            int c = tid + i * NT;
            int row = c / CPR, cc = c % CPR;
            if (TOTAL % NT == 0 || c < TOTAL)
                *reinterpret_cast<uint4*>(lds + L::off(row, cc * CH)) = r[i];
        }
    }
};

// MFMA operand fetches from an LDS tile.
//   fetch_km: operand whose k runs along the tile's columns.  `row` is the lane's own row
//             (tile-relative, already including lane & 31); k0 the first column of this k-step.
//   fetch_tr: operand whose k runs along the tile's rows (two ds_read_b64_tr_b16 per operand).
//             `col0` is the first of the 32 columns of the MFMA block.  Natural order: k-slot e of lane
//             group g is row krow0 + 8 * g + e, the same k the k-major fetch gives that slot.
//             Interleaved order: slot e of group g is row krow0 + 8 * (e / 4) + 4 * g + (e % 4), the
//             order in which a 32x32 accumulator lays rows over registers, so that eight accumulator
//             registers of another MFMA can be fed back as the matching operand without a shuffle.
//             For fp32 (natural only) the single k-slot of group g is row krow0 + g.
template <typename T, int COLS>
__device__ __forceinline__ typename Elem<T>::opnd_t fetch_km(const T* tile, int row, int k0, int lane) {
    typedef TileLayout<T, COLS> L;
    int g = lane >> 5;
    if constexpr (sizeof(T) == 2) {
        return *reinterpret_cast<const uint4*>(tile + L::off(row, k0 + 8 * g));
    } else {
        return tile[L::off(row, k0 + g)];
    }
}

template <typename T, int COLS, bool INTERLEAVED>
__device__ __forceinline__ typename Elem<T>::opnd_t fetch_tr(const T* tile, int krow0, int col0, int lane) {
    typedef TileLayout<T, COLS> L;
    int g = lane >> 5;
    if constexpr (sizeof(T) == 2) {
        int p = lane & 15;
        int col = col0 + 16 * ((lane & 31) >> 4) + 4 * (p & 3);
        int r0 = krow0 + (INTERLEAVED ? 4 * g : 8 * g) + (p >> 2);
        int r1 = r0 + (INTERLEAVED ? 8 : 4);
        short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TP_LDS_PTR(short4v, tile + L::off(r0, col)));
        short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TP_LDS_PTR(short4v, tile + L::off(r1, col)));
        uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
        return make_uint4(l2.x, l2.y, h2.x, h2.y);
    } else {
        static_assert(!INTERLEAVED || sizeof(T) == 2, "fp32 interleaved fetches address rows directly");
        return tile[L::off(krow0 + g, col0 + (lane & 31))];
    }
}

// The same fetches split into "compute the lane's LDS offset once" and "load from a precomputed
// address", for loops that revisit the same tile positions (the offsets do not depend on the k-tile).
template <typename T, int COLS>
__device__ __forceinline__ int km_offset(int row, int k0, int lane) {
    static_assert(sizeof(T) == 2, "16-bit tiles");
    return TileLayout<T, COLS>::off(row, k0 + 8 * (lane >> 5));
}
template <typename T, int COLS, bool INTERLEAVED>
__device__ __forceinline__ void tr_offsets(int krow0, int col0, int lane, int& o0, int& o1) {
    static_assert(sizeof(T) == 2, "16-bit tiles");
    typedef TileLayout<T, COLS> L;
    const int g = lane >> 5, p = lane & 15;
    const int col = col0 + 16 * ((lane & 31) >> 4) + 4 * (p & 3);
    const int r0 = krow0 + (INTERLEAVED ? 4 * g : 8 * g) + (p >> 2);
    o0 = L::off(r0, col);
    o1 = L::off(r0 + (INTERLEAVED ? 8 : 4), col);
}
// the transposed fetch of a 16x16x32 operand: k-slot e of the lane's group q = lane >> 4 is row krow0 + 8 * q + e,
// the lane's row / column of the block is col0 + (lane & 15)
template <typename T, int COLS>
__device__ __forceinline__ void tr_offsets16(int krow0, int col0, int lane, int& o0, int& o1) {
    static_assert(sizeof(T) == 2, "16-bit tiles");
    typedef TileLayout<T, COLS> L;
    const int q = lane >> 4, p = lane & 15;
    const int col = col0 + 4 * (p & 3);
    const int r0 = krow0 + 8 * q + (p >> 2);
    o0 = L::off(r0, col);
    o1 = L::off(r0 + 4, col);
}
template <typename T> __device__ __forceinline__ uint4 load_km(const T* p) {
    return *reinterpret_cast<const uint4*>(p);
}
template <typename T> __device__ __forceinline__ uint4 load_tr(const T* p0, const T* p1) {
    short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TP_LDS_PTR(short4v, p0));
    short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(TP_LDS_PTR(short4v, p1));
    uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
    return make_uint4(l2.x, l2.y, h2.x, h2.y);
}

// Pack 8 fp32 accumulator values (registers j0 .. j0+7 of a 32x32 block) into one 16-bit MFMA operand.
template <typename T>
__device__ __forceinline__ uint4 pack8(const float* v) {
    T h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = Elem<T>::from_float(v[e]);
    return *reinterpret_cast<uint4*>(h);
}

template <typename T> __device__ __forceinline__ void store4(T* dst, float a, float b, float c, float d) {
    if constexpr (sizeof(T) == 2) {
        T h[4] = {Elem<T>::from_float(a), Elem<T>::from_float(b), Elem<T>::from_float(c), Elem<T>::from_float(d)};
        *reinterpret_cast<uint2*>(dst) = *reinterpret_cast<uint2*>(h);
    } else {
        *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
    }
}

template <typename T> __device__ __forceinline__ void load4(const T* src, float* out) {
    if constexpr (sizeof(T) == 2) {
        uint2 raw = *reinterpret_cast<const uint2*>(src);
        const T* h = reinterpret_cast<const T*>(&raw);
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = Elem<T>::to_float(h[e]);
    } else {
        float4 v = *reinterpret_cast<const float4*>(src);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// ---------------------------------------------------------------------------------------------
// Direct global -> LDS tile loads (global_load_lds_dwordx4).  A wave instruction writes 64 consecutive
// 16-byte chunks of LDS, so the XOR swizzle of the tile layout is applied on the global side: the lane
// that fills LDS chunk (row, pc) loads the global chunk (row, pc ^ swz(row)).  Chunks outside the matrix
// are loaded from a zero buffer so that every lane issues every load and the per-tile vmcnt accounting
// is exact.  The loads are inline asm: the compiler does not see them as LDS writes (it would otherwise
// force vmcnt(0) before every ds_read); kernels wait with wait_vmcnt<n>() + s_barrier once per tile.
// ---------------------------------------------------------------------------------------------
static __device__ __attribute__((aligned(16))) unsigned int g_zero_chunk[4] = {0u, 0u, 0u, 0u};

__device__ __forceinline__ void dma16(const void* gptr, const void* lds_wave_base) {
    unsigned lds = (unsigned)(unsigned long)(__attribute__((address_space(3))) const void*)lds_wave_base;
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds)) : "memory");
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N <= 63, "vmcnt immediate is 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}

// Tile loads for a tile that slides along one axis in equal steps (the k loop of a GEMM): the per-lane source
// pointers are computed once, every step is one 64-bit add per load.  `ALONG_COLS` says whether the tile slides along its columns (k-major operand) or its rows.
// Lanes whose fixed coordinate is outside the matrix point at the zero chunk with stride 0; the sliding
// coordinate is checked only on the steps the caller flags as possibly partial.
template <typename T, int ROWS, int COLS, int NT, bool ALONG_COLS> struct SlidingTileDma {
    static constexpr int CPR = COLS / 8;
    static constexpr int TOTAL = ROWS * CPR;
    static constexpr int N = TOTAL / NT;
    static_assert(TOTAL % NT == 0 && NT % 64 == 0, "tile must split evenly over the waves");
    const char* ptr[N];     // source of this lane's chunk in the NEXT tile to issue
    long step[N];           // bytes to advance per tile (0 for lanes pinned to the zero chunk)
    int slide[N];           // offset of this lane's chunk along the sliding axis inside a tile
    int pos;                // sliding coordinate of the next tile to issue, relative to the start

    // fixed0 / fixed_max: first coordinate and bound of the axis that does not slide;
    // slide0: start of the sliding axis; tile_step: elements to slide per tile.
    __device__ __forceinline__ void init(const T* __restrict__ base, long ld, int fixed0, int fixed_max,
                                         int slide0, int tile_step, int tid) {
        const int lane = tid & 63, wave = tid >> 6;
        pos = 0;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = (i * (NT / 64) + wave) * 64 + lane;
            const int row = p / CPR, pc = p % CPR;
            const int lc = pc ^ swz16<COLS>(row);
            const int fx = ALONG_COLS ? row : lc * 8;
            slide[i] = ALONG_COLS ? lc * 8 : row;
            const bool ok = fixed0 + fx < fixed_max;
            const long gr = ALONG_COLS ? fixed0 + fx : slide0 + slide[i];
            const long gc = ALONG_COLS ? slide0 + slide[i] : fixed0 + fx;
            ptr[i] = ok ? reinterpret_cast<const char*>(base + gr * ld + gc)
                        : reinterpret_cast<const char*>(g_zero_chunk);
            step[i] = ok ? (ALONG_COLS ? (long)tile_step : (long)tile_step * ld) * (long)sizeof(T) : 0;
        }
    }
    // issues the next tile; `len` is the extent of the sliding axis from its start, `tile_step` as in
    // init.  Chunks at or beyond len load zeros.
    __device__ __forceinline__ void issue(T* lds, int len, int tile_step, int tid) {
        const int wave = tid >> 6;
        if (pos + tile_step <= len) {          // uniform: the whole tile is inside
#pragma unroll
            for (int i = 0; i < N; ++i) {
                dma16(ptr[i], lds + (i * (NT / 64) + wave) * 512);
                ptr[i] += step[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                const void* src = pos + slide[i] < len ? (const void*)ptr[i] : (const void*)g_zero_chunk;
                dma16(src, lds + (i * (NT / 64) + wave) * 512);
                ptr[i] += step[i];
            }
        }
        pos += tile_step;
    }
};

// Loads whose source is a wave-uniform 64-bit base in SGPRs plus a 32-bit per-lane byte offset (no vector ALU
// work for the address), with the LDS destination (byte address of the wave's first chunk, wave-uniform) given
// as an integer, which spares the null check of a generic-to-LDS pointer cast per load.
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(unsigned long)(__attribute__((address_space(3))) const void*)p;
}
// Tells the compiler that a pointer is the same in every lane (moves it to scalar registers).
template <typename P> __device__ __forceinline__ P* uniform_ptr(P* p) {
    unsigned long v = (unsigned long)p;
    unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
    unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (P*)(((unsigned long)hi << 32) | lo);
}
__device__ __forceinline__ void dma16_saddr_lds(unsigned off, const void* sbase, unsigned lds_wave_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(off), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)) : "memory");
}

// One dword per lane into 256 bytes of LDS at lds_wave_base (wave-uniform byte address).
__device__ __forceinline__ void dma4(const void* gptr, unsigned lds_wave_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off"
                 :: "v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_wave_base)) : "memory");
}

// Tile loads for full tiles only: the lane's chunk is a loop-invariant 32-bit byte offset from a wave-uniform
// tile origin that advances by a scalar step, so a tile costs one VGPR per load and no vector ALU work.
// Coordinates of the fixed axis beyond the matrix are CLAMPED to the last valid row / chunk (the caller never
// stores results that depend on them); the sliding axis must be a whole number of tiles.
template <typename T, int ROWS, int COLS, int NT, bool ALONG_COLS, bool KM16 = false> struct ClampTileDma {
    static constexpr int CPR = COLS / 8;
    static constexpr int TOTAL = ROWS * CPR;
    static constexpr int N = TOTAL / NT;
    static_assert(TOTAL % NT == 0 && NT % 64 == 0, "tile must split evenly over the waves");
    unsigned off[N];
    const char* origin;     // wave-uniform
    long step;              // bytes per tile

    __device__ __forceinline__ void init(const T* __restrict__ base, long ld, int fixed0, int fixed_max,
                                         int slide0, int tile_step, int tid) {
        const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int p = (i * (NT / 64) + wave) * 64 + lane;
            const int row = p / CPR, pc = p % CPR;
            const int lc = pc ^ swz16<COLS, KM16>(row);
            int fx = ALONG_COLS ? row : lc * 8;
            const int sl = ALONG_COLS ? lc * 8 : row;
            const int last = fixed_max - (ALONG_COLS ? 1 : 8) - fixed0;
            fx = fx < last ? fx : last;
            off[i] = (unsigned)((ALONG_COLS ? (long)fx * ld + sl : (long)sl * ld + fx) * (long)sizeof(T));
        }
        origin = reinterpret_cast<const char*>(base + (ALONG_COLS ? (long)fixed0 * ld + slide0 : (long)slide0 * ld + fixed0));
        step = (ALONG_COLS ? (long)tile_step : (long)tile_step * ld) * (long)sizeof(T);
    }
    // lds_bytes: LDS byte address of the tile (an integer: no generic-pointer cast and its null check per load);
    // wave_uniform: the wave's index, already in a scalar register.
    __device__ __forceinline__ void issue(unsigned lds_bytes, int wave_uniform) {
        const char* o = uniform_ptr(origin);
#pragma unroll
        for (int i = 0; i < N; ++i)
            dma16_saddr_lds(off[i], o, lds_bytes + (unsigned)((i * (NT / 64) + wave_uniform) * 512 * (int)sizeof(T)));
        origin += step;
    }
    // the same, one load at a time (for loops that spread a tile's loads between other instructions): load i of
    // the tile at `origin`; `advance` moves on to the next tile
    __device__ __forceinline__ void issue_one(int i, unsigned lds_bytes, int wave_uniform) const {
        dma16_saddr_lds(off[i], uniform_ptr(origin), lds_bytes + (unsigned)((i * (NT / 64) + wave_uniform) * 512 * (int)sizeof(T)));
    }
    __device__ __forceinline__ void advance() { origin += step; }
};

// error plumbing shared by the host-side entry points
void set_error(const char* fmt, ...);

}  // namespace tp
