// LDS tile staging shared by the MFMA kernels (GEMM, attention).
//
// A tile is ROWS x 64 bf16 held in LDS as [row][64] (128 B per row); the 16-byte chunk index is
// XORed with swz(row) so that staging writes and ds_read_b128 fragment reads cover all banks.
// Two sources: a "k-contiguous" operand (memory [rows][ld], 64 consecutive k per row) is copied
// chunk by chunk; a "transposed" operand (memory [k][ld], the tile's rows contiguous) is loaded as
// 4 k x 8 rows per lane and written as eight 8-byte k-runs.  256 lanes cooperate.
#pragma once
#include "common.h"

namespace pp {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int BK = 64;
constexpr int kGemmThreads = 256;

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// Consecutive hardware work-group ids go round-robin over the 8 XCDs, each with a private L2.  This
// remap gives every XCD a contiguous range of logical ids (the grid must be a multiple of 8 and
// logical ids past the real count are skipped by the caller), so that work-groups sharing operands
// share an L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t bid, uint32_t grid) {
    const uint32_t per_xcd = grid >> 3;
    return (bid & 7) * per_xcd + (bid >> 3);
}


// ---- global -> register staging -----------------------------------------------------------
// K-contiguous operand: memory [rows_total][ld], tile = ROWS x 64.
template <int ROWS>
__device__ __forceinline__ void gload_kc(uint4 (&r)[ROWS * 8 / kGemmThreads], const uint16_t* base,
                                         int64_t ld, int64_t row0, int64_t rows_total, int64_t k0,
                                         int64_t K, int tid) {
#pragma unroll
    for (int i = 0; i < ROWS * 8 / kGemmThreads; ++i) {
        const int id = tid + kGemmThreads * i;
        const int row = id >> 3, ch = id & 7;
        const int64_t gr = row0 + row, gk = k0 + ch * 8;
        if (gr < rows_total && gk < K)
            r[i] = *reinterpret_cast<const uint4*>(base + gr * ld + gk);
        else
            r[i] = make_uint4(0, 0, 0, 0);
    }
}
template <int ROWS>
__device__ __forceinline__ void sstore_kc(const uint4 (&r)[ROWS * 8 / kGemmThreads], uint16_t* lds,
                                          int tid) {
#pragma unroll
    for (int i = 0; i < ROWS * 8 / kGemmThreads; ++i) {
        const int id = tid + kGemmThreads * i;
        const int row = id >> 3, ch = id & 7;
        *reinterpret_cast<uint4*>(lds + row * BK + ((ch ^ swz(row)) << 3)) = r[i];
    }
}

// Transposed operand: memory [K][ld] with the tile's rows contiguous.  Half-block = 4 k x 8 rows.
template <int ROWS>
struct TrCfg {
    static constexpr int kHalfBlocks = (BK / 4) * (ROWS / 8);
    static constexpr int kPerThread = (kHalfBlocks + kGemmThreads - 1) / kGemmThreads;
};
template <int ROWS>
__device__ __forceinline__ void gload_tr(uint4 (&r)[TrCfg<ROWS>::kPerThread * 4],
                                         const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t k0, int64_t K, int tid) {
#pragma unroll
    for (int i = 0; i < TrCfg<ROWS>::kPerThread; ++i) {
        const int id = tid + kGemmThreads * i;
        const int mc = id % (ROWS / 8), kq = id / (ROWS / 8);
        const int64_t gr = row0 + mc * 8;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const int64_t gk = k0 + kq * 4 + kk;
            if (id < TrCfg<ROWS>::kHalfBlocks && gr < rows_total && gk < K)
                r[i * 4 + kk] = *reinterpret_cast<const uint4*>(base + gk * ld + gr);
            else
                r[i * 4 + kk] = make_uint4(0, 0, 0, 0);
        }
    }
}
__device__ __forceinline__ uint32_t word_of(const uint4& v, int w) {
    return w == 0 ? v.x : (w == 1 ? v.y : (w == 2 ? v.z : v.w));
}
template <int ROWS>
__device__ __forceinline__ void sstore_tr(const uint4 (&r)[TrCfg<ROWS>::kPerThread * 4],
                                          uint16_t* lds, int tid) {
#pragma unroll
    for (int i = 0; i < TrCfg<ROWS>::kPerThread; ++i) {
        const int id = tid + kGemmThreads * i;
        if (id < TrCfg<ROWS>::kHalfBlocks) {
            const int mc = id % (ROWS / 8), kq = id / (ROWS / 8);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int w = j >> 1;
                const uint32_t x0 = word_of(r[i * 4 + 0], w), x1 = word_of(r[i * 4 + 1], w);
                const uint32_t x2 = word_of(r[i * 4 + 2], w), x3 = word_of(r[i * 4 + 3], w);
                uint2 o;
                if (j & 1) {
                    o.x = (x0 >> 16) | (x1 & 0xffff0000u);
                    o.y = (x2 >> 16) | (x3 & 0xffff0000u);
                } else {
                    o.x = (x0 & 0xffffu) | (x1 << 16);
                    o.y = (x2 & 0xffffu) | (x3 << 16);
                }
                const int row = mc * 8 + j;
                *reinterpret_cast<uint2*>(lds + row * BK + (((kq >> 1) ^ swz(row)) << 3) +
                                          ((kq & 1) << 2)) = o;
            }
        }
    }
}

template <int ROWS, bool TR>
struct Stage;
template <int ROWS>
struct Stage<ROWS, false> {
    uint4 r[ROWS * 8 / kGemmThreads];
    __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t k0, int64_t K, int tid) {
        gload_kc<ROWS>(r, base, ld, row0, rows_total, k0, K, tid);
    }
    __device__ __forceinline__ void store(uint16_t* lds, int tid) { sstore_kc<ROWS>(r, lds, tid); }
};
template <int ROWS>
struct Stage<ROWS, true> {
    uint4 r[TrCfg<ROWS>::kPerThread * 4];
    __device__ __forceinline__ void load(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t k0, int64_t K, int tid) {
        gload_tr<ROWS>(r, base, ld, row0, rows_total, k0, K, tid);
    }
    __device__ __forceinline__ void store(uint16_t* lds, int tid) { sstore_tr<ROWS>(r, lds, tid); }
};


// ---- buffer-resource staging (branch-free global loads) ---------------------------------------
// Same tiles as above, loaded with raw buffer loads: the hardware range check returns zero for
// addresses past the end of the operand, so rows (k-contiguous operands) and k indices (transposed
// operands) beyond the matrix need no branches; 32-bit offsets replace 64-bit address arithmetic.
// The remaining edge (k tail of a k-contiguous operand, row tail of a transposed one) is masked
// with selects, and only in tiles that touch it.  Operands must span less than 4 GiB from the tile
// origin.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint64_t bytes) {
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}

template <int ROWS, bool TR, int NTHREADS = kGemmThreads>
struct BufStage;

template <int ROWS, int NTHREADS>
struct BufStage<ROWS, false, NTHREADS> {
    static constexpr int kChunks = ROWS * 8 / NTHREADS;
    static_assert(ROWS * 8 % NTHREADS == 0, "tile rows must divide evenly over the lanes");
    u32x4_t r[kChunks];
    __amdgpu_buffer_rsrc_t rsrc;
    int voff[kChunks];
    int soff[kChunks];
    int kcol;  // first k of this lane's chunk within a tile
    int K;
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int tid) {
        rsrc = make_rsrc(base + row0 * ld, (uint64_t)(rows_total - row0) * (uint64_t)ld * 2);
        K = (int)K_;
        kcol = (tid & 7) * 8;
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int id = tid + NTHREADS * i;
            const int row = id >> 3, ch = id & 7;
            voff[i] = (int)((row * ld + ch * 8) * 2);
            soff[i] = row * BK + ((ch ^ swz(row)) << 3);
        }
    }
    __device__ __forceinline__ void load(int k0) {
#pragma unroll
        for (int i = 0; i < kChunks; ++i)
            r[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[i] + k0 * 2, 0, 0);
        if (k0 + BK > K) {  // k tail: this lane's chunk may lie past K
            if (k0 + kcol >= K) {
#pragma unroll
                for (int i = 0; i < kChunks; ++i) r[i] = u32x4_t{0, 0, 0, 0};
            }
        }
    }
    __device__ __forceinline__ void store(uint16_t* lds) const {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) *reinterpret_cast<u32x4_t*>(lds + soff[i]) = r[i];
    }
};

template <int ROWS, int NTHREADS>
struct BufStage<ROWS, true, NTHREADS> {
    static constexpr int kHalfBlocks = (BK / 4) * (ROWS / 8);
    static constexpr int kPer = (kHalfBlocks + NTHREADS - 1) / NTHREADS;
    u32x4_t r[kPer * 4];
    __amdgpu_buffer_rsrc_t rsrc;
    int voff[kPer];
    int ld2;          // bytes per k row
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int tid) {
        const uint64_t bytes = ((uint64_t)K_ * (uint64_t)ld - (uint64_t)row0) * 2;
        // keep the "nothing to load" offset out of range: cap the resource below it
        rsrc = make_rsrc(base + row0, bytes < 0x7ffffff0ull ? bytes : 0x7ffffff0ull);
        ld2 = (int)(ld * 2);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int id = tid + NTHREADS * i;
            const int mc = id % (ROWS / 8), kq = id / (ROWS / 8);
            const bool valid = id < kHalfBlocks && (row0 + mc * 8 < rows_total);
            // lanes with nothing to load aim past the end of the buffer: the range check returns 0
            voff[i] = valid ? (int)((kq * 4 * ld + mc * 8) * 2) : (int)0x7ffffff0;
        }
    }
    __device__ __forceinline__ void load(int k0) {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                r[i * 4 + kk] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[i] + (k0 + kk) * ld2, 0, 0);
            }
        }
    }
    __device__ __forceinline__ void store(uint16_t* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int id = tid + NTHREADS * i;
            if (id < kHalfBlocks) {
                const int mc = id % (ROWS / 8), kq = id / (ROWS / 8);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int w = j >> 1;
                    const uint32_t x0 = r[i * 4 + 0][w], x1 = r[i * 4 + 1][w];
                    const uint32_t x2 = r[i * 4 + 2][w], x3 = r[i * 4 + 3][w];
                    uint2 o;
                    if (j & 1) {
                        o.x = (x0 >> 16) | (x1 & 0xffff0000u);
                        o.y = (x2 >> 16) | (x3 & 0xffff0000u);
                    } else {
                        o.x = (x0 & 0xffffu) | (x1 << 16);
                        o.y = (x2 & 0xffffu) | (x3 << 16);
                    }
                    const int row = mc * 8 + j;
                    *reinterpret_cast<uint2*>(lds + row * BK + (((kq >> 1) ^ swz(row)) << 3) +
                                              ((kq & 1) << 2)) = o;
                }
            }
        }
    }
    __device__ __forceinline__ void store(uint16_t* lds) const { store(lds, threadIdx.x); }
};

// ---- direct-to-LDS staging -------------------------------------------------------------------
// A buffer load with the lds modifier writes each lane's 16 bytes to LDS at (wave-uniform base +
// 16 * lane) without passing through registers, so one wave instruction fills 1 KiB = 8 tile rows.
// The XOR swizzle is applied on the global side: lane l of a row fetches chunk (l & 7) ^ swz(row).
// Loads complete in order, so "tile t has landed" is a vmcnt wait that leaves the younger tiles in
// flight.  Only k-contiguous operands can be staged this way.
typedef __attribute__((address_space(3))) void* lds_void_ptr_t;

__device__ __forceinline__ void load_to_lds_b128(__amdgpu_buffer_rsrc_t rsrc, uint16_t* lds_wave_base,
                                                 int voffset, int soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr_t)lds_wave_base, 16, voffset, soffset, 0, 0);
#endif
}

// s_waitcnt with only the vector-memory counter constrained (N outstanding loads allowed).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}
// s_waitcnt lgkmcnt(0): every LDS access of this wave has completed.
__device__ __forceinline__ void wait_lds() { __builtin_amdgcn_s_waitcnt(0xC07F); }

template <int ROWS, bool TR>
struct DmaStage;

// K-contiguous operand: memory [rows][ld]; LDS tile [ROWS][64 k], chunk index XORed with swz(row).
template <int ROWS>
struct DmaStage<ROWS, false> {
    static constexpr int kLoads = ROWS / 8 / 4;  // 1 KiB pieces per wave, 4 waves
    static_assert(ROWS % 32 == 0, "tile rows must divide over 4 waves x 8 rows");
    __amdgpu_buffer_rsrc_t rsrc;
    int voff[kLoads];
    int kcol[kLoads];  // first k of this lane's chunk within a tile
    int K;
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int wave, int lane) {
        const uint64_t bytes = (uint64_t)(rows_total - row0) * (uint64_t)ld * 2;
        rsrc = make_rsrc(base + row0 * ld, bytes < 0x7ffffff0ull ? bytes : 0x7ffffff0ull);
        K = (int)K_;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int row = (i * 4 + wave) * 8 + (lane >> 3);
            const int ch = (lane & 7) ^ swz(row);
            voff[i] = (int)((row * ld + ch * 8) * 2);
            kcol[i] = ch * 8;
        }
    }
    // Issues the loads of the k-tile starting at k0 into the LDS tile at `lds`.
    __device__ __forceinline__ void load(uint16_t* lds, int k0, int wave) const {
        if (k0 + BK <= K) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                load_to_lds_b128(rsrc, lds + (i * 4 + wave) * 512, voff[i], k0 * 2);
        } else {
            // k tail: chunks past K aim beyond the end of the buffer, which the range check zero-fills
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                load_to_lds_b128(rsrc, lds + (i * 4 + wave) * 512,
                                 k0 + kcol[i] < K ? voff[i] + k0 * 2 : (int)0x7ffffff0, 0);
        }
    }
};

// Transposed operand: memory [K][ld] with the tile's rows contiguous; LDS tile [64 k][ROWS] as in
// memory, the 16-byte chunk index of k-row k XORed with (k & 3) << 2 so that the four k-rows a
// transposing read touches at once fall into different banks.
template <int ROWS>
struct DmaStage<ROWS, true> {
    static constexpr int kChunksPerRow = ROWS / 8;
    static constexpr int kRowsPerLoad = 64 / kChunksPerRow;
    static constexpr int kLoads = BK / kRowsPerLoad / 4;
    static_assert(ROWS % 128 == 0 && ROWS <= 512, "transposed tiles are staged 128 rows at a time");
    __amdgpu_buffer_rsrc_t rsrc;
    int voff[kLoads];
    int ld2;  // bytes per k-row of the operand
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int wave, int lane) {
        const uint64_t bytes = ((uint64_t)K_ * (uint64_t)ld - (uint64_t)row0) * 2;
        rsrc = make_rsrc(base + row0, bytes < 0x7ffffff0ull ? bytes : 0x7ffffff0ull);
        ld2 = (int)(ld * 2);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int krow = (i * 4 + wave) * kRowsPerLoad + lane / kChunksPerRow;
            const int ch = (lane % kChunksPerRow) ^ ((krow & 3) << 2);
            const bool valid = row0 + ch * 8 < rows_total;
            // k is part of the lane offset so that k-rows past K fail the range check and read as 0
            voff[i] = valid ? (int)((krow * ld + ch * 8) * 2) : (int)0x7ffffff0;
        }
    }
    __device__ __forceinline__ void load(uint16_t* lds, int k0, int wave) const {
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            load_to_lds_b128(rsrc, lds + (i * 4 + wave) * 512, voff[i] + k0 * ld2, 0);
    }
};

// ---- MFMA operand fragments out of a staged tile ------------------------------------------------
// Fragment of v_mfma_f32_32x32x16_bf16 for 32 tile rows starting at r0: lane l holds, for row
// r0 + l % 32, the 8 consecutive k values 16 * ks + 8 * (l / 32) ...
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr_t;

template <int ROWS, bool TR>
struct FragReader;

template <int ROWS>
struct FragReader<ROWS, false> {
    static constexpr int kReads = 1;  // LDS instructions per fragment
    int off, sw, lh;
    __device__ __forceinline__ void init(int r0, int lane) {
        const int r = r0 + (lane & 31);
        off = r * BK;
        sw = swz(r);
        lh = lane >> 5;
    }
    __device__ __forceinline__ bf16x8_t read(const uint16_t* tile, int ks) const {
        return *reinterpret_cast<const bf16x8_t*>(tile + off + (((2 * ks + lh) ^ sw) << 3));
    }
};

// Transposing read: in each block of 16 lanes, lane 4 j + i fetches 4 consecutive rows
// (8 bytes) of k-row j, and ds_read_b64_tr_b16 hands lane m of the block the 4 k values of row m.
template <int ROWS>
struct FragReader<ROWS, true> {
    static constexpr int kReads = 2;
    int off;
    __device__ __forceinline__ void init(int r0, int lane) {
        const int blk = lane >> 4, g = blk >> 1, mb = blk & 1;
        const int j = (lane & 15) >> 2, i = lane & 3;
        const int m = r0 + 16 * mb + 4 * i;
        off = (8 * g + j) * ROWS + (((m >> 3) ^ (j << 2)) << 3) + (m & 7);
    }
    __device__ __forceinline__ bf16x8_t read(const uint16_t* tile, int ks) const {
#if defined(__HIP_DEVICE_COMPILE__)
        const uint16_t* p = tile + off + ks * 16 * ROWS;
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_t)p);
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_t)(p + 4 * ROWS));
        const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(bf16x8_t, v);
#else
        return bf16x8_t{};
#endif
    }
};

}  // namespace pp
