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

}  // namespace pp
