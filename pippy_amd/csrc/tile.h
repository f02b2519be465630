// LDS tile staging shared by the MFMA kernels (GEMM, attention).
//
// A tile is ROWS x KT bf16 (KT = 64 or 32 values of the reduction index).  Operand tiles are
// written to LDS by buffer loads with the lds modifier, never through registers.
//   * A "k-contiguous" operand (memory [rows][ld]) is held as [row][KT]; the 16-byte chunk index
//     is XORed with a function of the row so that the loads' writes and the ds_read_b128 fragment
//     reads cover all banks.
//   * A "transposed" operand (memory [k][ld], the tile's rows contiguous) is held as it lies in
//     memory, [KT][ROWS], and fragments come out through ds_read_b64_tr_b16.
// 256 lanes (4 waves) cooperate.
#pragma once
#include "common.h"
#include <type_traits>

namespace pp {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop that is unrolled by
// construction, for bodies that index register arrays with the loop variable.
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

constexpr int BK = 64;
constexpr int kGemmThreads = 256;

// Chunk swizzle of a k-contiguous tile with KT / 8 chunks per row: 8 chunks (128-byte rows) mix in
// row bits 0-2 and 3-5; 4 chunks (64-byte rows, four rows per 256 bytes of banks) use row bits 2-3.
template <int KT>
__device__ __forceinline__ int swz_kt(int row) {
    static_assert(KT == 64 || KT == 32, "tiles hold 64 or 32 values of k");
    return KT == 64 ? ((row ^ (row >> 3)) & 7) : ((row >> 2) & 3);
}
__device__ __forceinline__ int swz(int row) { return swz_kt<64>(row); }

// Consecutive hardware work-group ids go round-robin over the 8 XCDs, each with a private L2.  This
// remap gives every XCD a contiguous range of logical ids (the grid must be a multiple of 8 and
// logical ids past the real count are skipped by the caller), so that work-groups sharing operands
// share an L2.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t bid, uint32_t grid) {
    const uint32_t per_xcd = grid >> 3;
    return (bid & 7) * per_xcd + (bid >> 3);
}

// ---- buffer resources ------------------------------------------------------------------------
// Raw buffer loads are range-checked by the hardware: an address past the end of the operand
// returns zero, so rows (k-contiguous operands) and k indices (transposed operands) beyond the
// matrix need no branches, and 32-bit offsets replace 64-bit address arithmetic.  Operands must span
// less than 2 GiB from the tile origin.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint64_t bytes) {
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)n, 0x00020000);
}

// ---- direct-to-LDS staging -------------------------------------------------------------------
// A buffer load with the lds modifier writes each lane's 16 bytes to LDS at (wave-uniform base +
// 16 * lane) without passing through registers, so one wave instruction fills 1 KiB = 8 tile rows.
// The XOR swizzle is applied on the global side: lane l of a row fetches chunk (l & 7) ^ swz(row).
// Loads complete in order, so "tile t has landed" is a vmcnt wait that leaves the younger tiles in
// flight.
typedef __attribute__((address_space(3))) void* lds_void_ptr_t;

// The loads are written as inline assembly on purpose.  Issued through the compiler's builtin, the
// compiler knows that they write LDS, cannot tell which part, and therefore makes every later LDS read
// wait for ALL outstanding loads (s_waitcnt vmcnt(0) in front of the first fragment read of the next
// tile): the loads of tile t + 2 would then finish before tile t + 1 is touched, and nothing would
// overlap.  The kernels order loads and reads themselves, with explicit vmcnt waits and barriers: the
// statements carry no "memory" clobber (it would pin every LDS read of a loop body to its side of them);
// a stage is only ever refilled behind the barrier that follows its last read, and the compiler moves no
// memory access across a barrier.
struct LdsDmaRsrc {
    u32x4_t w;  // buffer resource words, wave-uniform (SGPRs)
};

__device__ __forceinline__ LdsDmaRsrc make_lds_dma_rsrc(const void* base, uint64_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    const uint32_t n = bytes > 0xffffffffull ? 0xffffffffu : (uint32_t)bytes;
    LdsDmaRsrc r;
    r.w.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
    r.w.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);  // stride 0: raw buffer
    r.w.z = __builtin_amdgcn_readfirstlane(n);
    r.w.w = 0x00020000u;
    return r;
}

// One wave load of 64 x 16 bytes to `lds_wave_base` + 16 * lane; `soffset` must be wave-uniform.
__device__ __forceinline__ void load_to_lds_b128(const LdsDmaRsrc& rsrc, uint16_t* lds_wave_base, int voffset,
                                                 int soffset) {
#if defined(__HIP_DEVICE_COMPILE__)
    const uint32_t lds_addr = (uint32_t)(uintptr_t)(lds_void_ptr_t)lds_wave_base;
    // s_mov + s_nop 3 = 5 wait states: what a VMEM instruction needs after a VALU instruction wrote one of
    // its SGPR operands (the compiler does not look for that hazard inside an asm statement), and more
    // than the one state that an M0 write needs before an LDS-direct load
    asm volatile("s_mov_b32 m0, %0\n\t"
                 "s_nop 3\n\t"
                 "buffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(voffset), "s"(rsrc.w),
                   "s"(__builtin_amdgcn_readfirstlane(soffset))
                 : "m0");
#endif
}

// The builtin form, for kernels that were tuned around the compiler's own waits (attention).
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

// W waves (4 or 8) cooperate on a tile.
template <int ROWS, bool TR, int KT = BK, int W = 4>
struct DmaStage;

// K-contiguous operand: memory [rows][ld]; LDS tile [ROWS][KT], chunk index XORed with swz_kt(row).
// One wave load fills 1 KiB: 8 rows of 64 k or 16 rows of 32 k.
template <int ROWS, int KT, int W>
struct DmaStage<ROWS, false, KT, W> {
    static constexpr int kChunks = KT / 8;              // 16-byte chunks per row
    static constexpr int kRowsPerLoad = 64 / kChunks;   // rows covered by one wave load
    static constexpr int kLoads = ROWS / kRowsPerLoad / W;
    static_assert(ROWS % (kRowsPerLoad * W) == 0, "tile rows must divide over the waves' loads");
    LdsDmaRsrc rsrc;
    int voff[kLoads];
    int kcol[kLoads];  // first k of this lane's chunk within a tile
    int K;
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int wave, int lane) {
        const uint64_t bytes = (uint64_t)(rows_total - row0) * (uint64_t)ld * 2;
        rsrc = make_lds_dma_rsrc(base + row0 * ld, bytes < 0x7ffffff0ull ? bytes : 0x7ffffff0ull);
        K = (int)K_;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int row = (i * W + wave) * kRowsPerLoad + lane / kChunks;
            const int ch = (lane % kChunks) ^ swz_kt<KT>(row);
            voff[i] = (int)((row * ld + ch * 8) * 2);
            kcol[i] = ch * 8;
        }
    }
    // Issues the loads of the k-tile starting at k0 into the LDS tile at `lds`.
    __device__ __forceinline__ void load(uint16_t* lds, int k0, int wave) const {
        if (k0 + KT <= K) {
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                load_to_lds_b128(rsrc, lds + (i * W + wave) * 512, voff[i], k0 * 2);
        } else {
            // k tail: chunks past K aim beyond the end of the buffer, which the range check zero-fills
#pragma unroll
            for (int i = 0; i < kLoads; ++i)
                load_to_lds_b128(rsrc, lds + (i * W + wave) * 512,
                                 k0 + kcol[i] < K ? voff[i] + k0 * 2 : (int)0x7ffffff0, 0);
        }
    }
};

// Transposed operand: memory [K][ld] with the tile's rows contiguous; LDS tile [KT][ROWS] as in
// memory, the 16-byte chunk index of k-row k XORed with (k & 3) << 2 so that the four k-rows a
// transposing read touches at once fall into different banks.
template <int ROWS, int KT, int W>
struct DmaStage<ROWS, true, KT, W> {
    static constexpr int kChunksPerRow = ROWS / 8;
    static constexpr int kRowsPerLoad = 64 / kChunksPerRow;
    static constexpr int kLoads = KT / kRowsPerLoad / W;
    static_assert(ROWS % 128 == 0 && ROWS <= 512, "transposed tiles are staged 128 rows at a time");
    static_assert(kLoads >= 1, "a wave load must not span more k-rows than a quarter of the tile");
    LdsDmaRsrc rsrc;
    int voff[kLoads];
    int ld2;  // bytes per k-row of the operand
    __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int64_t row0,
                                         int64_t rows_total, int64_t K_, int wave, int lane) {
        const uint64_t bytes = ((uint64_t)K_ * (uint64_t)ld - (uint64_t)row0) * 2;
        rsrc = make_lds_dma_rsrc(base + row0, bytes < 0x7ffffff0ull ? bytes : 0x7ffffff0ull);
        ld2 = (int)(ld * 2);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const int krow = (i * W + wave) * kRowsPerLoad + lane / kChunksPerRow;
            const int ch = (lane % kChunksPerRow) ^ ((krow & 3) << 2);
            const bool valid = row0 + ch * 8 < rows_total;
            // k is part of the lane offset so that k-rows past K fail the range check and read as 0
            voff[i] = valid ? (int)((krow * ld + ch * 8) * 2) : (int)0x7ffffff0;
        }
    }
    __device__ __forceinline__ void load(uint16_t* lds, int k0, int wave) const {
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            load_to_lds_b128(rsrc, lds + (i * W + wave) * 512, voff[i] + k0 * ld2, 0);
    }
};

// ---- MFMA operand fragments out of a staged tile ------------------------------------------------
// Fragment of v_mfma_f32_32x32x16_bf16 for 32 tile rows starting at r0: lane l holds, for row
// r0 + l % 32, the 8 consecutive k values 16 * ks + 8 * (l / 32) ...
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef short s16x8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr_t;

template <int ROWS, bool TR, int KT = BK>
struct FragReader;

template <int ROWS, int KT>
struct FragReader<ROWS, false, KT> {
    static constexpr int kReads = 1;  // LDS instructions per fragment
    int off, sw, lh;
    __device__ __forceinline__ void init(int r0, int lane) {
        const int r = r0 + (lane & 31);
        off = r * KT;
        sw = swz_kt<KT>(r);
        lh = lane >> 5;
    }
    __device__ __forceinline__ bf16x8_t read(const uint16_t* tile, int ks) const {
        return *reinterpret_cast<const bf16x8_t*>(tile + off + (((2 * ks + lh) ^ sw) << 3));
    }
};

// Transposing read: in each block of 16 lanes, lane 4 j + i fetches 4 consecutive rows
// (8 bytes) of k-row j, and ds_read_b64_tr_b16 hands lane m of the block the 4 k values of row m.
template <int ROWS, int KT>
struct FragReader<ROWS, true, KT> {
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
