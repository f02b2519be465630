// Flash-style multi-head attention for gfx950 (forward, and a two-kernel deterministic backward)
// on v_mfma_f32_32x32x16_bf16, head dimension 64 or 128.
//
// Forward: a work-group owns 64 query rows of one (batch, head) and streams keys/values through LDS
// in blocks of 64 rows.  Its 4 waves are 2 groups of 32 query rows x 2 halves of every key block:
// the two waves of a row group keep separate softmax statistics and output accumulators over their
// 32 of every 64 keys and merge them once, through LDS, after the last block.  That halves the
// length of the dependent chain MFMA -> softmax -> MFMA per key block, which is what bounds a causal
// launch (its longest work-group, not its total work).  Scores are produced transposed,
// S^T[kv][q] = K Q^T, so that a lane holds one query column: the online-softmax statistics are
// per-lane scalars (one cross-lane exchange with lane^32 per reduction) and the probabilities sit
// in registers in exactly the form the second MFMA wants as its B operand for
// O^T[d][q] += V^T[d][kv] P^T[kv][q].
//
// Backward: one kernel parallel over query blocks (64 queries) produces dQ and delta = rowsum(dO * O),
// one kernel parallel over key blocks (64 keys) then produces dK and dV, with the same 2 x 2 split of
// the waves: partial sums of the two halves are added in a fixed order through LDS.  No atomics:
// results are run-to-run identical.
//
// Staging: every streamed operand is a block of 64 rows kept in LDS exactly as it lies in memory,
// as one 64 x 64 bf16 tile per 64 columns of the head ([row][d], 128 B per row, 16-byte chunks
// XOR-swizzled by the row), filled by direct-to-LDS buffer loads, three stages deep (two for head
// dimension 128) with one barrier per block of 64 rows.  A fragment whose MFMA k index
// runs along d is a ds_read_b128 of one row; a fragment whose k index runs along the tile's rows
// (V^T in the forward pass, K^T, Q^T and dO^T in the backward pass) comes out of the same tile
// through ds_read_b64_tr_b16, so no transposed copy is ever made.
#include "tile.h"
#include <math.h>

namespace pp {

struct AttnArgs {
    const uint16_t* q; const uint16_t* k; const uint16_t* v;
    uint16_t* o; float* lse;
    const uint16_t* d_o;
    uint16_t* dq; uint16_t* dk; uint16_t* dv;
    float* delta;
    int64_t B, S, H, D, stride_b, stride_s;
    int64_t G;  // query heads per key / value head (1: multi-head attention)
    int64_t L;  // keys 0 .. L-1 of a sequence exist (L <= S); the forward masks the rest
    float scale;
    // backward, head dimension 64: fp32 [B * S / 64][ld_cs], row b * (S / 64) + j receives the column sums
    // over block j (64 tokens) of dq, dk and dv as stored, at the columns that the elements have relative
    // to dq (cs_k, cs_v: where the dk and dv sections start); null: no sums
    float* colsum;
    int64_t ld_cs, cs_k, cs_v;
};

// Column sums of a 64 x 64 block that its owners have written to `cs` as [column][65] floats (row = token
// within the block): every wave adds 16 rows of each column in ascending order, wave 0 then adds the four
// partial sums in wave order and writes the 64 sums.  Called by all 256 threads of the work-group.
constexpr int kColsumScratchFloats = 64 * 65 + 4 * 64;
__device__ __forceinline__ void attn_block_column_sums(float* cs, int tid, float* out) {
    const int c = tid & 63, rq = tid >> 6;
    float t = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) t += cs[c * 65 + rq * 16 + r];
    float* part = cs + 64 * 65;
    part[rq * 64 + c] = t;
    __syncthreads();
    if (rq == 0) out[c] = ((part[c] + part[64 + c]) + part[128 + c]) + part[192 + c];
}

union Frag {
    uint4 u;
    bf16x8_t v;
};
__device__ __forceinline__ bf16x8_t pack8(const float* p) {
    Frag f;
    f.u = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]),
                     pack_bf16(p[6], p[7]));
    return f.v;
}

constexpr float kLog2e = 1.44269504088896340736f;
constexpr int kTile = 64 * 64;  // elements of one staged tile
// LDS stages: 3 x 16 KiB for head dimension 64 (three work-groups per CU), 2 x 32 KiB for 128
constexpr int attn_stages(int D) { return D == 64 ? 3 : 2; }

// Chunk swizzle of a staged tile.  Rows r and r+1 start 32 banks apart; the first term spreads 16
// consecutive rows read at one chunk index (ds_read_b128 fragments), the second separates rows r
// and r+2, which a transposing read touches together.
__device__ __forceinline__ int swz_attn(int r) { return ((r ^ (r >> 3)) & 7) ^ ((r & 2) << 1); }

// Direct-to-LDS loader of 64-row blocks out of a [rows][stride] operand: DS tiles of 64 columns
// (128 B per row and tile), tile s at lds + s * kTile.
// ASM: the loads go out as inline assembly (see tile.h), which lets tiles stay in flight across LDS reads.
// Measured on the three kernels it changed nothing (forward 1.92 against 1.95 ms, backward 5.12 against
// 5.29 ms per GPT-2-small step, within the scatter between machines): a work-group's chain of dependent
// block steps, not its loads, sets the pace.  The kernels stay on the builtin form.
template <int DS, bool ASM = false>
struct AttnTileLoader {
    typename std::conditional<ASM, LdsDmaRsrc, __amdgpu_buffer_rsrc_t>::type rsrc;
    int voff[2];
    int row_bytes;
    __device__ __forceinline__ void init(const uint16_t* base, int64_t stride, int64_t rows, int wave, int lane) {
        if constexpr (ASM) rsrc = make_lds_dma_rsrc(base, (uint64_t)rows * (uint64_t)stride * 2);
        else rsrc = make_rsrc(base, (uint64_t)rows * (uint64_t)stride * 2);
        row_bytes = (int)(stride * 2);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row = (i * 4 + wave) * 8 + (lane >> 3);
            voff[i] = row * row_bytes + (((lane & 7) ^ swz_attn(row)) << 4);
        }
    }
    // `extra_bytes` shifts the columns (another head of the same rows)
    __device__ __forceinline__ void load(uint16_t* lds, int64_t row0, int wave, int extra_bytes = 0) const {
#pragma unroll
        for (int s = 0; s < DS; ++s)
#pragma unroll
            for (int i = 0; i < 2; ++i)
                load_to_lds_b128(rsrc, lds + s * kTile + (i * 4 + wave) * 512, voff[i] + s * 128,
                                 (int)row0 * row_bytes + extra_bytes);
    }
};

// 64 consecutive floats into LDS with one wave instruction.
__device__ __forceinline__ void load_floats_to_lds(__amdgpu_buffer_rsrc_t rsrc, float* lds, int64_t first, int lane) {
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_ptr_t)lds, 4, lane * 4, (int)first * 4, 0, 0);
#endif
}

// Fragment with k along d: row `row` of the tile, 16-byte chunk `chunk`.
__device__ __forceinline__ bf16x8_t read_row_frag(const uint16_t* tile, int row, int chunk) {
    return *reinterpret_cast<const bf16x8_t*>(tile + row * 64 + ((chunk ^ swz_attn(row)) << 3));
}

// Fragment with k along the tile's rows, for 32 columns d0 .. d0+31 and the 16 rows r0 .. r0+15.
// The k slots of lane group g = lane / 32 are rows r0 + 4g .. + 3 and r0 + 8 + 4g .. + 3: the order
// in which a lane of a 32x32 MFMA result holds 8 of its 16 values, so that probabilities computed
// in registers can be the other operand without a shuffle.  Inside each block of 16 lanes, lane
// 4j + i fetches columns 4i .. 4i+3 of row j, and the hardware hands lane m the 4 rows of column m.
__device__ __forceinline__ bf16x8_t read_col_frag(const uint16_t* tile, int r0, int d0, int lane) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int g = lane >> 5, mb = (lane >> 4) & 1, j = (lane & 15) >> 2, i = lane & 3;
    const int d = d0 + 16 * mb + 4 * i;
    const int r_lo = r0 + 4 * g + j, r_hi = r_lo + 8;
    const uint16_t* p_lo = tile + r_lo * 64 + (((d >> 3) ^ swz_attn(r_lo)) << 3) + (d & 7);
    const uint16_t* p_hi = tile + r_hi * 64 + (((d >> 3) ^ swz_attn(r_hi)) << 3) + (d & 7);
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_t)p_lo);
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr_t)p_hi);
    const s16x8_t v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8_t, v);
#else
    return bf16x8_t{};
#endif
}

// Pipeline step shared by the three kernels: block j of `nb` has landed for every wave, and the
// stage that block j-1 occupied is free.  LPT loads per block per wave; with NS stages, NS - 2
// younger blocks may stay in flight.
template <int LPT, int NS>
__device__ __forceinline__ void await_block(int64_t j, int64_t nb) {
    static_assert(NS == 2 || NS == 3, "two or three stages");
    if (NS == 3 && j + 1 < nb) wait_vmcnt<(NS == 3 ? LPT : 0)>(); else wait_vmcnt<0>();
    wait_lds();
    __builtin_amdgcn_s_barrier();
}

extern __shared__ __attribute__((aligned(16))) uint16_t attn_lds[];

// Which (batch, head) and which block a work-group takes.  All work-groups of a (batch, head) stay on
// one XCD (their K and V share its L2).  `ord` counts a head's blocks from the longest: under a causal
// mask block `ord` of the query-parallel kernels is query block nx - 1 - ord (it sees the most keys), of
// the key-parallel kernel key block ord (it is seen by the most queries).
//
// A causal launch is bound by how its unequal blocks meet on the CUs.  Numbered head by head, the
// work-groups that arrive on an XCD one after the other repeat the same ramp of lengths for every head,
// and the CUs end up with very unequal sums (measured: as slow as the launch without a mask, which
// does twice the work).  Here the blocks of an XCD are ranked by length across its heads, every head's
// longest first, so that the work-groups which share a CU at any time are of about one length and the
// late arrivals are the short ones: 24.7 -> 18.9 us forward and 62.8 -> 49.3 us backward at
// [4, 12, 1024, 64].  (Dealing the ranked blocks to the CUs in rounds of alternating direction measured
// the same for every round length from 8 to 96; fewer resident work-groups per CU, which lets the
// dispatcher place the short blocks as slots free up, measured slower.)  The assignment is a
// permutation of the same work, so results do not depend on it.
__device__ __forceinline__ bool attn_block_of(uint32_t bid, uint32_t grid, uint32_t nx, uint32_t heads,
                                              bool balance, uint32_t* bh, uint32_t* ord) {
    if (balance && heads % 8 == 0) {
        const uint32_t x = bid & 7, t = bid >> 3;      // XCD, arrival order inside it
        const uint32_t g = heads / 8;                  // heads per XCD
        if (t >= nx * g) return false;
        *bh = x * g + t % g;
        *ord = t / g;
        return true;
    }
    const uint32_t vid = xcd_remap(bid, grid);
    if (vid >= nx * heads) return false;
    *bh = vid / nx;
    *ord = vid % nx;
    return true;
}

// ---- forward ----------------------------------------------------------------------------------
// WAVES = 4: key blocks of 64, each row group's two waves take 32 keys of every block.  WAVES = 8: key
// blocks of 128 and four waves per row group.  A launch of few, short heads is bound by the chain of
// dependent block steps of its longest work-group (load -> K Q^T -> softmax -> P V, about 0.6 us per
// step whatever shares the CU), not by arithmetic: eight waves walk that chain in half the steps.
template <int D, int WAVES>
struct AttnFwdCfg {
    static constexpr int kParts = WAVES / 2;             // waves per row group = parts of a key block
    static constexpr int kBlockKeys = 32 * kParts;       // keys per block
    static constexpr int kTilesPerOperand = (D / 64) * (kBlockKeys / 64);
    static constexpr int kOperand = kTilesPerOperand * kTile;
    static constexpr int kStage = 2 * kOperand;
    static constexpr int kStages = (D == 64 && WAVES == 4) ? 3 : 2;
    static constexpr size_t kMerge = (size_t)2 * (kParts - 1) * (16 * (D / 32) + 2) * 64 * 4;
    static constexpr size_t kLds = (size_t)kStages * kStage * 2 > kMerge ? (size_t)kStages * kStage * 2 : kMerge;
};

template <int D, bool CAUSAL, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES == 8 ? 2 : (D == 64 ? 3 : 2)) void attn_fwd_kernel(const AttnArgs a) {
    static_assert(D == 64 || D == 128, "head dimension 64 or 128");
    static_assert(WAVES == 4 || WAVES == 8, "two or four waves per row group");
    typedef AttnFwdCfg<D, WAVES> Cfg;
    constexpr int KS = D / 16, DT = D / 32, DS = D / 64, NS = Cfg::kStages;
    constexpr int P = Cfg::kParts, KB = Cfg::kBlockKeys, KT = KB / 64;  // KT: 64-row tiles per block and operand column
    constexpr int kOperand = Cfg::kOperand, kStage = Cfg::kStage;
    uint16_t* const lds = attn_lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave & 1, part = wave >> 1;
    const int l32 = lane & 31, lh = lane >> 5;
    const uint32_t nx = (uint32_t)(a.S / 64);
    uint32_t bh, ord;
    if (!attn_block_of(blockIdx.x, gridDim.x, nx, (uint32_t)(a.H * a.B), CAUSAL, &bh, &ord)) return;
    const int64_t b = bh / a.H, h = bh % a.H;
    const int64_t q0 = (int64_t)(CAUSAL ? nx - 1 - ord : ord) * 64;
    const int64_t qw0 = q0 + 32 * grp;
    const int64_t qi = qw0 + l32;  // this lane's query row

    const uint16_t* qp = a.q + b * a.stride_b + h * D;
    // the 64-row tiles of a block are loaded by sets of four waves: waves 4 .. 7 take the second 64 keys
    const int lset = wave >> 2, lwave = wave & 3;
    AttnTileLoader<DS> lk, lv;
    lk.init(a.k + b * a.stride_b + (h / a.G) * D, a.stride_s, a.S, lwave, lane);
    lv.init(a.v + b * a.stride_b + (h / a.G) * D, a.stride_s, a.S, lwave, lane);
    const int64_t n_keys = CAUSAL ? q0 + 64 : a.L;
    const int64_t n_blocks = (n_keys + KB - 1) / KB;
    // LDS layout of an operand: [64-key tile of the block][64 columns of d] tiles of 64 x 64
    auto issue = [&](int stage, int64_t j) {
        lk.load(lds + stage * kStage + lset * DS * kTile, j * KB + 64 * lset, lwave);
        lv.load(lds + stage * kStage + kOperand + lset * DS * kTile, j * KB + 64 * lset, lwave);
    };

    bf16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + qi * a.stride_s + 16 * ks + 8 * lh);
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
        if (t < n_blocks) issue(t, t);

    f32x16_t oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[t][e] = 0.f;
    // l_run is this lane's share of the row sum (the other 16 of the wave's 32 keys are the partner
    // lane's, lane ^ 32): the shares meet once, after the last block
    float m_run = -INFINITY, l_run = 0.f;
    const float c = a.scale * kLog2e;
    const int partner = (lane ^ 32) << 2;  // byte index of the lane that holds the same query column
    const int ktile = (32 * part) / 64, krow = (32 * part) % 64;  // this wave's keys inside the block

    // The loop over blocks is unrolled by the number of stages: the stage of a block is then a constant of
    // its copy of the loop body, and the LDS addresses of the fragment reads are per-lane offsets computed
    // once plus immediate offsets, instead of vector additions in every step.
    for (int64_t j0 = 0; j0 < n_blocks; j0 += NS)
      static_for<NS>([&](auto stage_c) {
        constexpr int stage = decltype(stage_c)::value;
        const int64_t j = j0 + stage;
        if (j >= n_blocks) return;
        const int64_t kt0 = j * KB + 32 * part;  // first key of this wave's part of the block
        await_block<4 * DS, NS>(j, n_blocks);
        if (j + NS - 1 < n_blocks) issue(stage == 0 ? NS - 1 : stage - 1, j + NS - 1);
        const uint16_t* Ks = lds + stage * kStage + ktile * DS * kTile;
        const uint16_t* Vs = Ks + kOperand;
        // keys past the sequence (a last block of 128 that is half full) or past every query of the wave
        const bool active = kt0 < a.L && (!CAUSAL || (kt0 <= qw0 + 31));
        if (active) {
            bf16x8_t kf[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) kf[ks] = read_row_frag(Ks + (ks / 4) * kTile, krow + l32, 2 * (ks % 4) + lh);
            f32x16_t sacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[e] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks], qf[ks], sacc, 0, 0, 0);
            // sacc[v]: kv = kt0 + 8 (v/4) + 4 lh + v%4, q = qi
            if (CAUSAL && (kt0 + 31 > qw0)) {  // wave-uniform: only blocks on the diagonal pay for the mask
                const int lim = (int)(qi - kt0) - 4 * lh;  // keys 8 (v/4) + v%4 up to lim are visible
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (8 * (v >> 2) + (v & 3) > lim) sacc[v] = -INFINITY;
            }
            if (kt0 + 31 >= a.L) {  // wave-uniform: the block that holds the end of a padded sequence
                const int lim = (int)(a.L - 1 - kt0) - 4 * lh;
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (8 * (v >> 2) + (v & 3) > lim) sacc[v] = -INFINITY;
            }
            float mloc = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) mloc = fmaxf(mloc, sacc[v]);
            // The reference maximum of a row only has to keep the exponentials in range, so it is
            // moved (and the accumulators rescaled) only when some row of the wave exceeds it by
            // more than 2^8 after scaling; that happens in the first block of a row and almost
            // never again.  Any reference gives the same softmax after the final division.  m_run
            // tracks the maximum of the raw scores (c > 0, so scaling commutes with max) and is the
            // same in both lanes of a query column.
            if (__ballot(mloc * c > m_run * c + 8.0f)) {
                mloc = fmaxf(mloc, __int_as_float(__builtin_amdgcn_ds_bpermute(partner, __float_as_int(mloc))));
                const float m_new = fmaxf(m_run, mloc);
                const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c);
                l_run *= alpha;
                m_run = m_new;
#pragma unroll
                for (int t = 0; t < DT; ++t)
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[t][e] *= alpha;
            }
            // a row whose keys have all been masked so far has no reference yet: its scores are -inf
            const float mc = (m_run == -INFINITY ? 0.f : m_run) * c;
            float psum = 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sacc[v], c, -mc));
                sacc[v] = p;
                psum += p;
            }
            l_run += psum;
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                float pv[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) pv[e] = sacc[8 * gp + e];
                const bf16x8_t pb = pack8(pv);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16x8_t vf = read_col_frag(Vs + (dt / 2) * kTile, krow + 16 * gp, 32 * (dt % 2), lane);
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb, oacc[dt], 0, 0, 0);
                }
            }
        }
      });
    l_run += __int_as_float(__builtin_amdgcn_ds_bpermute(partner, __float_as_int(l_run)));

    // merge the parts of every key block in a fixed order: [grp][part - 1][16 DT + 2 values][64 lanes] floats
    wait_lds();
    __syncthreads();
    constexpr int kVals = 16 * DT + 2;
    float* const xs0 = reinterpret_cast<float*>(lds) + grp * ((P - 1) * kVals * 64) + lane;
    if (part != 0) {
        float* xs = xs0 + (part - 1) * (kVals * 64);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) xs[(16 * dt + e) * 64] = oacc[dt][e];
        xs[16 * DT * 64] = m_run;
        xs[(16 * DT + 1) * 64] = l_run;
    }
    __syncthreads();
    if (part == 0) {
        float m = m_run;  // finite after the merge: key 0 is visible to every query
#pragma unroll
        for (int p = 1; p < P; ++p) m = fmaxf(m, xs0[(p - 1) * (kVals * 64) + 16 * DT * 64]);
        const float a0 = m_run == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_run - m) * c);
        float l = l_run * a0;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[dt][e] *= a0;
#pragma unroll
        for (int p = 1; p < P; ++p) {
            const float* xs = xs0 + (p - 1) * (kVals * 64);
            const float mp = xs[16 * DT * 64], lp = xs[(16 * DT + 1) * 64];
            const float ap = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mp - m) * c);
            l += lp * ap;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) oacc[dt][e] += xs[(16 * dt + e) * 64] * ap;
        }
        const float inv_l = 1.0f / l;
        uint16_t* op = a.o + (b * a.S + qi) * (a.H * D) + h * D;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = oacc[dt][4 * g + e] * inv_l;
                const int d = 32 * dt + 8 * g + 4 * lh;
                *reinterpret_cast<uint2*>(op + d) = make_uint2(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]));
            }
        if (lh == 0) a.lse[(b * a.H + h) * a.S + qi] = m * a.scale + logf(l);
    }
}

// ---- backward: dK, dV (parallel over key blocks) ------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256, D == 64 ? 3 : 1) void attn_bwd_dkv_kernel(const AttnArgs a) {
    static_assert(D == 64 || D == 128, "head dimension 64 or 128");
    constexpr int KS = D / 16, DT = D / 32, DS = D / 64, NS = attn_stages(D);
    constexpr int kOperand = DS * kTile;     // one staged 64-row block of Q or dO
    constexpr int kStage = 2 * kOperand + 256;  // Q, dO, 64 lse, 64 delta
    uint16_t* const lds = attn_lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave & 1, half = wave >> 1;  // 32 keys of the block x 32 of every 64 queries
    const int l32 = lane & 31, lh = lane >> 5;
    const uint32_t nx = (uint32_t)(a.S / 64);
    uint32_t bh, ord;
    // a work-group owns 64 keys of one key / value head and walks the query blocks of every query head
    // of its group, one head after the other
    const int64_t Hkv = a.H / a.G;
    if (!attn_block_of(blockIdx.x, gridDim.x, nx, (uint32_t)(Hkv * a.B), CAUSAL, &bh, &ord)) return;
    const int64_t b = bh / Hkv, hk = bh % Hkv, h = hk * a.G;  // h: first query head of the group
    const int64_t kv0 = (int64_t)ord * 64;  // early key blocks see the most queries
    const int64_t kvw0 = kv0 + 32 * grp;
    const int64_t kvi = kvw0 + l32;  // this lane's key row

    const uint16_t* kp = a.k + b * a.stride_b + hk * D;
    const uint16_t* vp = a.v + b * a.stride_b + hk * D;
    const int64_t ldo = a.H * D;
    AttnTileLoader<DS, false> lq, ldo_;
    lq.init(a.q + b * a.stride_b + h * D, a.stride_s, a.S, wave, lane);
    ldo_.init(a.d_o + b * a.S * ldo + h * D, ldo, a.S, wave, lane);
    // waves 0 and 2 fetch lse, waves 1 and 3 delta (the same values twice: every wave issues the
    // same number of loads, which keeps the vmcnt arithmetic uniform)
    const float* stat = ((wave & 1) ? a.delta : a.lse) + (b * a.H + h) * a.S;
    const __amdgpu_buffer_rsrc_t rstat = make_rsrc(stat, (uint64_t)a.G * (uint64_t)a.S * 4);
    const int stat_off = 2 * kOperand + ((wave & 1) ? 128 : 0);

    const int jq_begin = CAUSAL ? (int)(kv0 / 64) : 0;
    const int nb_head = (int)(a.S / 64) - jq_begin;  // query blocks that see these keys, per query head
    const int64_t nb = a.G * nb_head;                // steps: the blocks of head 0 of the group, of head 1, ...
    int iss_g = 0, iss_b = 0;                        // head and block of the next step to be issued
    auto issue = [&](int stage, int64_t) {           // steps are issued in order
        uint16_t* st = lds + stage * kStage;
        const int row0 = (jq_begin + iss_b) * 64;
        lq.load(st, row0, wave, iss_g * D * 2);
        ldo_.load(st + kOperand, row0, wave, iss_g * D * 2);
        load_floats_to_lds(rstat, reinterpret_cast<float*>(st + stat_off), iss_g * (int)a.S + row0, lane);
        if (++iss_b == nb_head) {
            iss_b = 0;
            ++iss_g;
        }
    };

    bf16x8_t kf[KS], vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kf[ks] = *reinterpret_cast<const bf16x8_t*>(kp + kvi * a.stride_s + 16 * ks + 8 * lh);
        vf[ks] = *reinterpret_cast<const bf16x8_t*>(vp + kvi * a.stride_s + 16 * ks + 8 * lh);
    }
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
        if (t < nb) issue(t, t);

    f32x16_t dvacc[DT], dkacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            dvacc[t][e] = 0.f;
            dkacc[t][e] = 0.f;
        }
    const float c = a.scale * kLog2e;

    // (not unrolled by the number of stages as the other two kernels are: the per-lane offsets of its 24
    // fragment reads per block would not fit the register budget of three work-groups per CU)
    int stage = 0, cur_b = 0;  // cur_b: block of the current step within its head
    for (int64_t j = 0; j < nb; ++j) {
        const int64_t qc0 = (int64_t)(jq_begin + cur_b) * 64;
        cur_b = cur_b + 1 == nb_head ? 0 : cur_b + 1;
        await_block<4 * DS + 1, NS>(j, nb);
        if (j + NS - 1 < nb) issue(stage == 0 ? NS - 1 : stage - 1, j + NS - 1);
        const uint16_t* Qs = lds + stage * kStage;
        const uint16_t* Os = Qs + kOperand;
        const float* lse_s = reinterpret_cast<const float*>(Qs + 2 * kOperand);
        const float* delta_s = lse_s + 64;
        stage = stage + 1 == NS ? 0 : stage + 1;
        const int qt = half;
        const int64_t qt0 = qc0 + 32 * qt;
        if (!CAUSAL || (qt0 + 31 >= kvw0)) {  // else every query precedes every key: masked
            f32x16_t sacc, dpacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sacc[e] = 0.f;
                dpacc[e] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8_t qfr = read_row_frag(Qs + (ks / 4) * kTile, 32 * qt + l32, 2 * (ks % 4) + lh);
                const bf16x8_t ofr = read_row_frag(Os + (ks / 4) * kTile, 32 * qt + l32, 2 * (ks % 4) + lh);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr, kf[ks], sacc, 0, 0, 0);
                dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ofr, vf[ks], dpacc, 0, 0, 0);
            }
            // element v: q = qt0 + 8 (v/4) + 4 lh + v%4, kv = kvi
            const bool diag = CAUSAL && (qt0 < kvw0 + 31);
            float pv[16], dsv[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 l4 = *reinterpret_cast<const float4*>(lse_s + 32 * qt + 8 * g + 4 * lh);
                const float lq4[4] = {l4.x * kLog2e, l4.y * kLog2e, l4.z * kLog2e, l4.w * kLog2e};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    pv[4 * g + e] = __builtin_amdgcn_exp2f(fmaf(sacc[4 * g + e], c, -lq4[e]));
            }
            if (diag) {  // wave-uniform: only blocks on the diagonal pay for the mask
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (kvi > qt0 + 8 * (v >> 2) + 4 * lh + (v & 3)) pv[v] = 0.f;
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 d4 = *reinterpret_cast<const float4*>(delta_s + 32 * qt + 8 * g + 4 * lh);
                const float dq4[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) dsv[4 * g + e] = pv[4 * g + e] * (dpacc[4 * g + e] - dq4[e]);
            }
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const bf16x8_t pb = pack8(pv + 8 * gp);
                const bf16x8_t dsb = pack8(dsv + 8 * gp);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16x8_t otf = read_col_frag(Os + (dt / 2) * kTile, 32 * qt + 16 * gp, 32 * (dt % 2), lane);
                    const bf16x8_t qtf = read_col_frag(Qs + (dt / 2) * kTile, 32 * qt + 16 * gp, 32 * (dt % 2), lane);
                    dvacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(otf, pb, dvacc[dt], 0, 0, 0);
                    dkacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtf, dsb, dkacc[dt], 0, 0, 0);
                }
            }
        }
    }
    // add the partial sums of the two query halves: [grp][16 DT values][64 lanes] floats, dV then dK
    wait_lds();
    __builtin_amdgcn_s_barrier();
    float* xs = reinterpret_cast<float*>(lds) + grp * (16 * DT * 64) + lane;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        f32x16_t(&acc)[DT] = pass == 0 ? dvacc : dkacc;
        if (half == 1) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) xs[(16 * dt + e) * 64] = acc[dt][e];
        }
        __syncthreads();
        if (half == 0) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[dt][e] += xs[(16 * dt + e) * 64];
        }
        __syncthreads();
    }
    // dvacc[dt][v]: d = 32 dt + 8 (v/4) + 4 lh + v%4, kv = kvi
    bool sums = false;
    if constexpr (D == 64) sums = a.colsum != nullptr;  // uniform over the grid
    if (half != 0 && !sums) return;
    // column sums of the two tiles: the exchange buffers above are done with, so the scratch starts at the
    // head of LDS: [dv, dk][64 columns][65], then [dv, dk][4 waves][64]
    float* cs = reinterpret_cast<float*>(lds);
    constexpr int kTileScratch = 64 * 65;
    const int row = 32 * grp + l32;
    if (half == 0) {
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            f32x16_t(&acc)[DT] = pass == 0 ? dvacc : dkacc;
            uint16_t* outp = (pass == 0 ? a.dv : a.dk) + b * a.stride_b + hk * D + kvi * a.stride_s;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d = 32 * dt + 8 * g + 4 * lh;
                    float v[4] = {acc[dt][4 * g + 0], acc[dt][4 * g + 1], acc[dt][4 * g + 2], acc[dt][4 * g + 3]};
                    if (pass == 1) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] *= a.scale;
                    }
                    const uint32_t w0 = pack_bf16(v[0], v[1]), w1 = pack_bf16(v[2], v[3]);
                    *reinterpret_cast<uint2*>(outp + d) = make_uint2(w0, w1);
                    if constexpr (D == 64) {
                        if (sums) {
                            float* t = cs + pass * kTileScratch + row;
                            t[(d + 0) * 65] = bf16lo(w0); t[(d + 1) * 65] = bf16hi(w0);
                            t[(d + 2) * 65] = bf16lo(w1); t[(d + 3) * 65] = bf16hi(w1);
                        }
                    }
                }
        }
    }
    if constexpr (D == 64) {
        if (sums) {
            __syncthreads();
            // every wave adds 16 rows of each column of both tiles in ascending order; waves 0 and 1 then
            // add the four partial sums of dv and of dk in wave order
            const int c = tid & 63, rq = tid >> 6;
            float* part = cs + 2 * kTileScratch;
#pragma unroll
            for (int pass = 0; pass < 2; ++pass) {
                float t = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) t += cs[pass * kTileScratch + c * 65 + rq * 16 + r];
                part[(pass * 4 + rq) * 64 + c] = t;
            }
            __syncthreads();
            if (rq < 2) {
                const float* pp_ = part + rq * 4 * 64 + c;
                float* out = a.colsum + (b * (a.S / 64) + kv0 / 64) * a.ld_cs + (rq == 0 ? a.cs_v : a.cs_k) + hk * D;
                out[c] = ((pp_[0] + pp_[64]) + pp_[128]) + pp_[192];
            }
        }
    }
}

// ---- backward: dQ (parallel over query blocks) ---------------------------------------------------
template <int D, bool CAUSAL, bool EXACT>
__global__ __launch_bounds__(256, D == 64 ? 3 : (EXACT ? 1 : 2)) void attn_bwd_dq_kernel(const AttnArgs a) {
    static_assert(D == 64 || D == 128, "head dimension 64 or 128");
    constexpr int KS = D / 16, DT = D / 32, DS = D / 64, NS = attn_stages(D);
    constexpr int kOperand = DS * kTile;   // one staged 64-row block of K or V
    constexpr int kStage = 2 * kOperand;
    uint16_t* const lds = attn_lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave & 1, half = wave >> 1;  // 32 queries of the block x 32 of every 64 keys
    const int l32 = lane & 31, lh = lane >> 5;
    const uint32_t nx = (uint32_t)(a.S / 64);
    uint32_t bh, ord;
    if (!attn_block_of(blockIdx.x, gridDim.x, nx, (uint32_t)(a.H * a.B), CAUSAL, &bh, &ord)) return;
    const int64_t b = bh / a.H, h = bh % a.H;
    const int64_t q0 = (int64_t)(CAUSAL ? nx - 1 - ord : ord) * 64;
    const int64_t qw0 = q0 + 32 * grp;
    const int64_t qi = qw0 + l32;

    const uint16_t* qp = a.q + b * a.stride_b + h * D;
    const int64_t ldo = a.H * D;
    const uint16_t* dop = a.d_o + b * a.S * ldo + h * D;
    AttnTileLoader<DS> lk, lv;
    lk.init(a.k + b * a.stride_b + (h / a.G) * D, a.stride_s, a.S, wave, lane);
    lv.init(a.v + b * a.stride_b + (h / a.G) * D, a.stride_s, a.S, wave, lane);
    const int64_t n_blocks = CAUSAL ? q0 / 64 + 1 : a.S / 64;
    auto issue = [&](int stage, int64_t j) {
        lk.load(lds + stage * kStage, j * 64, wave);
        lv.load(lds + stage * kStage + kOperand, j * 64, wave);
    };

    bf16x8_t qf[KS], dof[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + qi * a.stride_s + 16 * ks + 8 * lh);
        dof[ks] = *reinterpret_cast<const bf16x8_t*>(dop + qi * ldo + 16 * ks + 8 * lh);
    }
    float lse_q = a.lse[(b * a.H + h) * a.S + qi] * kLog2e;
    // delta = rowsum(dO * O) of this lane's query row: the lane pair (lh = 0, 1) holds the row of dO, so
    // the same pieces of O make the dot product; it is stored for the dK / dV kernel, which runs next
    float delta_q = 0.f;
    {
        const uint16_t* op = a.o + b * a.S * ldo + h * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            Frag x, y;
            x.v = dof[ks];
            y.u = *reinterpret_cast<const uint4*>(op + qi * ldo + 16 * ks + 8 * lh);
            delta_q += bf16lo(x.u.x) * bf16lo(y.u.x) + bf16hi(x.u.x) * bf16hi(y.u.x) +
                       bf16lo(x.u.y) * bf16lo(y.u.y) + bf16hi(x.u.y) * bf16hi(y.u.y) +
                       bf16lo(x.u.z) * bf16lo(y.u.z) + bf16hi(x.u.z) * bf16hi(y.u.z) +
                       bf16lo(x.u.w) * bf16lo(y.u.w) + bf16hi(x.u.w) * bf16hi(y.u.w);
        }
        delta_q += __shfl_xor(delta_q, 32, 64);
    }
    // The row sum above comes from the rounded output of the forward; the sum of P * dP over the keys, which
    // this kernel forms anyway, is the same number in exact arithmetic and the one that is consistent with
    // the dS = P (dP - delta) of both backward kernels (their rows then sum to zero).  It is only complete
    // after the loop: it is what the dK / dV kernel gets, and with EXACT this kernel corrects its own
    // result by the difference, dQ -= (D - delta) * (P K), at the cost of one more MFMA per block and tile
    // (the error term is a multiple of the attention-weighted mean key, which dwarfs the true gradient of
    // the queries where attention is nearly uniform and the keys share a large common part).
    float d_consistent = 0.f;
    f32x16_t pkacc[EXACT ? DT : 1];
    if constexpr (EXACT) {
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) pkacc[t][e] = 0.f;
    }
#pragma unroll
    for (int t = 0; t < NS - 1; ++t)
        if (t < n_blocks) issue(t, t);
    const float c = a.scale * kLog2e;

    f32x16_t dqacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dqacc[t][e] = 0.f;

    // unrolled by the number of stages (see the forward kernel)
    for (int64_t j0 = 0; j0 < n_blocks; j0 += NS)
      static_for<NS>([&](auto stage_c) {
        constexpr int stage = decltype(stage_c)::value;
        const int64_t j = j0 + stage;
        if (j >= n_blocks) return;
        const int64_t kv0 = j * 64;
        await_block<4 * DS, NS>(j, n_blocks);
        if (j + NS - 1 < n_blocks) issue(stage == 0 ? NS - 1 : stage - 1, j + NS - 1);
        const uint16_t* Ks = lds + stage * kStage;
        const uint16_t* Vs = Ks + kOperand;
        const int t = half;
        const int64_t kt0 = kv0 + 32 * t;
        if (!CAUSAL || (kt0 <= qw0 + 31)) {
            f32x16_t sacc, dpacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sacc[e] = 0.f;
                dpacc[e] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8_t kfr = read_row_frag(Ks + (ks / 4) * kTile, 32 * t + l32, 2 * (ks % 4) + lh);
                const bf16x8_t vfr = read_row_frag(Vs + (ks / 4) * kTile, 32 * t + l32, 2 * (ks % 4) + lh);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr, qf[ks], sacc, 0, 0, 0);
                dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr, dof[ks], dpacc, 0, 0, 0);
            }
            // element v: kv = kt0 + 8 (v/4) + 4 lh + v%4, q = qi
            const bool diag = CAUSAL && (kt0 + 31 > qw0);
            float dsv[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) dsv[v] = __builtin_amdgcn_exp2f(fmaf(sacc[v], c, -lse_q));
            if (diag) {  // wave-uniform: only blocks on the diagonal pay for the mask
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (kt0 + 8 * (v >> 2) + 4 * lh + (v & 3) > qi) dsv[v] = 0.f;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) d_consistent = fmaf(dsv[v], dpacc[v], d_consistent);
            bf16x8_t pb[EXACT ? 2 : 1];
            if constexpr (EXACT) {
                pb[0] = pack8(dsv);
                pb[1] = pack8(dsv + 8);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) dsv[v] *= dpacc[v] - delta_q;
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const bf16x8_t dsb = pack8(dsv + 8 * gp);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16x8_t ktf = read_col_frag(Ks + (dt / 2) * kTile, 32 * t + 16 * gp, 32 * (dt % 2), lane);
                    dqacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf, dsb, dqacc[dt], 0, 0, 0);
                    if constexpr (EXACT)
                        pkacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf, pb[gp], pkacc[dt], 0, 0, 0);
                }
            }
        }
      });
    // this lane's keys and its partner's (lane ^ 32) make the row's share of this wave
    d_consistent += __shfl_xor(d_consistent, 32, 64);
    // add the partial sums of the two key halves: [grp][(EXACT ? 32 : 16) DT + 1 values][64 lanes] floats
    wait_lds();
    __builtin_amdgcn_s_barrier();
    constexpr int kMergeVals = (EXACT ? 32 : 16) * DT + 1;
    float* xs = reinterpret_cast<float*>(lds) + grp * (kMergeVals * 64) + lane;
    if (half == 1) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                xs[(16 * dt + e) * 64] = dqacc[dt][e];
                if constexpr (EXACT) xs[(16 * DT + 16 * dt + e) * 64] = pkacc[dt][e];
            }
        xs[(kMergeVals - 1) * 64] = d_consistent;
    }
    __syncthreads();
    bool sums = false;
    if constexpr (D == 64) sums = a.colsum != nullptr;  // uniform over the grid
    if (half != 0 && !sums) return;
    float* cs = reinterpret_cast<float*>(lds) + 2 * (kMergeVals * 64);  // behind the exchange buffers
    if (half == 0) {
        d_consistent += xs[(kMergeVals - 1) * 64];
        if (lh == 0) a.delta[(b * a.H + h) * a.S + qi] = d_consistent;
        const float r = d_consistent - delta_q;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                dqacc[dt][e] += xs[(16 * dt + e) * 64];
                if constexpr (EXACT) dqacc[dt][e] -= r * (pkacc[dt][e] + xs[(16 * DT + 16 * dt + e) * 64]);
            }
        uint16_t* dqp = a.dq + b * a.stride_b + h * D + qi * a.stride_s;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int d = 32 * dt + 8 * g + 4 * lh;
                const uint32_t w0 = pack_bf16(dqacc[dt][4 * g + 0] * a.scale, dqacc[dt][4 * g + 1] * a.scale);
                const uint32_t w1 = pack_bf16(dqacc[dt][4 * g + 2] * a.scale, dqacc[dt][4 * g + 3] * a.scale);
                *reinterpret_cast<uint2*>(dqp + d) = make_uint2(w0, w1);
                if constexpr (D == 64) {
                    if (sums) {
                        const int row = 32 * grp + l32;
                        cs[(d + 0) * 65 + row] = bf16lo(w0); cs[(d + 1) * 65 + row] = bf16hi(w0);
                        cs[(d + 2) * 65 + row] = bf16lo(w1); cs[(d + 3) * 65 + row] = bf16hi(w1);
                    }
                }
            }
    }
    if constexpr (D == 64) {
        if (sums) {
            __syncthreads();
            attn_block_column_sums(cs, tid, a.colsum + (b * (a.S / 64) + q0 / 64) * a.ld_cs + h * D);
        }
    }
}

static int attn_check(const char* who, const pp_attn_desc* d, bool bwd) {
    if (!d) return fail(PP_ERR_INVALID, "%s: null descriptor", who);
    if (d->B < 0 || d->S < 0 || d->H <= 0) return fail(PP_ERR_INVALID, "%s: bad shape", who);
    if (d->D != 64 && d->D != 128)
        return fail(PP_ERR_UNSUPPORTED, "%s: head_dim %lld (64 and 128 are built)", who, (long long)d->D);
    if (d->S % 64) return fail(PP_ERR_UNSUPPORTED, "%s: S %% 64 != 0 (S=%lld)", who, (long long)d->S);
    if (d->kv_len < 0 || d->kv_len > d->S)
        return fail(PP_ERR_INVALID, "%s: kv_len %d outside [0, S = %lld]", who, d->kv_len, (long long)d->S);
    if (d->kv_group < 0 || (d->kv_group > 1 && d->H % d->kv_group))
        return fail(PP_ERR_INVALID, "%s: kv_group %d does not divide H = %lld", who, d->kv_group, (long long)d->H);
    if ((d->stride_s % 8) || (d->stride_b % 8)) return fail(PP_ERR_INVALID, "%s: strides must be multiples of 8", who);
    if (d->stride_s < d->H * d->D) return fail(PP_ERR_INVALID, "%s: stride_s < H*D", who);
    if (!d->q || !d->k || !d->v || !d->o || !d->lse) return fail(PP_ERR_INVALID, "%s: null pointer", who);
    if (!aligned(d->q, 16) || !aligned(d->k, 16) || !aligned(d->v, 16) || !aligned(d->o, 16))
        return fail(PP_ERR_INVALID, "%s: q/k/v/o must be 16-byte aligned", who);
    if (bwd) {
        if (!d->d_o || !d->dq || !d->dk || !d->dv || !d->delta) return fail(PP_ERR_INVALID, "%s: null pointer", who);
        if (!aligned(d->d_o, 16) || !aligned(d->dq, 16) || !aligned(d->dk, 16) || !aligned(d->dv, 16))
            return fail(PP_ERR_INVALID, "%s: gradients must be 16-byte aligned", who);
        if (d->colsum) {
            if (d->D != 64) return fail(PP_ERR_UNSUPPORTED, "%s: column sums are built for head_dim 64", who);
            const int64_t g = d->kv_group > 1 ? d->kv_group : 1;
            const int64_t off_k = static_cast<const uint16_t*>(d->dk) - static_cast<const uint16_t*>(d->dq);
            const int64_t off_v = static_cast<const uint16_t*>(d->dv) - static_cast<const uint16_t*>(d->dq);
            if (off_k < d->H * d->D || off_v < d->H * d->D || off_k + d->H / g * d->D > d->ld_colsum ||
                off_v + d->H / g * d->D > d->ld_colsum || d->H * d->D > d->ld_colsum)
                return fail(PP_ERR_INVALID, "%s: column sums need dq, dk, dv as sections of one row of at most "
                            "ld_colsum = %lld elements, dq first", who, (long long)d->ld_colsum);
        }
    }
    if ((d->S / 64) * d->H * d->B > 0x7fffff00ll) return fail(PP_ERR_UNSUPPORTED, "%s: grid too large", who);
    return PP_OK;
}

static AttnArgs to_args(const pp_attn_desc* d) {
    AttnArgs a;
    a.q = (const uint16_t*)d->q; a.k = (const uint16_t*)d->k; a.v = (const uint16_t*)d->v;
    a.o = (uint16_t*)d->o; a.lse = d->lse;
    a.d_o = (const uint16_t*)d->d_o;
    a.dq = (uint16_t*)d->dq; a.dk = (uint16_t*)d->dk; a.dv = (uint16_t*)d->dv;
    a.delta = d->delta;
    a.B = d->B; a.S = d->S; a.H = d->H; a.D = d->D;
    a.stride_b = d->stride_b; a.stride_s = d->stride_s;
    a.G = d->kv_group > 1 ? d->kv_group : 1;
    a.L = d->kv_len > 0 ? d->kv_len : d->S;
    a.scale = d->scale;
    a.colsum = d->dq ? d->colsum : nullptr;
    a.ld_cs = d->ld_colsum;
    a.cs_k = d->dq ? static_cast<const uint16_t*>(d->dk) - static_cast<const uint16_t*>(d->dq) : 0;
    a.cs_v = d->dq ? static_cast<const uint16_t*>(d->dv) - static_cast<const uint16_t*>(d->dq) : 0;
    return a;
}

// Dynamic LDS of the three kernels: stages, or the merge buffers of the epilogue if those are larger.
static size_t attn_lds_bytes(int D, bool dkv, bool exact_dq = false) {
    const size_t stage = (size_t)2 * (D / 64) * kTile * 2 + (dkv ? 512 : 0);
    // the exchange buffers of the epilogue and, behind them, the scratch of the column sums (head size 64)
    const size_t merge = (size_t)2 * ((exact_dq ? 32 : 16) * (D / 32) + 2) * 64 * 4 +
                         (D == 64 ? (size_t)kColsumScratchFloats * 4 : 0);
    const size_t stages = (size_t)attn_stages(D) * stage;
    return stages > merge ? stages : merge;
}

template <auto kernel>
static int attn_launch(const char* name, dim3 grid, int threads, size_t lds, hipStream_t st, const AttnArgs& a) {
    // one attribute call per kernel (the kernel is a template argument, so is the static) and process
    static const hipError_t attr_rc =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr_rc != hipSuccess)
        return fail(PP_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS: %s", name, lds, hipGetErrorString(attr_rc));
    hipLaunchKernelGGL(kernel, grid, dim3(threads), lds, st, a);
    return check_launch(name);
}

// Eight waves per work-group when the launch has fewer than two work-groups per CU: its duration is
// then the chain of its longest work-group (15.9 -> 10.9 us at [1, 12, 1024, 64] causal).  With more,
// the four-wave form's three work-groups per CU keep the CUs busy and its smaller key blocks waste less
// on the diagonal (18.6 against 20.6 us at [4, 12, 1024, 64] causal).
static bool attn_fwd_wide(const pp_attn_desc* d) {
    return d->D == 64 && (d->S / 64) * d->H * d->B < 2 * 256 && d->S >= 256;
}

template <int D>
static int attn_fwd_d(const pp_attn_desc* d, const AttnArgs& a, dim3 grid, hipStream_t st) {
    if constexpr (D == 64) {
        if (attn_fwd_wide(d)) {
            const size_t lds = AttnFwdCfg<D, 8>::kLds;
            return d->causal ? attn_launch<attn_fwd_kernel<D, true, 8>>("attn_fwd_kernel", grid, 512, lds, st, a)
                             : attn_launch<attn_fwd_kernel<D, false, 8>>("attn_fwd_kernel", grid, 512, lds, st, a);
        }
    }
    const size_t lds = AttnFwdCfg<D, 4>::kLds;
    return d->causal ? attn_launch<attn_fwd_kernel<D, true, 4>>("attn_fwd_kernel", grid, 256, lds, st, a)
                     : attn_launch<attn_fwd_kernel<D, false, 4>>("attn_fwd_kernel", grid, 256, lds, st, a);
}

template <int D>
static int attn_bwd_d(const pp_attn_desc* d, const AttnArgs& a, dim3 grid, hipStream_t st) {
    // the dQ kernel goes first: it also computes delta = rowsum(dO * O), which the dK / dV kernel reads
    const bool exact = (d->flags & PP_ATTN_EXACT_DQ) != 0;
    const size_t lds_kv = attn_lds_bytes(D, true), lds_q = attn_lds_bytes(D, false, exact);
    // one work-group per 64 keys of a key / value head
    const dim3 grid_kv((uint32_t)(((d->S / 64) * (d->H / a.G) * d->B + 7) / 8 * 8));
    int rc;
    if (d->causal) {
        rc = exact ? attn_launch<attn_bwd_dq_kernel<D, true, true>>("attn_bwd_dq_kernel", grid, 256, lds_q, st, a)
                   : attn_launch<attn_bwd_dq_kernel<D, true, false>>("attn_bwd_dq_kernel", grid, 256, lds_q, st, a);
        if (rc) return rc;
        return attn_launch<attn_bwd_dkv_kernel<D, true>>("attn_bwd_dkv_kernel", grid_kv, 256, lds_kv, st, a);
    }
    rc = exact ? attn_launch<attn_bwd_dq_kernel<D, false, true>>("attn_bwd_dq_kernel", grid, 256, lds_q, st, a)
               : attn_launch<attn_bwd_dq_kernel<D, false, false>>("attn_bwd_dq_kernel", grid, 256, lds_q, st, a);
    if (rc) return rc;
    return attn_launch<attn_bwd_dkv_kernel<D, false>>("attn_bwd_dkv_kernel", grid_kv, 256, lds_kv, st, a);
}

}  // namespace pp

using namespace pp;

extern "C" int pp_attn_fwd(const pp_attn_desc* d, pp_stream stream) {
    int rc = attn_check("pp_attn_fwd", d, false);
    if (rc) return rc;
    if (d->B == 0 || d->S == 0) return PP_OK;
    const AttnArgs a = to_args(d);
    const dim3 grid((uint32_t)(((d->S / 64) * d->H * d->B + 7) / 8 * 8));
    hipStream_t st = static_cast<hipStream_t>(stream);
    return d->D == 64 ? attn_fwd_d<64>(d, a, grid, st) : attn_fwd_d<128>(d, a, grid, st);
}

extern "C" int pp_attn_bwd(const pp_attn_desc* d, pp_stream stream) {
    int rc = attn_check("pp_attn_bwd", d, true);
    if (rc) return rc;
    if (d->B == 0 || d->S == 0) return PP_OK;
    const AttnArgs a = to_args(d);
    const dim3 grid((uint32_t)(((d->S / 64) * d->H * d->B + 7) / 8 * 8));
    hipStream_t st = static_cast<hipStream_t>(stream);
    return d->D == 64 ? attn_bwd_d<64>(d, a, grid, st) : attn_bwd_d<128>(d, a, grid, st);
}
