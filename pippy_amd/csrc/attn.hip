// Flash-style multi-head attention for gfx950 (forward, and a two-kernel deterministic backward)
// on v_mfma_f32_32x32x16_bf16.
//
// Forward: a work-group owns 128 query rows of one (batch, head); each of its 4 waves owns 32 rows.
// Keys/values stream through LDS in blocks of 64.  Scores are produced transposed,
// S^T[kv][q] = K Q^T, so that a lane holds one query column: the online-softmax statistics are
// per-lane scalars (one cross-lane exchange with lane^32 per reduction) and the probabilities sit
// in registers in exactly the form the second MFMA wants as its B operand for
// O^T[d][q] += V^T[d][kv] P^T[kv][q].  V is transposed on its way into LDS.
//
// Backward: delta = rowsum(dO * O); one kernel parallel over key blocks produces dK and dV, one
// kernel parallel over query blocks produces dQ.  No atomics: results are run-to-run identical.
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
    float scale;
};

union Frag {
    uint4 u;
    bf16x8_t v;
};

// Two 8-byte k-runs (chunks chunk0 and chunk0 + 1, offset 4*lh) of one row of a swizzled tile.
__device__ __forceinline__ bf16x8_t read_runs(const uint16_t* tile, int row, int chunk0, int lh) {
    const uint2 a = *reinterpret_cast<const uint2*>(tile + row * BK + (((chunk0) ^ swz(row)) << 3) + 4 * lh);
    const uint2 b = *reinterpret_cast<const uint2*>(tile + row * BK + (((chunk0 + 1) ^ swz(row)) << 3) + 4 * lh);
    Frag f;
    f.u = make_uint4(a.x, a.y, b.x, b.y);
    return f.v;
}
__device__ __forceinline__ bf16x8_t read_chunk(const uint16_t* tile, int row, int chunk) {
    return *reinterpret_cast<const bf16x8_t*>(tile + row * BK + ((chunk ^ swz(row)) << 3));
}
__device__ __forceinline__ bf16x8_t pack8(const float* p) {
    Frag f;
    f.u = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]),
                     pack_bf16(p[6], p[7]));
    return f.v;
}

constexpr float kLog2e = 1.44269504088896340736f;
constexpr float kLn2 = 0.69314718055994530942f;

// ---- forward ----------------------------------------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_fwd_kernel(const AttnArgs a) {
    constexpr int DS = D / 64;   // 64-wide sub-tiles along d
    constexpr int KS = D / 16;   // MFMA k steps along d
    constexpr int DT = D / 32;   // 32-row tiles of O^T
    __shared__ __attribute__((aligned(16))) uint16_t Ks[DS][64 * BK];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[D * BK];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t b = blockIdx.z, h = blockIdx.y;
    // causal: late query blocks have the most key blocks; launch them first
    const int64_t q0 = (int64_t)(CAUSAL ? gridDim.x - 1 - blockIdx.x : blockIdx.x) * 128;
    const int64_t qw0 = q0 + 32 * wave;
    const int64_t qi = qw0 + l32;  // this lane's query row

    const uint16_t* qp = a.q + b * a.stride_b + h * D;
    const uint16_t* kp = a.k + b * a.stride_b + h * D;
    const uint16_t* vp = a.v + b * a.stride_b + h * D;

    bf16x8_t qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + qi * a.stride_s + 16 * ks + 8 * lh);

    f32x16_t oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[t][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const float c = a.scale * kLog2e;

    const int64_t n_blocks = CAUSAL ? (q0 + 128 + 63) / 64 : a.S / 64;
    Stage<64, false> sk[DS];
    Stage<D, true> sv;
#pragma unroll
    for (int s = 0; s < DS; ++s) sk[s].load(kp, a.stride_s, 0, a.S, 64 * s, D, tid);
    sv.load(vp, a.stride_s, 0, D, 0, a.S, tid);

    for (int64_t j = 0; j < n_blocks; ++j) {
        const int64_t kv0 = j * 64;
#pragma unroll
        for (int s = 0; s < DS; ++s) sk[s].store(Ks[s], tid);
        sv.store(Vt, tid);
        __syncthreads();
        if (j + 1 < n_blocks) {
#pragma unroll
            for (int s = 0; s < DS; ++s) sk[s].load(kp, a.stride_s, kv0 + 64, a.S, 64 * s, D, tid);
            sv.load(vp, a.stride_s, 0, D, kv0 + 64, a.S, tid);
        }
        const bool active = !CAUSAL || (kv0 <= qw0 + 31);
        if (active) {
            f32x16_t sacc[2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) sacc[t][e] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const bf16x8_t kf = read_chunk(Ks[ks / 4], 32 * t + l32, 2 * (ks % 4) + lh);
                    sacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[ks], sacc[t], 0, 0, 0);
                }
            }
            // sacc[t][v]: kv = kv0 + 32 t + 8 (v/4) + 4 lh + v%4, q = qi
            const bool diag = CAUSAL && (kv0 + 63 > qw0);
            // m_run tracks the maximum of the raw scores; c > 0, so scaling commutes with max
            float mloc = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    if (diag) {
                        const int64_t kv = kv0 + 32 * t + 8 * (v >> 2) + 4 * lh + (v & 3);
                        if (kv > qi) sacc[t][v] = -INFINITY;
                    }
                    mloc = fmaxf(mloc, sacc[t][v]);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            const float m_new = fmaxf(m_run, mloc);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
            const float mc = m_new * c;
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float p = __builtin_amdgcn_exp2f(fmaf(sacc[t][v], c, -mc));
                    sacc[t][v] = p;
                    psum += p;
                }
            psum += __shfl_xor(psum, 32, 64);
            l_run = l_run * alpha + psum;
            m_run = m_new;
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int e = 0; e < 16; ++e) oacc[t][e] *= alpha;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int gp = 0; gp < 2; ++gp) {
                    float pv[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) pv[e] = sacc[t][8 * gp + e];
                    const bf16x8_t pb = pack8(pv);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const bf16x8_t vf = read_runs(Vt, 32 * dt + l32, 4 * t + 2 * gp, lh);
                        oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb, oacc[dt], 0, 0, 0);
                    }
                }
        }
        __syncthreads();
    }

    const float inv_l = 1.0f / l_run;
    uint16_t* op = a.o + (b * a.S + qi) * (a.H * D) + h * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * dt + 8 * g + 4 * lh;
            *reinterpret_cast<uint2*>(op + d) =
                make_uint2(pack_bf16(oacc[dt][4 * g + 0] * inv_l, oacc[dt][4 * g + 1] * inv_l),
                           pack_bf16(oacc[dt][4 * g + 2] * inv_l, oacc[dt][4 * g + 3] * inv_l));
        }
    if (lh == 0) a.lse[(b * a.H + h) * a.S + qi] = m_run * a.scale + logf(l_run);
}

// ---- backward: delta[b, h, q] = sum_d dO * O ---------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_delta_kernel(const AttnArgs a) {
    constexpr int LPH = D / 8;  // lanes per head
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // over B*S
    if (row >= a.B * a.S) return;
    const int64_t bidx = row / a.S, q = row - bidx * a.S;
    const int64_t width = a.H * D;
    const int nchunk = (int)(width >> 3);
    for (int c0 = 0; c0 < nchunk; c0 += 64) {
        const int cidx = c0 + lane;
        float s = 0.f;
        if (cidx < nchunk) {
            const uint4 x = *reinterpret_cast<const uint4*>(a.d_o + row * width + (int64_t)cidx * 8);
            const uint4 y = *reinterpret_cast<const uint4*>(a.o + row * width + (int64_t)cidx * 8);
            s = bf16lo(x.x) * bf16lo(y.x) + bf16hi(x.x) * bf16hi(y.x) + bf16lo(x.y) * bf16lo(y.y) +
                bf16hi(x.y) * bf16hi(y.y) + bf16lo(x.z) * bf16lo(y.z) + bf16hi(x.z) * bf16hi(y.z) +
                bf16lo(x.w) * bf16lo(y.w) + bf16hi(x.w) * bf16hi(y.w);
        }
#pragma unroll
        for (int o = LPH / 2; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (cidx < nchunk && (lane % LPH) == 0) {
            const int64_t h = cidx / LPH;
            a.delta[(bidx * a.H + h) * a.S + q] = s;
        }
    }
}

// ---- backward: dK, dV (parallel over key blocks) ------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_dkv_kernel(const AttnArgs a) {
    constexpr int DS = D / 64, KS = D / 16, DT = D / 32;
    __shared__ __attribute__((aligned(16))) uint16_t Qs[DS][64 * BK];   // [q][d]
    __shared__ __attribute__((aligned(16))) uint16_t Os[DS][64 * BK];   // dO [q][d]
    __shared__ __attribute__((aligned(16))) uint16_t Qt[D * BK];        // [d][q]
    __shared__ __attribute__((aligned(16))) uint16_t Ot[D * BK];        // dO [d][q]
    __shared__ __attribute__((aligned(16))) float lse_s[64];
    __shared__ __attribute__((aligned(16))) float delta_s[64];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t b = blockIdx.z, h = blockIdx.y;
    const int64_t kv0 = (int64_t)blockIdx.x * 128;
    const int64_t kvw0 = kv0 + 32 * wave;
    const int64_t kvi = kvw0 + l32;  // this lane's key row

    const uint16_t* qp = a.q + b * a.stride_b + h * D;
    const uint16_t* kp = a.k + b * a.stride_b + h * D;
    const uint16_t* vp = a.v + b * a.stride_b + h * D;
    const int64_t ldo = a.H * D;
    const uint16_t* dop = a.d_o + b * a.S * ldo + h * D;
    const float* lsep = a.lse + (b * a.H + h) * a.S;
    const float* deltap = a.delta + (b * a.H + h) * a.S;

    bf16x8_t kf[KS], vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        kf[ks] = *reinterpret_cast<const bf16x8_t*>(kp + kvi * a.stride_s + 16 * ks + 8 * lh);
        vf[ks] = *reinterpret_cast<const bf16x8_t*>(vp + kvi * a.stride_s + 16 * ks + 8 * lh);
    }
    f32x16_t dvacc[DT], dkacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            dvacc[t][e] = 0.f;
            dkacc[t][e] = 0.f;
        }
    const float c = a.scale * kLog2e;

    const int64_t jq_begin = CAUSAL ? kv0 / 64 : 0;
    const int64_t jq_end = a.S / 64;
    Stage<64, false> sq[DS], so[DS];
    Stage<D, true> sqt, sot;
    float lse_r = 0.f, delta_r = 0.f;
    {
        const int64_t qc0 = jq_begin * 64;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            sq[s].load(qp, a.stride_s, qc0, a.S, 64 * s, D, tid);
            so[s].load(dop, ldo, qc0, a.S, 64 * s, D, tid);
        }
        sqt.load(qp, a.stride_s, 0, D, qc0, a.S, tid);
        sot.load(dop, ldo, 0, D, qc0, a.S, tid);
        if (tid < 64) {
            lse_r = lsep[qc0 + tid] * kLog2e;
            delta_r = deltap[qc0 + tid];
        }
    }
    for (int64_t jq = jq_begin; jq < jq_end; ++jq) {
        const int64_t qc0 = jq * 64;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            sq[s].store(Qs[s], tid);
            so[s].store(Os[s], tid);
        }
        sqt.store(Qt, tid);
        sot.store(Ot, tid);
        if (tid < 64) {
            lse_s[tid] = lse_r;
            delta_s[tid] = delta_r;
        }
        __syncthreads();
        if (jq + 1 < jq_end) {
#pragma unroll
            for (int s = 0; s < DS; ++s) {
                sq[s].load(qp, a.stride_s, qc0 + 64, a.S, 64 * s, D, tid);
                so[s].load(dop, ldo, qc0 + 64, a.S, 64 * s, D, tid);
            }
            sqt.load(qp, a.stride_s, 0, D, qc0 + 64, a.S, tid);
            sot.load(dop, ldo, 0, D, qc0 + 64, a.S, tid);
            if (tid < 64) {
                lse_r = lsep[qc0 + 64 + tid] * kLog2e;
                delta_r = deltap[qc0 + 64 + tid];
            }
        }
#pragma unroll
        for (int qt = 0; qt < 2; ++qt) {
            const int64_t qt0 = qc0 + 32 * qt;
            if (CAUSAL && (qt0 + 31 < kvw0)) continue;  // every query precedes every key: masked
            f32x16_t sacc, dpacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sacc[e] = 0.f;
                dpacc[e] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8_t qfr = read_chunk(Qs[ks / 4], 32 * qt + l32, 2 * (ks % 4) + lh);
                const bf16x8_t ofr = read_chunk(Os[ks / 4], 32 * qt + l32, 2 * (ks % 4) + lh);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qfr, kf[ks], sacc, 0, 0, 0);
                dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ofr, vf[ks], dpacc, 0, 0, 0);
            }
            // element v: q = qt0 + 8 (v/4) + 4 lh + v%4, kv = kvi
            const bool diag = CAUSAL && (qt0 < kvw0 + 31);
            float pv[16], dsv[16];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float4 l4 = *reinterpret_cast<const float4*>(lse_s + 32 * qt + 8 * g + 4 * lh);
                const float4 d4 = *reinterpret_cast<const float4*>(delta_s + 32 * qt + 8 * g + 4 * lh);
                const float lq[4] = {l4.x, l4.y, l4.z, l4.w};
                const float dq_[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int v = 4 * g + e;
                    float p = __builtin_amdgcn_exp2f(fmaf(sacc[v], c, -lq[e]));
                    if (diag) {
                        const int64_t qrow = qt0 + 8 * g + 4 * lh + e;
                        if (kvi > qrow) p = 0.f;
                    }
                    pv[v] = p;
                    dsv[v] = p * (dpacc[v] - dq_[e]);
                }
            }
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const bf16x8_t pb = pack8(pv + 8 * gp);
                const bf16x8_t dsb = pack8(dsv + 8 * gp);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16x8_t otf = read_runs(Ot, 32 * dt + l32, 4 * qt + 2 * gp, lh);
                    const bf16x8_t qtf = read_runs(Qt, 32 * dt + l32, 4 * qt + 2 * gp, lh);
                    dvacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(otf, pb, dvacc[dt], 0, 0, 0);
                    dkacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qtf, dsb, dkacc[dt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
    // dvacc[dt][v]: d = 32 dt + 8 (v/4) + 4 lh + v%4, kv = kvi
    uint16_t* dkp = a.dk + b * a.stride_b + h * D + kvi * a.stride_s;
    uint16_t* dvp = a.dv + b * a.stride_b + h * D + kvi * a.stride_s;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * dt + 8 * g + 4 * lh;
            *reinterpret_cast<uint2*>(dvp + d) =
                make_uint2(pack_bf16(dvacc[dt][4 * g + 0], dvacc[dt][4 * g + 1]),
                           pack_bf16(dvacc[dt][4 * g + 2], dvacc[dt][4 * g + 3]));
            *reinterpret_cast<uint2*>(dkp + d) =
                make_uint2(pack_bf16(dkacc[dt][4 * g + 0] * a.scale, dkacc[dt][4 * g + 1] * a.scale),
                           pack_bf16(dkacc[dt][4 * g + 2] * a.scale, dkacc[dt][4 * g + 3] * a.scale));
        }
}

// ---- backward: dQ (parallel over query blocks) ---------------------------------------------------
template <int D, bool CAUSAL>
__global__ __launch_bounds__(256) void attn_bwd_dq_kernel(const AttnArgs a) {
    constexpr int DS = D / 64, KS = D / 16, DT = D / 32;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[DS][64 * BK];  // [kv][d]
    __shared__ __attribute__((aligned(16))) uint16_t Vs[DS][64 * BK];  // [kv][d]
    __shared__ __attribute__((aligned(16))) uint16_t Kt[D * BK];       // [d][kv]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t b = blockIdx.z, h = blockIdx.y;
    const int64_t q0 = (int64_t)(CAUSAL ? gridDim.x - 1 - blockIdx.x : blockIdx.x) * 128;
    const int64_t qw0 = q0 + 32 * wave;
    const int64_t qi = qw0 + l32;

    const uint16_t* qp = a.q + b * a.stride_b + h * D;
    const uint16_t* kp = a.k + b * a.stride_b + h * D;
    const uint16_t* vp = a.v + b * a.stride_b + h * D;
    const int64_t ldo = a.H * D;
    const uint16_t* dop = a.d_o + b * a.S * ldo + h * D;

    bf16x8_t qf[KS], dof[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        qf[ks] = *reinterpret_cast<const bf16x8_t*>(qp + qi * a.stride_s + 16 * ks + 8 * lh);
        dof[ks] = *reinterpret_cast<const bf16x8_t*>(dop + qi * ldo + 16 * ks + 8 * lh);
    }
    const float lse_q = a.lse[(b * a.H + h) * a.S + qi] * kLog2e;
    const float delta_q = a.delta[(b * a.H + h) * a.S + qi];
    const float c = a.scale * kLog2e;

    f32x16_t dqacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) dqacc[t][e] = 0.f;

    const int64_t n_blocks = CAUSAL ? (q0 + 128 + 63) / 64 : a.S / 64;
    Stage<64, false> sk[DS], sv[DS];
    Stage<D, true> skt;
#pragma unroll
    for (int s = 0; s < DS; ++s) {
        sk[s].load(kp, a.stride_s, 0, a.S, 64 * s, D, tid);
        sv[s].load(vp, a.stride_s, 0, a.S, 64 * s, D, tid);
    }
    skt.load(kp, a.stride_s, 0, D, 0, a.S, tid);

    for (int64_t j = 0; j < n_blocks; ++j) {
        const int64_t kv0 = j * 64;
#pragma unroll
        for (int s = 0; s < DS; ++s) {
            sk[s].store(Ks[s], tid);
            sv[s].store(Vs[s], tid);
        }
        skt.store(Kt, tid);
        __syncthreads();
        if (j + 1 < n_blocks) {
#pragma unroll
            for (int s = 0; s < DS; ++s) {
                sk[s].load(kp, a.stride_s, kv0 + 64, a.S, 64 * s, D, tid);
                sv[s].load(vp, a.stride_s, kv0 + 64, a.S, 64 * s, D, tid);
            }
            skt.load(kp, a.stride_s, 0, D, kv0 + 64, a.S, tid);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int64_t kt0 = kv0 + 32 * t;
            if (CAUSAL && (kt0 > qw0 + 31)) continue;
            f32x16_t sacc, dpacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sacc[e] = 0.f;
                dpacc[e] = 0.f;
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8_t kfr = read_chunk(Ks[ks / 4], 32 * t + l32, 2 * (ks % 4) + lh);
                const bf16x8_t vfr = read_chunk(Vs[ks / 4], 32 * t + l32, 2 * (ks % 4) + lh);
                sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr, qf[ks], sacc, 0, 0, 0);
                dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr, dof[ks], dpacc, 0, 0, 0);
            }
            // element v: kv = kt0 + 8 (v/4) + 4 lh + v%4, q = qi
            const bool diag = CAUSAL && (kt0 + 31 > qw0);
            float dsv[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float p = __builtin_amdgcn_exp2f(fmaf(sacc[v], c, -lse_q));
                if (diag) {
                    const int64_t kv = kt0 + 8 * (v >> 2) + 4 * lh + (v & 3);
                    if (kv > qi) p = 0.f;
                }
                dsv[v] = p * (dpacc[v] - delta_q);
            }
#pragma unroll
            for (int gp = 0; gp < 2; ++gp) {
                const bf16x8_t dsb = pack8(dsv + 8 * gp);
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    const bf16x8_t ktf = read_runs(Kt, 32 * dt + l32, 4 * t + 2 * gp, lh);
                    dqacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ktf, dsb, dqacc[dt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }
    uint16_t* dqp = a.dq + b * a.stride_b + h * D + qi * a.stride_s;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d = 32 * dt + 8 * g + 4 * lh;
            *reinterpret_cast<uint2*>(dqp + d) =
                make_uint2(pack_bf16(dqacc[dt][4 * g + 0] * a.scale, dqacc[dt][4 * g + 1] * a.scale),
                           pack_bf16(dqacc[dt][4 * g + 2] * a.scale, dqacc[dt][4 * g + 3] * a.scale));
        }
}

static int attn_check(const char* who, const pp_attn_desc* d, bool bwd) {
    if (!d) return fail(PP_ERR_INVALID, "%s: null descriptor", who);
    if (d->B < 0 || d->S < 0 || d->H <= 0) return fail(PP_ERR_INVALID, "%s: bad shape", who);
    if (d->D != 64) return fail(PP_ERR_UNSUPPORTED, "%s: head_dim %lld (only 64 is built)", who, (long long)d->D);
    if (d->S % 128) return fail(PP_ERR_UNSUPPORTED, "%s: S %% 128 != 0 (S=%lld)", who, (long long)d->S);
    if ((d->stride_s % 8) || (d->stride_b % 8)) return fail(PP_ERR_INVALID, "%s: strides must be multiples of 8", who);
    if (d->stride_s < d->H * d->D) return fail(PP_ERR_INVALID, "%s: stride_s < H*D", who);
    if (!d->q || !d->k || !d->v || !d->o || !d->lse) return fail(PP_ERR_INVALID, "%s: null pointer", who);
    if (!aligned(d->q, 16) || !aligned(d->k, 16) || !aligned(d->v, 16) || !aligned(d->o, 16))
        return fail(PP_ERR_INVALID, "%s: q/k/v/o must be 16-byte aligned", who);
    if (bwd) {
        if (!d->d_o || !d->dq || !d->dk || !d->dv || !d->delta) return fail(PP_ERR_INVALID, "%s: null pointer", who);
        if (!aligned(d->d_o, 16) || !aligned(d->dq, 16) || !aligned(d->dk, 16) || !aligned(d->dv, 16))
            return fail(PP_ERR_INVALID, "%s: gradients must be 16-byte aligned", who);
    }
    if (d->S / 128 > 65535 || d->H > 65535 || d->B > 65535) return fail(PP_ERR_UNSUPPORTED, "%s: grid too large", who);
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
    a.scale = d->scale;
    return a;
}

}  // namespace pp

using namespace pp;

extern "C" int pp_attn_fwd(const pp_attn_desc* d, pp_stream stream) {
    int rc = attn_check("pp_attn_fwd", d, false);
    if (rc) return rc;
    if (d->B == 0 || d->S == 0) return PP_OK;
    const AttnArgs a = to_args(d);
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 grid((uint32_t)(d->S / 128), (uint32_t)d->H, (uint32_t)d->B);
    if (d->causal) hipLaunchKernelGGL((attn_fwd_kernel<64, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((attn_fwd_kernel<64, false>), grid, dim3(256), 0, st, a);
    return check_launch("attn_fwd_kernel");
}

extern "C" int pp_attn_bwd(const pp_attn_desc* d, pp_stream stream) {
    int rc = attn_check("pp_attn_bwd", d, true);
    if (rc) return rc;
    if (d->B == 0 || d->S == 0) return PP_OK;
    const AttnArgs a = to_args(d);
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(attn_delta_kernel<64>, dim3((uint32_t)((d->B * d->S + 3) / 4)), dim3(256), 0, st, a);
    dim3 grid((uint32_t)(d->S / 128), (uint32_t)d->H, (uint32_t)d->B);
    if (d->causal) {
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<64, true>), grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL((attn_bwd_dq_kernel<64, true>), grid, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((attn_bwd_dkv_kernel<64, false>), grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL((attn_bwd_dq_kernel<64, false>), grid, dim3(256), 0, st, a);
    }
    return check_launch("attn_bwd");
}
