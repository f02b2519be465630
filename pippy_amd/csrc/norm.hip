// LayerNorm forward / input-gradient / weight-gradient and the bias-gradient column sum.
// All HBM-bound: one wave owns one row and keeps it in registers (a single read of x per pass);
// column reductions are two-stage (per-128-row partials, then an ordered final sum), so results
// do not depend on scheduling.
#include "common.h"

namespace pp {

constexpr int kRowsPerBlock = 4;  // one wave per row

// ---- forward ----------------------------------------------------------------------------------
template <int NV>
__global__ __launch_bounds__(256) void layernorm_fwd_kernel(const uint16_t* __restrict__ x,
                                                            const uint16_t* __restrict__ gamma,
                                                            const uint16_t* __restrict__ beta,
                                                            uint16_t* __restrict__ y,
                                                            float* __restrict__ mean_out,
                                                            float* __restrict__ rstd_out, int64_t rows,
                                                            int C, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nchunk = C >> 3;
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * C);
    float v[NV][8];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunk) {
            const uint4 w = xr[c];
            v[i][0] = bf16lo(w.x); v[i][1] = bf16hi(w.x); v[i][2] = bf16lo(w.y); v[i][3] = bf16hi(w.y);
            v[i][4] = bf16lo(w.z); v[i][5] = bf16hi(w.z); v[i][6] = bf16lo(w.w); v[i][7] = bf16hi(w.w);
#pragma unroll
            for (int e = 0; e < 8; ++e) s += v[i][e];
        }
    }
    // a null mean_out selects RMSNorm: nothing is subtracted and rstd = 1 / sqrt(mean(x^2) + eps)
    const float mean = mean_out ? wave_sum(s) / (float)C : 0.f;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunk) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float d = v[i][e] - mean;
                q += d * d;
            }
        }
    }
    const float var = wave_sum(q) / (float)C;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (lane == 0) {
        if (mean_out) mean_out[row] = mean;
        rstd_out[row] = rstd;
    }
    uint4* yr = reinterpret_cast<uint4*>(y + row * C);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunk) {
            const uint4 gw = reinterpret_cast<const uint4*>(gamma)[c];
            const float gf[8] = {bf16lo(gw.x), bf16hi(gw.x), bf16lo(gw.y), bf16hi(gw.y),
                                 bf16lo(gw.z), bf16hi(gw.z), bf16lo(gw.w), bf16hi(gw.w)};
            float bfv[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (beta) {
                const uint4 bw = reinterpret_cast<const uint4*>(beta)[c];
                bfv[0] = bf16lo(bw.x); bfv[1] = bf16hi(bw.x); bfv[2] = bf16lo(bw.y); bfv[3] = bf16hi(bw.y);
                bfv[4] = bf16lo(bw.z); bfv[5] = bf16hi(bw.z); bfv[6] = bf16lo(bw.w); bfv[7] = bf16hi(bw.w);
            }
            float o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (v[i][e] - mean) * rstd * gf[e] + bfv[e];
            yr[c] = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]),
                               pack_bf16(o[6], o[7]));
        }
    }
}

// a * b + c with the product rounded before the sum, whatever contraction the compiler is allowed elsewhere:
// the two input-gradient kernels below must write the same bits
__device__ __forceinline__ float mul_then_add(float a, float b, float c) {
#pragma clang fp contract(off)
    const float p = a * b;
    return p + c;
}

// ---- input gradient ---------------------------------------------------------------------------
template <int NV>
__global__ __launch_bounds__(256) void layernorm_bwd_input_kernel(
    const uint16_t* __restrict__ dy, const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma,
    const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
    const uint16_t* __restrict__ dres, uint16_t* __restrict__ dx, int64_t rows, int C) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nchunk = C >> 3;
    const float mean = mean_in ? mean_in[row] : 0.f, rstd = rstd_in[row];  // null mean: RMSNorm
    const uint4* xr = reinterpret_cast<const uint4*>(x + row * C);
    const uint4* gr = reinterpret_cast<const uint4*>(dy + row * C);
    float xh[NV][8], wd[NV][8];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunk) {
            const uint4 xw = xr[c], dw = gr[c], gw = reinterpret_cast<const uint4*>(gamma)[c];
            const float xf[8] = {bf16lo(xw.x), bf16hi(xw.x), bf16lo(xw.y), bf16hi(xw.y),
                                 bf16lo(xw.z), bf16hi(xw.z), bf16lo(xw.w), bf16hi(xw.w)};
            const float df[8] = {bf16lo(dw.x), bf16hi(dw.x), bf16lo(dw.y), bf16hi(dw.y),
                                 bf16lo(dw.z), bf16hi(dw.z), bf16lo(dw.w), bf16hi(dw.w)};
            const float gf[8] = {bf16lo(gw.x), bf16hi(gw.x), bf16lo(gw.y), bf16hi(gw.y),
                                 bf16lo(gw.z), bf16hi(gw.z), bf16lo(gw.w), bf16hi(gw.w)};
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                xh[i][e] = (xf[e] - mean) * rstd;
                wd[i][e] = df[e] * gf[e];
                s1 += wd[i][e] * xh[i][e];
                s2 += wd[i][e];
            }
        }
    }
    const float c1 = wave_sum(s1) / (float)C;
    const float c2 = mean_in ? wave_sum(s2) / (float)C : 0.f;
    uint4* outr = reinterpret_cast<uint4*>(dx + row * C);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunk) {
            float o[8];
            float rf[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if (dres) {
                const uint4 rw = reinterpret_cast<const uint4*>(dres + row * C)[c];
                rf[0] = bf16lo(rw.x); rf[1] = bf16hi(rw.x); rf[2] = bf16lo(rw.y); rf[3] = bf16hi(rw.y);
                rf[4] = bf16lo(rw.z); rf[5] = bf16hi(rw.z); rf[6] = bf16lo(rw.w); rf[7] = bf16hi(rw.w);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = mul_then_add(wd[i][e] - c1 * xh[i][e] - c2, rstd, rf[e]);
            outr[c] = make_uint4(pack_bf16(o[0], o[1]), pack_bf16(o[2], o[3]), pack_bf16(o[4], o[5]),
                                 pack_bf16(o[6], o[7]));
        }
    }
}

// ---- input gradient that also leaves column sums --------------------------------------------
// The same arithmetic per row; a block owns kSumRows consecutive rows (WAVES waves of RW rows each) and
// writes one row of partial column sums per requested quantity: sum of dy (dbeta) and of dy * xhat
// (dgamma) into ws_w [2][n_part][C], sum of the rounded dx (the bias gradient of the linear layer that
// produced the normalised tensor's input) into ws_dx [n_part][C].  Rows are added in ascending order
// within a wave and the waves in wave order, so the sums do not depend on scheduling.
constexpr int kSumRows = PP_LN_SUM_ROWS;

template <int NV, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void layernorm_bwd_input_sums_kernel(
    const uint16_t* __restrict__ dy, const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma,
    const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
    const uint16_t* __restrict__ dres, uint16_t* __restrict__ dx, int64_t rows, int C,
    float* __restrict__ ws_w, float* __restrict__ ws_dx, int64_t n_part) {
    constexpr int RW = kSumRows / WAVES;  // rows per wave, their loads in flight together
    static_assert(RW * WAVES == kSumRows, "the waves share the block's rows evenly");
    extern __shared__ __attribute__((aligned(16))) float red[];  // [quantities][WAVES][C]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nchunk = C >> 3;
    float gf[NV][8];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = lane + 64 * i;
        const uint4 gw = c < nchunk ? reinterpret_cast<const uint4*>(gamma)[c] : make_uint4(0, 0, 0, 0);
        gf[i][0] = bf16lo(gw.x); gf[i][1] = bf16hi(gw.x); gf[i][2] = bf16lo(gw.y); gf[i][3] = bf16hi(gw.y);
        gf[i][4] = bf16lo(gw.z); gf[i][5] = bf16hi(gw.z); gf[i][6] = bf16lo(gw.w); gf[i][7] = bf16hi(gw.w);
    }
    float sb[NV][8], sg[NV][8], sx[NV][8];
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) sb[i][e] = sg[i][e] = sx[i][e] = 0.f;
    const int64_t row0 = (int64_t)blockIdx.x * kSumRows + wave * RW;
    uint4 xw[RW][NV], dw[RW][NV], rw[RW][NV];
    float mean[RW], rstd[RW];
#pragma unroll
    for (int j = 0; j < RW; ++j) {
        const int64_t row = row0 + j;
        const bool live = row < rows;
        mean[j] = live && mean_in ? mean_in[row] : 0.f;
        rstd[j] = live ? rstd_in[row] : 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane + 64 * i;
            const bool on = live && c < nchunk;
            xw[j][i] = on ? reinterpret_cast<const uint4*>(x + row * C)[c] : make_uint4(0, 0, 0, 0);
            dw[j][i] = on ? reinterpret_cast<const uint4*>(dy + row * C)[c] : make_uint4(0, 0, 0, 0);
            rw[j][i] = on && dres ? reinterpret_cast<const uint4*>(dres + row * C)[c] : make_uint4(0, 0, 0, 0);
        }
    }
#pragma unroll
    for (int j = 0; j < RW; ++j) {
        const int64_t row = row0 + j;
        if (row >= rows) continue;  // wave-uniform
        float xh[NV][8], wd[NV][8];
        float s1 = 0.f, s2 = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const uint4 a = xw[j][i], d = dw[j][i];
            const float xf[8] = {bf16lo(a.x), bf16hi(a.x), bf16lo(a.y), bf16hi(a.y),
                                 bf16lo(a.z), bf16hi(a.z), bf16lo(a.w), bf16hi(a.w)};
            const float df[8] = {bf16lo(d.x), bf16hi(d.x), bf16lo(d.y), bf16hi(d.y),
                                 bf16lo(d.z), bf16hi(d.z), bf16lo(d.w), bf16hi(d.w)};
            const bool on = lane + 64 * i < nchunk;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                xh[i][e] = on ? (xf[e] - mean[j]) * rstd[j] : 0.f;
                wd[i][e] = df[e] * gf[i][e];
                s1 += wd[i][e] * xh[i][e];
                s2 += wd[i][e];
                sb[i][e] += df[e];
                sg[i][e] += df[e] * xh[i][e];
            }
        }
        const float c1 = wave_sum(s1) / (float)C;
        const float c2 = mean_in ? wave_sum(s2) / (float)C : 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int c = lane + 64 * i;
            if (c < nchunk) {
                const uint4 r = rw[j][i];
                const float rf[8] = {bf16lo(r.x), bf16hi(r.x), bf16lo(r.y), bf16hi(r.y),
                                     bf16lo(r.z), bf16hi(r.z), bf16lo(r.w), bf16hi(r.w)};
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float o0 = mul_then_add(wd[i][e] - c1 * xh[i][e] - c2, rstd[j], rf[e]);
                    const float o1 = mul_then_add(wd[i][e + 1] - c1 * xh[i][e + 1] - c2, rstd[j], rf[e + 1]);
                    w[e >> 1] = pack_bf16(o0, o1);
                    sx[i][e] += bf16lo(w[e >> 1]);
                    sx[i][e + 1] += bf16hi(w[e >> 1]);
                }
                reinterpret_cast<uint4*>(dx + row * C)[c] = make_uint4(w[0], w[1], w[2], w[3]);
            }
        }
    }
    // the waves' sums, in wave order; the requested quantities side by side in LDS, one barrier for all
    const int kRowFloats = C, kSetFloats = WAVES * C;
    float* const outs[3] = {ws_w, ws_w ? ws_w + n_part * C : nullptr, ws_dx};
    int set = 0;
#pragma unroll
    for (int pass = 0; pass < 3; ++pass) {
        if (!outs[pass]) continue;  // uniform over the grid
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            if (lane + 64 * i >= nchunk) continue;
            const float* s = pass == 0 ? sb[i] : pass == 1 ? sg[i] : sx[i];
            float4* r = reinterpret_cast<float4*>(&red[set * kSetFloats + wave * kRowFloats + (lane + 64 * i) * 8]);
            r[0] = make_float4(s[0], s[1], s[2], s[3]);
            r[1] = make_float4(s[4], s[5], s[6], s[7]);
        }
        ++set;
    }
    __syncthreads();
    // four columns per lane and step, over the requested quantities laid end to end
    const int n_sets = set, quads = C >> 2;
    for (int q = threadIdx.x; q < n_sets * quads; q += WAVES * 64) {
        const int which = q / quads, c4 = q - which * quads;
        const float4* r = reinterpret_cast<const float4*>(red + which * kSetFloats) + c4;
        float4 v[WAVES];
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v[w] = r[w * (kRowFloats >> 2)];
        float4 t = v[0];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) { t.x += v[w].x; t.y += v[w].y; t.z += v[w].z; t.w += v[w].w; }
        // set number `which` is the which-th requested quantity
        int pass = 0, seen = 0;
#pragma unroll
        for (int p = 0; p < 3; ++p)
            if (outs[p]) { if (seen == which) pass = p; ++seen; }
        reinterpret_cast<float4*>(outs[pass] + (int64_t)blockIdx.x * C)[c4] = t;
    }
}

// ---- column reductions (dgamma / dbeta / bias gradient) ---------------------------------------
// Stage 1: block (rb, cb) reduces rows [128*rb, 128*rb+128) of columns [256*cb, 256*cb+256).
// Lane layout: 32 column chunks (8 columns each) x 8 row phases.
template <bool WITH_X>
__global__ __launch_bounds__(256) void colreduce_partial_kernel(
    const uint16_t* __restrict__ dy, int64_t ld_dy, const uint16_t* __restrict__ x,
    const float* __restrict__ mean_in, const float* __restrict__ rstd_in, float* __restrict__ part_g,
    float* __restrict__ part_b, int64_t rows, int64_t C) {
    __shared__ float red[8][32][8 + 1];
    const int cc = threadIdx.x & 31, rp = threadIdx.x >> 5;
    const int64_t col0 = (int64_t)blockIdx.y * 256 + cc * 8;
    const int64_t row_begin = (int64_t)blockIdx.x * 128;
    float sg[8] = {0, 0, 0, 0, 0, 0, 0, 0}, sb[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (col0 < C) {
        for (int it = 0; it < 16; ++it) {
            const int64_t r = row_begin + it * 8 + rp;
            if (r < rows) {
                const uint4 dw = *reinterpret_cast<const uint4*>(dy + r * ld_dy + col0);
                const float df[8] = {bf16lo(dw.x), bf16hi(dw.x), bf16lo(dw.y), bf16hi(dw.y),
                                     bf16lo(dw.z), bf16hi(dw.z), bf16lo(dw.w), bf16hi(dw.w)};
#pragma unroll
                for (int e = 0; e < 8; ++e) sb[e] += df[e];
                if (WITH_X) {
                    const float mean = mean_in ? mean_in[r] : 0.f, rstd = rstd_in[r];
                    const uint4 xw = *reinterpret_cast<const uint4*>(x + r * C + col0);
                    const float xf[8] = {bf16lo(xw.x), bf16hi(xw.x), bf16lo(xw.y), bf16hi(xw.y),
                                         bf16lo(xw.z), bf16hi(xw.z), bf16lo(xw.w), bf16hi(xw.w)};
#pragma unroll
                    for (int e = 0; e < 8; ++e) sg[e] += df[e] * ((xf[e] - mean) * rstd);
                }
            }
        }
    }
    // reduce the 8 row phases in a fixed order
#pragma unroll
    for (int pass = 0; pass < (WITH_X ? 2 : 1); ++pass) {
        float* s = pass == 0 ? sb : sg;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 8; ++e) red[rp][cc][e] = s[e];
        __syncthreads();
        if (rp == 0 && col0 < C) {
            float* out = (pass == 0 ? part_b : part_g) + (int64_t)blockIdx.x * C + col0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = 0.f;
#pragma unroll
                for (int p = 0; p < 8; ++p) t += red[p][cc][e];
                out[e] = t;
            }
        }
    }
}

// part[0], part[stride], ... summed in that order; the loads of 8 terms are issued together, the
// additions stay a chain (a loop of load-then-add pays one memory latency per term).
__device__ __forceinline__ float ordered_column_sum(const float* __restrict__ part, int64_t n, int64_t stride) {
    float t = 0.f;
    int64_t p = 0;
    for (; p + 8 <= n; p += 8) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = part[(p + k) * stride];
#pragma unroll
        for (int k = 0; k < 8; ++k) t += v[k];
    }
    for (; p < n; ++p) t += part[p * stride];
    return t;
}

// Stage 2: ordered sum of the per-row-block partials, one lane per column.
__global__ __launch_bounds__(256) void colreduce_final_kernel(const float* __restrict__ part,
                                                              int64_t n_part, int64_t C, void* out,
                                                              int out_f32) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const float t = ordered_column_sum(part + c, n_part, C);
    if (out_f32) static_cast<float*>(out)[c] = t;
    else static_cast<uint16_t*>(out)[c] = f32_to_bf16(t);
}

// ---- grouped column reductions -------------------------------------------------------------------
// All bias-gradient and LayerNorm weight-gradient reductions of one weight-gradient pass in two
// launches (partials, then ordered final sums) instead of two or three tiny launches each.
constexpr int kMaxColGroup = PP_COLREDUCE_MAX_GROUP;

struct ColDesc {
    const uint16_t* dy;
    const uint16_t* x;
    const float* mean;
    const float* rstd;
    void* out_sum;
    void* out_dot;
    float* ws;       // [2][n_part][C]: sums, then dots
    int64_t ld_dy;
    int rows, C, n_part, n_cb, out_f32;
    int ready;  // the workspace already holds n_part rows of partial sums (a producer kernel wrote them)
};

struct ColGroupArgs {
    ColDesc d[kMaxColGroup];
    uint32_t part_start[kMaxColGroup + 1];   // block ranges of the partial kernel
    uint32_t final_start[kMaxColGroup + 1];  // block ranges of the final kernel
    int n;
};

__global__ __launch_bounds__(256) void colgroup_partial_kernel(const ColGroupArgs ga) {
    __shared__ float red[8][32][8 + 1];
    uint32_t b = blockIdx.x;
    int i = 0;
    while (i + 1 < ga.n && b >= ga.part_start[i + 1]) ++i;
    b -= ga.part_start[i];
    const ColDesc& d = ga.d[i];
    const int rb = b / d.n_cb, cb = b % d.n_cb;
    const int cc = threadIdx.x & 31, rp = threadIdx.x >> 5;
    const int col0 = cb * 256 + cc * 8;
    const int row_begin = rb * 128;
    const bool with_x = d.x != nullptr;
    float sg[8] = {0, 0, 0, 0, 0, 0, 0, 0}, sb[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (col0 < d.C) {
        for (int it = 0; it < 16; ++it) {
            const int r = row_begin + it * 8 + rp;
            if (r < d.rows) {
                const uint4 dw = *reinterpret_cast<const uint4*>(d.dy + (int64_t)r * d.ld_dy + col0);
                const float df[8] = {bf16lo(dw.x), bf16hi(dw.x), bf16lo(dw.y), bf16hi(dw.y),
                                     bf16lo(dw.z), bf16hi(dw.z), bf16lo(dw.w), bf16hi(dw.w)};
#pragma unroll
                for (int e = 0; e < 8; ++e) sb[e] += df[e];
                if (with_x) {
                    const float mean = d.mean ? d.mean[r] : 0.f, rstd = d.rstd[r];
                    const uint4 xw = *reinterpret_cast<const uint4*>(d.x + (int64_t)r * d.C + col0);
                    const float xf[8] = {bf16lo(xw.x), bf16hi(xw.x), bf16lo(xw.y), bf16hi(xw.y),
                                         bf16lo(xw.z), bf16hi(xw.z), bf16lo(xw.w), bf16hi(xw.w)};
#pragma unroll
                    for (int e = 0; e < 8; ++e) sg[e] += df[e] * ((xf[e] - mean) * rstd);
                }
            }
        }
    }
    for (int pass = 0; pass < (with_x ? 2 : 1); ++pass) {
        const float* s = pass == 0 ? sb : sg;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 8; ++e) red[rp][cc][e] = s[e];
        __syncthreads();
        if (rp == 0 && col0 < d.C) {
            float* out = d.ws + ((int64_t)pass * d.n_part + rb) * d.C + col0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = 0.f;
#pragma unroll
                for (int p = 0; p < 8; ++p) t += red[p][cc][e];
                out[e] = t;
            }
        }
    }
}

__global__ __launch_bounds__(256) void colgroup_final_kernel(const ColGroupArgs ga) {
    uint32_t b = blockIdx.x;
    int i = 0;
    while (i + 1 < ga.n && b >= ga.final_start[i + 1]) ++i;
    b -= ga.final_start[i];
    const ColDesc& d = ga.d[i];
    if (d.ready) {
        // partial sums left by a producer, many rows of them: 32 columns per block, the rows dealt out to 8
        // phases (phase p adds rows p, p + 8, ... in ascending order), the phases added in phase order
        __shared__ float red[8][32 + 1];
        const int cc = threadIdx.x & 31, rp = threadIdx.x >> 5;
        const int c = b * 32 + cc;
        for (int pass = 0; pass < 2; ++pass) {
            void* out = pass == 0 ? d.out_sum : d.out_dot;
            if (!out) continue;  // uniform over the block
            const float* part = d.ws + (int64_t)pass * d.n_part * d.C + c;
            float t = 0.f;
            if (c < d.C) {
                // 16 loads in flight per lane (a loop of load-then-add pays one memory latency per term); the
                // additions stay a chain in ascending row order
                int p = rp;
                for (; p + 8 * 15 < d.n_part; p += 8 * 16) {
                    float v[16];
#pragma unroll
                    for (int k = 0; k < 16; ++k) v[k] = part[(int64_t)(p + 8 * k) * d.C];
#pragma unroll
                    for (int k = 0; k < 16; ++k) t += v[k];
                }
                for (; p < d.n_part; p += 8) t += part[(int64_t)p * d.C];
            }
            __syncthreads();
            red[rp][cc] = t;
            __syncthreads();
            if (rp == 0 && c < d.C) {
                float sum = 0.f;
#pragma unroll
                for (int q = 0; q < 8; ++q) sum += red[q][cc];
                if (d.out_f32) static_cast<float*>(out)[c] = sum;
                else static_cast<uint16_t*>(out)[c] = f32_to_bf16(sum);
            }
        }
        return;
    }
    const int c = b * 256 + threadIdx.x;
    if (c >= d.C) return;
    for (int pass = 0; pass < 2; ++pass) {
        void* out = pass == 0 ? d.out_sum : d.out_dot;
        if (!out || (pass == 1 && !d.x)) continue;
        const float* part = d.ws + (int64_t)pass * d.n_part * d.C;
        const float t = ordered_column_sum(part + c, d.n_part, d.C);
        if (d.out_f32) static_cast<float*>(out)[c] = t;
        else static_cast<uint16_t*>(out)[c] = f32_to_bf16(t);
    }
}

template <int NV>
static void launch_ln_fwd(const void* x, const void* gamma, const void* beta, void* y, float* mean,
                          float* rstd, int64_t rows, int C, float eps, hipStream_t st) {
    const uint32_t nb = (uint32_t)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    hipLaunchKernelGGL(layernorm_fwd_kernel<NV>, dim3(nb), dim3(256), 0, st, (const uint16_t*)x,
                       (const uint16_t*)gamma, (const uint16_t*)beta, (uint16_t*)y, mean, rstd, rows, C, eps);
}
template <int NV>
static void launch_ln_bwd_in(const void* dy, const void* x, const void* gamma, const float* mean,
                             const float* rstd, const void* dres, void* dx, int64_t rows, int C,
                             hipStream_t st) {
    const uint32_t nb = (uint32_t)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    hipLaunchKernelGGL(layernorm_bwd_input_kernel<NV>, dim3(nb), dim3(256), 0, st, (const uint16_t*)dy,
                       (const uint16_t*)x, (const uint16_t*)gamma, mean, rstd, (const uint16_t*)dres,
                       (uint16_t*)dx, rows, C);
}

#ifndef PP_LN_SUM_WAVES
#define PP_LN_SUM_WAVES 8
#endif
template <int NV>
static int launch_ln_bwd_in_sums(const void* dy, const void* x, const void* gamma, const float* mean,
                                 const float* rstd, const void* dres, void* dx, int64_t rows, int C,
                                 float* ws_w, float* ws_dx, hipStream_t st) {
    constexpr int WAVES = PP_LN_SUM_WAVES;
    // one set of WAVES rows per requested quantity
    const size_t lds = (size_t)((ws_w ? 2 : 0) + (ws_dx ? 1 : 0)) * WAVES * C * sizeof(float);
    static_assert((size_t)3 * WAVES * PP_LN_SUM_MAX_C * sizeof(float) <= 160 * 1024, "LDS of one CU");
    static const hipError_t attr_rc = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&layernorm_bwd_input_sums_kernel<NV, WAVES>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)3 * WAVES * PP_LN_SUM_MAX_C * sizeof(float)));
    if (attr_rc != hipSuccess)
        return fail(PP_ERR_LAUNCH, "pp_layernorm_bwd_input_sums: cannot reserve %zu bytes of LDS: %s", lds,
                    hipGetErrorString(attr_rc));
    const int64_t n_part = (rows + kSumRows - 1) / kSumRows;
    hipLaunchKernelGGL((layernorm_bwd_input_sums_kernel<NV, WAVES>), dim3((uint32_t)n_part), dim3(WAVES * 64), lds, st,
                       (const uint16_t*)dy, (const uint16_t*)x, (const uint16_t*)gamma, mean, rstd,
                       (const uint16_t*)dres, (uint16_t*)dx, rows, C, ws_w, ws_dx, n_part);
    return PP_OK;
}

static int ln_check(const char* who, int64_t rows, int64_t C) {
    if (rows < 0 || C <= 0) return fail(PP_ERR_INVALID, "%s: bad shape", who);
    if (C % 8) return fail(PP_ERR_UNSUPPORTED, "%s: C %% 8 != 0 (C=%lld)", who, (long long)C);
    if (C > 64 * 8 * 16) return fail(PP_ERR_UNSUPPORTED, "%s: C > 8192", who);
    return PP_OK;
}

}  // namespace pp

using namespace pp;

extern "C" int pp_layernorm_fwd(const void* x, const void* gamma, const void* beta, void* y,
                                float* mean, float* rstd, int64_t rows, int64_t C, float eps,
                                pp_stream stream) {
    int rc = ln_check("pp_layernorm_fwd", rows, C);
    if (rc) return rc;
    if (rows == 0) return PP_OK;
    if (!x || !gamma || !y || !rstd) return fail(PP_ERR_INVALID, "pp_layernorm_fwd: null pointer");
    if (!mean && beta) return fail(PP_ERR_INVALID, "pp_layernorm_fwd: RMSNorm (null mean) has no beta");
    if (!aligned(x, 16) || !aligned(y, 16) || !aligned(gamma, 16) || !aligned(beta, 16))
        return fail(PP_ERR_INVALID, "pp_layernorm_fwd: pointers must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nv = (int)((C / 8 + 63) / 64);
    if (nv <= 1) launch_ln_fwd<1>(x, gamma, beta, y, mean, rstd, rows, (int)C, eps, st);
    else if (nv <= 2) launch_ln_fwd<2>(x, gamma, beta, y, mean, rstd, rows, (int)C, eps, st);
    else if (nv <= 4) launch_ln_fwd<4>(x, gamma, beta, y, mean, rstd, rows, (int)C, eps, st);
    else if (nv <= 8) launch_ln_fwd<8>(x, gamma, beta, y, mean, rstd, rows, (int)C, eps, st);
    else launch_ln_fwd<16>(x, gamma, beta, y, mean, rstd, rows, (int)C, eps, st);
    return check_launch("layernorm_fwd_kernel");
}

extern "C" int pp_layernorm_bwd_input(const void* dy, const void* x, const void* gamma,
                                      const float* mean, const float* rstd, const void* dres,
                                      void* dx, int64_t rows, int64_t C, pp_stream stream) {
    int rc = ln_check("pp_layernorm_bwd_input", rows, C);
    if (rc) return rc;
    if (rows == 0) return PP_OK;
    if (!dy || !x || !gamma || !rstd || !dx)
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_input: null pointer");
    if (!aligned(x, 16) || !aligned(dy, 16) || !aligned(gamma, 16) || !aligned(dres, 16) || !aligned(dx, 16))
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_input: pointers must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nv = (int)((C / 8 + 63) / 64);
    if (nv <= 1) launch_ln_bwd_in<1>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, st);
    else if (nv <= 2) launch_ln_bwd_in<2>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, st);
    else if (nv <= 4) launch_ln_bwd_in<4>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, st);
    else if (nv <= 8) launch_ln_bwd_in<8>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, st);
    else launch_ln_bwd_in<16>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, st);
    return check_launch("layernorm_bwd_input_kernel");
}

extern "C" int pp_layernorm_bwd_input_sums(const void* dy, const void* x, const void* gamma, const float* mean,
                                           const float* rstd, const void* dres, void* dx, int64_t rows,
                                           int64_t C, float* ws_weight, float* ws_dx, pp_stream stream) {
    if (!ws_weight && !ws_dx) return pp_layernorm_bwd_input(dy, x, gamma, mean, rstd, dres, dx, rows, C, stream);
    int rc = ln_check("pp_layernorm_bwd_input_sums", rows, C);
    if (rc) return rc;
    if (C > PP_LN_SUM_MAX_C)
        return fail(PP_ERR_UNSUPPORTED, "pp_layernorm_bwd_input_sums: C = %lld exceeds %d (the waves' sums of a block meet in "
                    "LDS); use pp_layernorm_bwd_input and the column reductions", (long long)C, PP_LN_SUM_MAX_C);
    if (rows == 0) return PP_OK;
    if (!dy || !x || !gamma || !rstd || !dx)
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_input_sums: null pointer");
    if (!aligned(x, 16) || !aligned(dy, 16) || !aligned(gamma, 16) || !aligned(dres, 16) || !aligned(dx, 16))
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_input_sums: pointers must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nv = (int)((C / 8 + 63) / 64);
    if (nv <= 1) rc = launch_ln_bwd_in_sums<1>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, ws_weight, ws_dx, st);
    else rc = launch_ln_bwd_in_sums<2>(dy, x, gamma, mean, rstd, dres, dx, rows, (int)C, ws_weight, ws_dx, st);
    if (rc) return rc;
    return check_launch("layernorm_bwd_input_sums_kernel");
}

extern "C" int pp_layernorm_bwd_weight(const void* dy, const void* x, const float* mean,
                                       const float* rstd, void* dgamma, void* dbeta, int out_dtype,
                                       float* workspace, int64_t rows, int64_t C, pp_stream stream) {
    if (rows < 0 || C <= 0) return fail(PP_ERR_INVALID, "pp_layernorm_bwd_weight: bad shape");
    if (C % 8) return fail(PP_ERR_UNSUPPORTED, "pp_layernorm_bwd_weight: C %% 8 != 0");
    if (!dy || !x || !rstd || !dgamma || !workspace)
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_weight: null pointer");
    if (!aligned(x, 16) || !aligned(dy, 16))
        return fail(PP_ERR_INVALID, "pp_layernorm_bwd_weight: pointers must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n_part = (rows + 127) / 128;
    float* part_b = workspace;
    float* part_g = workspace + n_part * C;
    if (n_part > 0) {
        dim3 grid((uint32_t)n_part, (uint32_t)((C + 255) / 256));
        hipLaunchKernelGGL(colreduce_partial_kernel<true>, grid, dim3(256), 0, st, (const uint16_t*)dy, C,
                           (const uint16_t*)x, mean, rstd, part_g, part_b, rows, C);
    }
    const uint32_t nb = (uint32_t)((C + 255) / 256);
    hipLaunchKernelGGL(colreduce_final_kernel, dim3(nb), dim3(256), 0, st, part_g, n_part, C, dgamma,
                       out_dtype == PP_F32);
    if (dbeta)
        hipLaunchKernelGGL(colreduce_final_kernel, dim3(nb), dim3(256), 0, st, part_b, n_part, C, dbeta,
                           out_dtype == PP_F32);
    return check_launch("layernorm_bwd_weight");
}

extern "C" int pp_colsum_bf16(const void* dY, int64_t M, int64_t N, int64_t ld, void* out,
                              int out_dtype, float* workspace, pp_stream stream) {
    if (M < 0 || N <= 0 || ld < N) return fail(PP_ERR_INVALID, "pp_colsum_bf16: bad shape");
    if ((N % 8) || (ld % 8)) return fail(PP_ERR_UNSUPPORTED, "pp_colsum_bf16: N and ld must be multiples of 8");
    if (!dY || !out || !workspace) return fail(PP_ERR_INVALID, "pp_colsum_bf16: null pointer");
    if (!aligned(dY, 16)) return fail(PP_ERR_INVALID, "pp_colsum_bf16: dY must be 16-byte aligned");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n_part = (M + 127) / 128;
    if (n_part > 0) {
        dim3 grid((uint32_t)n_part, (uint32_t)((N + 255) / 256));
        hipLaunchKernelGGL(colreduce_partial_kernel<false>, grid, dim3(256), 0, st, (const uint16_t*)dY, ld,
                           (const uint16_t*)nullptr, (const float*)nullptr, (const float*)nullptr,
                           (float*)nullptr, workspace, M, N);
    }
    hipLaunchKernelGGL(colreduce_final_kernel, dim3((uint32_t)((N + 255) / 256)), dim3(256), 0, st,
                       workspace, n_part, N, out, out_dtype == PP_F32);
    return check_launch("colsum");
}

// ---- column sum with the partial sums in a library-owned array -----------------------------------
// For callers that cannot allocate (a loop under graph capture, a harness that forbids it): the
// per-row-block partial sums of pp_colsum_bf16 live in a file-scope device array instead of a
// caller-provided workspace.  Every GPU holds its own copy of the array at its own address, so the
// address is looked up once per device, with that device current, and only that pointer is ever
// handed to a kernel or a copy: the array's name is a host-side stand-in, not a device address.
namespace pp {
constexpr int64_t kColsumScratchFloats = PP_COLSUM_NOALLOC_MAX_FLOATS;
static __device__ __align__(256) float g_colsum_scratch[kColsumScratchFloats];

constexpr int kMaxDevices = 64;
static float* g_colsum_scratch_ptr[kMaxDevices];  // per device, null until looked up

// The device address of the current device's copy of the array; null (and a message) on failure.
static float* colsum_scratch_for_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        fail(PP_ERR_LAUNCH, "pp_colsum_bf16_noalloc: cannot identify the current device (%s)",
             e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return nullptr;
    }
    float* p = __atomic_load_n(&g_colsum_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (p) return p;
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_colsum_scratch));
    if (e != hipSuccess || !sym) {
        fail(PP_ERR_LAUNCH, "pp_colsum_bf16_noalloc: hipGetSymbolAddress failed on device %d: %s", dev,
             hipGetErrorString(e));
        return nullptr;
    }
    // two threads racing here look up the same address; the store is idempotent
    __atomic_store_n(&g_colsum_scratch_ptr[dev], static_cast<float*>(sym), __ATOMIC_RELEASE);
    return static_cast<float*>(sym);
}
}  // namespace pp

extern "C" int pp_colsum_bf16_noalloc(const void* dY, int64_t M, int64_t N, int64_t ld, void* out,
                                      int out_dtype, pp_stream stream) {
    if (M < 0 || N <= 0 || ld < N) return fail(PP_ERR_INVALID, "pp_colsum_bf16_noalloc: bad shape");
    const int64_t n_part = (M + 127) / 128;
    if (n_part * N > kColsumScratchFloats)
        return fail(PP_ERR_UNSUPPORTED,
                    "pp_colsum_bf16_noalloc: ceil(M / 128) * N = %lld partial sums exceed the built-in "
                    "array of %lld floats; use pp_colsum_bf16 with a workspace", (long long)(n_part * N),
                    (long long)kColsumScratchFloats);
    float* scratch = colsum_scratch_for_current_device();
    if (!scratch) return PP_ERR_LAUNCH;
    // every partial sum that the final kernel reads is written by the partial kernel of this call, so
    // nothing left by an earlier call needs clearing
    return pp_colsum_bf16(dY, M, N, ld, out, out_dtype, scratch, stream);
}

extern "C" int pp_colreduce_grouped(const pp_colreduce_desc* descs, int n, pp_stream stream) {
    if (n < 0 || (n > 0 && !descs)) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: bad list");
    hipStream_t st = static_cast<hipStream_t>(stream);
    for (int i0 = 0; i0 < n; i0 += kMaxColGroup) {
        ColGroupArgs ga;
        ga.n = 0;
        uint64_t pb = 0, fb = 0;
        const int cnt = (n - i0 < kMaxColGroup) ? n - i0 : kMaxColGroup;
        for (int i = 0; i < cnt; ++i) {
            const pp_colreduce_desc& s = descs[i0 + i];
            if (s.rows < 0 || s.C <= 0 || s.ld_dy < s.C) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: bad shape in %d", i0 + i);
            if (!(s.n_part_ready > 0) && ((s.C % 8) || (s.ld_dy % 8))) return fail(PP_ERR_UNSUPPORTED, "pp_colreduce_grouped: C and ld must be multiples of 8");
            const bool ready = s.n_part_ready > 0;
            if ((!ready && !s.dy) || !s.workspace || (!s.out_sum && !s.out_dot)) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: null pointer in %d", i0 + i);
            if (!ready && s.out_dot && (!s.x || !s.rstd)) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: out_dot needs x and rstd");
            if (s.n_part_ready < 0) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: negative n_part_ready in %d", i0 + i);
            if (!aligned(s.dy, 16) || !aligned(s.x, 16)) return fail(PP_ERR_INVALID, "pp_colreduce_grouped: dy and x must be 16-byte aligned");
            if (s.rows > 0x7fffffff || s.C > 0x7fffffff) return fail(PP_ERR_UNSUPPORTED, "pp_colreduce_grouped: shape too large");
            ColDesc& d = ga.d[ga.n];
            d.dy = static_cast<const uint16_t*>(s.dy);
            d.x = s.out_dot ? static_cast<const uint16_t*>(s.x) : nullptr;
            d.mean = s.mean; d.rstd = s.rstd;
            d.out_sum = s.out_sum; d.out_dot = s.out_dot;
            d.ws = s.workspace;
            d.ld_dy = s.ld_dy;
            d.rows = (int)s.rows; d.C = (int)s.C;
            d.ready = ready;
            d.n_part = ready ? s.n_part_ready : (int)((s.rows + 127) / 128);
            d.n_cb = (int)((s.C + 255) / 256);
            d.out_f32 = s.out_dtype == PP_F32;
            ga.part_start[ga.n] = (uint32_t)pb;
            ga.final_start[ga.n] = (uint32_t)fb;
            if (!ready) pb += (uint64_t)d.n_part * d.n_cb;
            fb += ready ? (uint64_t)((s.C + 31) / 32) : (uint64_t)d.n_cb;
            ++ga.n;
        }
        if (pb > 0x7fffffffull) return fail(PP_ERR_UNSUPPORTED, "pp_colreduce_grouped: too many blocks");
        ga.part_start[ga.n] = (uint32_t)pb;
        ga.final_start[ga.n] = (uint32_t)fb;
        if (pb) hipLaunchKernelGGL(colgroup_partial_kernel, dim3((uint32_t)pb), dim3(256), 0, st, ga);
        if (fb) hipLaunchKernelGGL(colgroup_final_kernel, dim3((uint32_t)fb), dim3(256), 0, st, ga);
    }
    return check_launch("colreduce_grouped");
}
