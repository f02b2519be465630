// Routing of a top-2 mixture-of-experts layer: expert selection, the permutation that groups the
// (token, slot) pairs of each expert into consecutive rows, and the row gathers / weighted sums
// either side of the expert GEMMs.  Everything stays on the device: the per-expert row counts are
// written to memory and read by the segmented GEMM, never by the host.
//
// Vocabulary: T tokens, E experts, `topk` slots per token; the flat slot index of (token t, slot k)
// is f = t * topk + k; a permuted row r holds one flat slot, rows are ordered by expert and, within
// an expert, by ascending f (so the permutation does not depend on scheduling).
#include "common.h"

namespace pp {

__device__ __forceinline__ void moe_unpack8(const uint4& w, float (&f)[8]) {
    f[0] = bf16lo(w.x); f[1] = bf16hi(w.x); f[2] = bf16lo(w.y); f[3] = bf16hi(w.y);
    f[4] = bf16lo(w.z); f[5] = bf16hi(w.z); f[6] = bf16lo(w.w); f[7] = bf16hi(w.w);
}
__device__ __forceinline__ uint4 moe_pack8(const float (&f)[8]) {
    return make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
}

// One lane per token: the two largest logits (the lower expert index wins a tie) and their
// softmax weights renormalised over the pair, which is the softmax of the two logits alone.
__global__ __launch_bounds__(256) void moe_router_top2_kernel(const uint16_t* __restrict__ logits, int64_t ld,
                                                              int64_t T, int E, int32_t* __restrict__ idx,
                                                              float* __restrict__ gate) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    const uint16_t* row = logits + t * ld;
    float best = bf16_to_f32(row[0]), second = -INFINITY;
    int bi = 0, si = -1;
    for (int e = 1; e < E; ++e) {
        const float v = bf16_to_f32(row[e]);
        if (v > best) {
            second = best; si = bi;
            best = v; bi = e;
        } else if (v > second || si < 0) {
            second = v; si = e;
        }
    }
    const float eb = __expf(second - best);  // <= 1
    const float ga = 1.0f / (1.0f + eb);
    idx[2 * t] = bi;
    idx[2 * t + 1] = si;
    gate[2 * t] = ga;
    gate[2 * t + 1] = (second == best) ? ga : eb * ga;
}

// Counting sort of n flat slots by expert, in one work-group of 1024 lanes (n is a few thousand
// to a few hundred thousand: the time is negligible next to the expert GEMMs).  Writes
//   seg_start[0 .. E]: first row of every expert, seg_start[E] = number of rows placed,
//   row_src[r] = flat slot held by row r,  pos[f] = row of flat slot f (-1 for an expert id
//   outside [0, E), whose slot is dropped).
constexpr int kMoeMaxExperts = 64;
__global__ __launch_bounds__(1024) void moe_permute_kernel(const int32_t* __restrict__ idx, int n, int E,
                                                           int32_t* __restrict__ seg_start,
                                                           int32_t* __restrict__ row_src,
                                                           int32_t* __restrict__ pos) {
    __shared__ int cnt[kMoeMaxExperts];
    __shared__ int base[kMoeMaxExperts];
    __shared__ int wave_cnt[16][kMoeMaxExperts];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid < kMoeMaxExperts) cnt[tid] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += 1024) {
        const int e = idx[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int s = 0;
        for (int e = 0; e < E; ++e) {
            seg_start[e] = s;
            base[e] = s;
            s += cnt[e];
        }
        seg_start[E] = s;
    }
    __syncthreads();
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int c0 = 0; c0 < n; c0 += 1024) {
        const int i = c0 + tid;
        int e = (i < n) ? idx[i] : -1;
        if (e >= E) e = -1;
        int rank = 0;
        for (int ee = 0; ee < E; ++ee) {
            const unsigned long long m = __ballot(e == ee);
            if (e == ee) rank = __popcll(m & below);
            if (lane == 0) wave_cnt[wave][ee] = __popcll(m);
        }
        __syncthreads();
        if (e >= 0) {
            int r = base[e] + rank;
            for (int w = 0; w < wave; ++w) r += wave_cnt[w][e];
            row_src[r] = i;
            pos[i] = r;
        } else if (i < n) {
            pos[i] = -1;
        }
        __syncthreads();
        if (tid < E) {
            int s = 0;
            for (int w = 0; w < 16; ++w) s += wave_cnt[w][tid];
            base[tid] += s;
        }
        __syncthreads();
    }
}

// dst[r, :] = scale[f] * src[f / topk, :]  with f = row_src[r]  (scale null: plain gather).
// One wave per row, 16 bytes per lane and access.
__global__ __launch_bounds__(256) void moe_gather_kernel(const uint16_t* __restrict__ src, int64_t ld_src,
                                                         const int32_t* __restrict__ row_src,
                                                         const int32_t* __restrict__ n_rows_dev, int topk,
                                                         const float* __restrict__ scale,
                                                         uint16_t* __restrict__ dst, int64_t ld_dst, int64_t R,
                                                         int C8) {
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * 4;
    const int64_t n_rows = n_rows_dev ? min((int64_t)*n_rows_dev, R) : R;
    for (int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); r < n_rows; r += waves) {
        const int f = row_src[r];
        const float s = scale ? scale[f] : 1.0f;
        const uint4* sp = reinterpret_cast<const uint4*>(src + (int64_t)(f / topk) * ld_src);
        uint4* dp = reinterpret_cast<uint4*>(dst + r * ld_dst);
        for (int c = lane; c < C8; c += 64) {
            uint4 w = sp[c];
            if (scale) {
                float v[8];
                moe_unpack8(w, v);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] *= s;
                w = moe_pack8(v);
            }
            dp[c] = w;
        }
    }
}

// out[t, :] = resid[t, :] + sum_k gate[f] * y[pos[f], :],  f = t * topk + k  (resid, gate optional;
// a dropped slot, pos[f] < 0, contributes nothing).  fp32 sum, one rounding.
__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t* __restrict__ y, int64_t ld_y,
                                                          const int32_t* __restrict__ pos,
                                                          const float* __restrict__ gate, int topk,
                                                          const uint16_t* __restrict__ resid, int64_t ld_resid,
                                                          uint16_t* __restrict__ out, int64_t ld_out, int64_t T,
                                                          int C8) {
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * 4;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += waves) {
        for (int c = lane; c < C8; c += 64) {
            float acc[8];
            if (resid) {
                moe_unpack8(reinterpret_cast<const uint4*>(resid + t * ld_resid)[c], acc);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = 0.f;
            }
            for (int k = 0; k < topk; ++k) {
                const int r = pos[t * topk + k];
                if (r < 0) continue;
                const float gk = gate ? gate[t * topk + k] : 1.0f;
                float v[8];
                moe_unpack8(reinterpret_cast<const uint4*>(y + (int64_t)r * ld_y)[c], v);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[e] = fmaf(gk, v[e], acc[e]);
            }
            reinterpret_cast<uint4*>(out + t * ld_out)[c] = moe_pack8(acc);
        }
    }
}

// Gradient of the routing weights back to the router logits.  With gate = softmax over the
// selected logits,  dgate_k = <dout[t], y[pos(t, k)]>  and
//   dlogit[idx_k] = gate_k * (dgate_k - sum_j gate_j dgate_j),  zero for the experts not selected.
// One wave per token; topk <= 8.
constexpr int kMoeMaxTopk = 8;
__global__ __launch_bounds__(256) void moe_gate_bwd_kernel(const uint16_t* __restrict__ dout, int64_t ld_dout,
                                                           const uint16_t* __restrict__ y, int64_t ld_y,
                                                           const int32_t* __restrict__ pos,
                                                           const int32_t* __restrict__ idx,
                                                           const float* __restrict__ gate, int topk, int E,
                                                           uint16_t* __restrict__ dlogits, int64_t ld_dl,
                                                           int64_t T, int C8) {
    const int lane = threadIdx.x & 63;
    const int64_t waves = (int64_t)gridDim.x * 4;
    for (int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); t < T; t += waves) {
        float dg[kMoeMaxTopk];
#pragma unroll
        for (int k = 0; k < kMoeMaxTopk; ++k) dg[k] = 0.f;
        for (int c = lane; c < C8; c += 64) {
            float d[8];
            moe_unpack8(reinterpret_cast<const uint4*>(dout + t * ld_dout)[c], d);
#pragma unroll
            for (int k = 0; k < kMoeMaxTopk; ++k) {
                if (k >= topk) break;
                const int r = pos[t * topk + k];
                if (r < 0) continue;
                float v[8];
                moe_unpack8(reinterpret_cast<const uint4*>(y + (int64_t)r * ld_y)[c], v);
#pragma unroll
                for (int e = 0; e < 8; ++e) dg[k] = fmaf(d[e], v[e], dg[k]);
            }
        }
        float mean = 0.f;
#pragma unroll
        for (int k = 0; k < kMoeMaxTopk; ++k) {
            if (k >= topk) break;
            dg[k] = wave_sum(dg[k]);
            mean = fmaf(gate[t * topk + k], dg[k], mean);
        }
        // columns E .. round_up(E, 8) - 1 (the padding of a router with an expert count that is not a
        // multiple of 8; ld_dl is a multiple of 8) are written as zeros
        for (int e = lane; e < ((E + 7) & ~7); e += 64) {
            float v = 0.f;
#pragma unroll
            for (int k = 0; k < kMoeMaxTopk; ++k) {
                if (k >= topk) break;
                if (idx[t * topk + k] == e) v += gate[t * topk + k] * (dg[k] - mean);
            }
            dlogits[t * ld_dl + e] = f32_to_bf16(v);
        }
    }
}

static int row_grid(int64_t rows) {
    const int64_t blocks = (rows + 3) / 4;
    return (int)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

static bool rows_ok(const void* p, int64_t ld) { return p && aligned(p, 16) && (ld & 7) == 0; }

}  // namespace pp

using namespace pp;

extern "C" int pp_moe_router_top2(const void* logits, int64_t ld, int64_t T, int E, int32_t* topk_idx,
                                  float* gate, pp_stream stream) {
    if (T < 0 || E < 2 || ld < E || !logits || !topk_idx || !gate)
        return fail(PP_ERR_INVALID, "pp_moe_router_top2: bad arguments (T=%lld E=%d)", (long long)T, E);
    if (T == 0) return PP_OK;
    hipLaunchKernelGGL(moe_router_top2_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(logits), ld, T, E, topk_idx, gate);
    return check_launch("moe_router_top2_kernel");
}

extern "C" int pp_moe_permute(const int32_t* expert_of_slot, int64_t n_slots, int E, int32_t* seg_start,
                              int32_t* row_src, int32_t* pos, pp_stream stream) {
    if (n_slots < 0 || n_slots > 0x7fffffff || E < 1 || E > kMoeMaxExperts || !seg_start ||
        (n_slots > 0 && (!expert_of_slot || !row_src || !pos)))
        return fail(PP_ERR_INVALID, "pp_moe_permute: bad arguments (n_slots=%lld E=%d, at most %d experts)",
                    (long long)n_slots, E, kMoeMaxExperts);
    hipLaunchKernelGGL(moe_permute_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       expert_of_slot, (int)n_slots, E, seg_start, row_src, pos);
    return check_launch("moe_permute_kernel");
}

extern "C" int pp_moe_gather(const void* src, int64_t ld_src, const int32_t* row_src, const int32_t* n_rows_dev,
                             int topk, const float* scale, void* dst, int64_t ld_dst, int64_t R, int64_t C,
                             pp_stream stream) {
    if (R < 0 || C < 0 || (C & 7) || topk < 1 || !row_src || !rows_ok(src, ld_src) || !rows_ok(dst, ld_dst) ||
        ld_src < C || ld_dst < C)
        return fail(PP_ERR_INVALID, "pp_moe_gather: bad arguments (R=%lld C=%lld)", (long long)R, (long long)C);
    if (R == 0 || C == 0) return PP_OK;
    hipLaunchKernelGGL(moe_gather_kernel, dim3(row_grid(R)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(src), ld_src, row_src, n_rows_dev, topk, scale,
                       static_cast<uint16_t*>(dst), ld_dst, R, (int)(C / 8));
    return check_launch("moe_gather_kernel");
}

extern "C" int pp_moe_combine(const void* y, int64_t ld_y, const int32_t* pos, const float* gate, int topk,
                              const void* resid, int64_t ld_resid, void* out, int64_t ld_out, int64_t T,
                              int64_t C, pp_stream stream) {
    if (T < 0 || C < 0 || (C & 7) || topk < 1 || !pos || !rows_ok(y, ld_y) || !rows_ok(out, ld_out) ||
        ld_y < C || ld_out < C || (resid && (!rows_ok(resid, ld_resid) || ld_resid < C)))
        return fail(PP_ERR_INVALID, "pp_moe_combine: bad arguments (T=%lld C=%lld)", (long long)T, (long long)C);
    if (T == 0 || C == 0) return PP_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(row_grid(T)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(y), ld_y, pos, gate, topk, static_cast<const uint16_t*>(resid),
                       ld_resid, static_cast<uint16_t*>(out), ld_out, T, (int)(C / 8));
    return check_launch("moe_combine_kernel");
}

extern "C" int pp_moe_gate_bwd(const void* dout, int64_t ld_dout, const void* y, int64_t ld_y,
                               const int32_t* pos, const int32_t* topk_idx, const float* gate, int topk, int E,
                               void* dlogits, int64_t ld_dl, int64_t T, int64_t C, pp_stream stream) {
    if (T < 0 || C < 0 || (C & 7) || topk < 1 || topk > kMoeMaxTopk || E < 1 || !pos || !topk_idx || !gate ||
        !dlogits || ld_dl < ((E + 7) & ~7) || !rows_ok(dout, ld_dout) || !rows_ok(y, ld_y) || ld_dout < C || ld_y < C)
        return fail(PP_ERR_INVALID, "pp_moe_gate_bwd: bad arguments (T=%lld C=%lld topk=%d)", (long long)T,
                    (long long)C, topk);
    if (T == 0) return PP_OK;
    hipLaunchKernelGGL(moe_gate_bwd_kernel, dim3(row_grid(T)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(dout), ld_dout, static_cast<const uint16_t*>(y), ld_y, pos,
                       topk_idx, gate, topk, E, static_cast<uint16_t*>(dlogits), ld_dl, T, (int)(C / 8));
    return check_launch("moe_gate_bwd_kernel");
}
