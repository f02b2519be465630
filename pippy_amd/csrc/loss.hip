// Cross-entropy (mean over non-ignored rows) fused with its gradient w.r.t. the logits.
// HBM-bound: each logits row is read from memory once and kept in registers across the max,
// sum-of-exponentials and gradient passes; the gradient row is written once.
#include "common.h"
#include <math.h>

namespace pp {

// ws[rows] = number of valid targets, ws[rows + 1] = 1 / max(count, 1)
__global__ __launch_bounds__(256) void ce_count_kernel(const int64_t* __restrict__ target, int64_t rows,
                                                       int64_t V, int64_t ignore_index,
                                                       float* __restrict__ ws) {
    __shared__ int part[4];
    int c = 0;
    for (int64_t r = threadIdx.x; r < rows; r += 256) {
        const int64_t t = target[r];
        c += (t != ignore_index && t >= 0 && t < V) ? 1 : 0;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        const int n = part[0] + part[1] + part[2] + part[3];
        ws[rows] = (float)n;
        ws[rows + 1] = 1.0f / (float)(n > 0 ? n : 1);
    }
}

constexpr int kCeThreads = 1024;
constexpr float kLog2e = 1.44269504088896340736f;

__device__ __forceinline__ float block_reduce_max(float v, float* sh) {
    v = wave_max(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = sh[0];
#pragma unroll
    for (int i = 1; i < kCeThreads / 64; ++i) r = fmaxf(r, sh[i]);
    return r;
}
__device__ __forceinline__ float block_reduce_sum(float v, float* sh) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < kCeThreads / 64; ++i) r += sh[i];
    return r;
}

// bf16 logits, one work-group per row, NC 16-byte chunks per lane held in registers.
// The kernel is bound by VALU issue as much as by HBM, so the per-element work is kept minimal:
// columns past V are turned into -inf when the row is loaded (no bounds checks afterwards), the
// exponentials exp(x - max) of the sum pass replace the logits in the registers (as bf16) and the
// gradient pass only scales them; the "- 1" of the target column is patched into the chunk that
// holds it before that chunk is stored.
// Rows are read and written through buffer instructions: one VGPR byte offset per lane serves every
// chunk (the chunk's 16 KiB stride is a scalar offset), which keeps the kernel within 64 VGPRs, so
// that two work-groups of 16 waves share a CU and one row's store phase overlaps the other's load
// phase; chunks past the row's end read as zero and are not written.
typedef unsigned int ce_u32x4_t __attribute__((ext_vector_type(4)));

template <int NC>
__global__ __launch_bounds__(kCeThreads, 8) void ce_row_bf16_kernel(
    const uint16_t* __restrict__ logits, const int64_t* __restrict__ target, uint16_t* __restrict__ dlogits,
    float* __restrict__ ws, int64_t rows, int V, int64_t ld, int64_t ignore_index) {
    __shared__ float sh[kCeThreads / 64];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const uint16_t* xr = logits + row * ld;
    const int nchunk_v = (V + 7) >> 3;          // chunks holding at least one valid column
    constexpr uint32_t kNegInf2 = 0xff80ff80u;  // two bf16 -inf
    const __amdgpu_buffer_rsrc_t src =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(xr), 0, nchunk_v * 16, 0x00020000);
    const int voff = tid * 16;
    uint4 w[NC];
#pragma unroll
    for (int i = 0; i < NC; ++i) {
        const ce_u32x4_t r = __builtin_amdgcn_raw_buffer_load_b128(src, voff, i * kCeThreads * 16, 0);
        w[i] = make_uint4(r.x, r.y, r.z, r.w);
    }
#pragma unroll
    for (int i = 0; i < NC; ++i) {
        const int c = tid + kCeThreads * i;
        if (c * 8 + 8 > V) {  // the chunk that straddles V, and the chunks past it
            uint32_t u[4] = {w[i].x, w[i].y, w[i].z, w[i].w};
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (c * 8 + e >= V)
                    u[e >> 1] = (e & 1) ? ((u[e >> 1] & 0x0000ffffu) | 0xff800000u)
                                        : ((u[e >> 1] & 0xffff0000u) | 0x0000ff80u);
            w[i] = make_uint4(u[0], u[1], u[2], u[3]);
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
        mx = fmaxf(mx, fmaxf(fmaxf(bf16lo(w[i].x), bf16hi(w[i].x)), fmaxf(bf16lo(w[i].y), bf16hi(w[i].y))));
        mx = fmaxf(mx, fmaxf(fmaxf(bf16lo(w[i].z), bf16hi(w[i].z)), fmaxf(bf16lo(w[i].w), bf16hi(w[i].w))));
        __builtin_amdgcn_sched_barrier(0);  // one chunk's temporaries at a time
    }
    mx = block_reduce_max(mx, sh);
    // The row stays packed across the reduction: without this the compiler keeps the 8 * NC unpacked
    // values of the max pass alive for the sum pass, which doubles the kernel's registers.
#pragma unroll
    for (int i = 0; i < NC; ++i) asm volatile("" : "+v"(w[i].x), "+v"(w[i].y), "+v"(w[i].z), "+v"(w[i].w));
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NC; ++i) {
        const float f[8] = {bf16lo(w[i].x), bf16hi(w[i].x), bf16lo(w[i].y), bf16hi(w[i].y),
                            bf16lo(w[i].z), bf16hi(w[i].z), bf16lo(w[i].w), bf16hi(w[i].w)};
        float ex[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            ex[e] = __builtin_amdgcn_exp2f((f[e] - mx) * kLog2e);
            s += ex[e];
        }
        w[i] = make_uint4(pack_bf16(ex[0], ex[1]), pack_bf16(ex[2], ex[3]), pack_bf16(ex[4], ex[5]),
                          pack_bf16(ex[6], ex[7]));
        // pack here, not where the values are used: the fp32 exponentials must not stay alive
        asm volatile("" : "+v"(w[i].x), "+v"(w[i].y), "+v"(w[i].z), "+v"(w[i].w));
        __builtin_amdgcn_sched_barrier(0);
    }
    s = block_reduce_sum(s, sh);
    const float lse = mx + logf(s);
    const int64_t t = target[row];
    const bool valid = (t != ignore_index && t >= 0 && t < V);
    const float xt = valid ? bf16_to_f32(xr[t]) : 0.f;
    if (tid == 0) ws[row] = valid ? (lse - xt) : 0.f;
    if (!dlogits) return;
    const float scale = valid ? ws[rows + 1] : 0.f;
    const float ps = scale / s;  // exp(x - max) * ps = softmax * scale
    uint16_t* dr = dlogits + row * ld;
    // ld / 8 chunks are written (padding columns get exp(-inf) * ps = 0); stores past them are dropped
    const __amdgpu_buffer_rsrc_t dst = __builtin_amdgcn_make_buffer_rsrc(dr, 0, (int)(ld >> 3) * 16, 0x00020000);
    // the target column gets softmax - 1: patched into its chunk by the lane that stores it
    const int tc = valid ? (int)(t >> 3) : -1;
    const uint32_t corr = f32_to_bf16((__builtin_amdgcn_exp2f((xt - mx) * kLog2e) / s - 1.0f) * scale);
#pragma unroll
    for (int i = 0; i < NC; ++i) {
        ce_u32x4_t o = {pack_bf16(bf16lo(w[i].x) * ps, bf16hi(w[i].x) * ps),
                        pack_bf16(bf16lo(w[i].y) * ps, bf16hi(w[i].y) * ps),
                        pack_bf16(bf16lo(w[i].z) * ps, bf16hi(w[i].z) * ps),
                        pack_bf16(bf16lo(w[i].w) * ps, bf16hi(w[i].w) * ps)};
        if (tid + kCeThreads * i == tc) {
            const int e = (int)(t & 7);
            const uint32_t keep = (e & 1) ? 0x0000ffffu : 0xffff0000u, put = (e & 1) ? (corr << 16) : corr;
            if ((e >> 1) == 0) o.x = (o.x & keep) | put;
            if ((e >> 1) == 1) o.y = (o.y & keep) | put;
            if ((e >> 1) == 2) o.z = (o.z & keep) | put;
            if ((e >> 1) == 3) o.w = (o.w & keep) | put;
        }
        __builtin_amdgcn_raw_buffer_store_b128(o, dst, voff, i * kCeThreads * 16, 0);
        // The next chunk's arithmetic reuses the registers this store reads.  The compiler pads a
        // 128-bit buffer store with wait states only when its scalar offset is not a register; with
        // the offset in an SGPR some lanes were seen to store the overwritten value, so pad by hand.
        asm volatile("s_nop 3");
        __builtin_amdgcn_sched_barrier(0);
    }
}

// fp32 logits (small class counts): one wave per row, three passes over the row.
__global__ __launch_bounds__(256) void ce_row_f32_kernel(const float* __restrict__ logits,
                                                         const int64_t* __restrict__ target,
                                                         float* __restrict__ dlogits, float* __restrict__ ws,
                                                         int64_t rows, int V, int64_t ld,
                                                         int64_t ignore_index) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* xr = logits + row * ld;
    float mx = -INFINITY;
    for (int c = lane; c < V; c += 64) mx = fmaxf(mx, xr[c]);
    mx = wave_max(mx);
    float s = 0.f;
    for (int c = lane; c < V; c += 64) s += expf(xr[c] - mx);
    s = wave_sum(s);
    const float lse = mx + logf(s);
    const int64_t t = target[row];
    const bool valid = (t != ignore_index && t >= 0 && t < V);
    if (lane == 0) ws[row] = valid ? (lse - xr[valid ? t : 0]) : 0.f;
    if (!dlogits) return;
    const float scale = valid ? ws[rows + 1] : 0.f;
    float* dr = dlogits + row * ld;
    for (int c = lane; c < ld; c += 64)
        dr[c] = (c < V) ? (expf(xr[c] - lse) - (c == t ? 1.0f : 0.0f)) * scale : 0.f;
}

// loss = (sum_r ws[r]) / count, summed in a fixed order; NaN when every row is ignored (the mean over no
// rows, as torch.nn.functional.cross_entropy returns it; the gradient is zero then)
__global__ __launch_bounds__(256) void ce_finalize_kernel(const float* __restrict__ ws, int64_t rows,
                                                          float* __restrict__ loss) {
    __shared__ float part[256];
    float s = 0.f;
    for (int64_t r = threadIdx.x; r < rows; r += 256) s += ws[r];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = ws[rows] > 0.f ? part[0] * ws[rows + 1] : __builtin_nanf("");
}

}  // namespace pp

using namespace pp;

extern "C" int pp_ce_loss(const void* logits, const int64_t* target, float* loss, void* dlogits,
                          float* workspace, int64_t rows, int64_t V, int64_t ld, int64_t ignore_index,
                          int logits_dtype, pp_stream stream) {
    if (rows < 0 || V <= 0 || ld < V) return fail(PP_ERR_INVALID, "pp_ce_loss: bad shape");
    if (!logits || !target || !loss || !workspace) return fail(PP_ERR_INVALID, "pp_ce_loss: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(ce_count_kernel, dim3(1), dim3(256), 0, st, target, rows, V, ignore_index, workspace);
    if (rows > 0) {
        if (logits_dtype == PP_F32) {
            hipLaunchKernelGGL(ce_row_f32_kernel, dim3((uint32_t)((rows + 3) / 4)), dim3(256), 0, st,
                               (const float*)logits, target, (float*)dlogits, workspace, rows, (int)V, ld,
                               ignore_index);
        } else {
            if ((ld % 8) || !aligned(logits, 16) || !aligned(dlogits, 16))
                return fail(PP_ERR_INVALID, "pp_ce_loss: bf16 logits need ld %% 8 == 0 and 16-byte alignment");
            const int64_t chunks = ld / 8;
            const int nc = (int)((chunks + kCeThreads - 1) / kCeThreads);
            const dim3 grid((uint32_t)rows), block(kCeThreads);
#define PP_CE_LAUNCH(NC)                                                                              \
    hipLaunchKernelGGL(ce_row_bf16_kernel<NC>, grid, block, 0, st, (const uint16_t*)logits, target,   \
                       (uint16_t*)dlogits, workspace, rows, (int)V, ld, ignore_index)
            if (nc <= 1) PP_CE_LAUNCH(1);
            else if (nc <= 2) PP_CE_LAUNCH(2);
            else if (nc <= 4) PP_CE_LAUNCH(4);
            else if (nc <= 8) PP_CE_LAUNCH(8);
            else return fail(PP_ERR_UNSUPPORTED, "pp_ce_loss: more than 65536 classes");
#undef PP_CE_LAUNCH
        }
    }
    hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(256), 0, st, workspace, rows, loss);
    return check_launch("ce_loss");
}
