// Token + position embedding lookup and its gradient (HBM-bound gathers / scatters).
#include "common.h"

namespace pp {

// One wave per token; each lane moves 16-byte chunks of the row.
__global__ __launch_bounds__(256) void embed_fwd_kernel(const int64_t* __restrict__ ids,
                                                        const uint16_t* __restrict__ wte,
                                                        const uint16_t* __restrict__ wpe,
                                                        const uint16_t* __restrict__ extra_row,
                                                        uint16_t* __restrict__ y, int64_t n_tok,
                                                        int64_t seq, int C, int64_t vocab,
                                                        const int64_t* __restrict__ pos_ids, int64_t n_pos) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tok) return;
    int64_t id = ids[t];
    // out-of-range ids read row 0 rather than faulting; callers validate ids on the host side
    if (id < 0 || id >= vocab) id = 0;
    const uint4* src = reinterpret_cast<const uint4*>(wte + id * C);
    // the row of the position table: t % seq, or the caller's own index (out of range reads row 0)
    int64_t p = t % seq;
    if (pos_ids) {
        p = pos_ids[t];
        if (p < 0 || p >= n_pos) p = 0;
    }
    const uint4* pos = wpe ? reinterpret_cast<const uint4*>(wpe + p * C) : nullptr;
    const uint4* ext = reinterpret_cast<const uint4*>(extra_row);
    uint4* dst = reinterpret_cast<uint4*>(y + t * C);
    for (int c = lane; c < (C >> 3); c += 64) {
        uint4 a = src[c];
        if (pos || ext) {
            // the sum is formed in fp32 and rounded once
            float f[8] = {bf16lo(a.x), bf16hi(a.x), bf16lo(a.y), bf16hi(a.y),
                          bf16lo(a.z), bf16hi(a.z), bf16lo(a.w), bf16hi(a.w)};
            if (pos) {
                const uint4 b = pos[c];
                f[0] += bf16lo(b.x); f[1] += bf16hi(b.x); f[2] += bf16lo(b.y); f[3] += bf16hi(b.y);
                f[4] += bf16lo(b.z); f[5] += bf16hi(b.z); f[6] += bf16lo(b.w); f[7] += bf16hi(b.w);
            }
            if (ext) {
                const uint4 b = ext[c];
                f[0] += bf16lo(b.x); f[1] += bf16hi(b.x); f[2] += bf16lo(b.y); f[3] += bf16hi(b.y);
                f[4] += bf16lo(b.z); f[5] += bf16hi(b.z); f[6] += bf16lo(b.w); f[7] += bf16hi(b.w);
            }
            a = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
        }
        dst[c] = a;
    }
}

// d_wte[id, :] += g[id, :] with g[id, :] the sum of dy[t, :] over the tokens t with ids[t] == id, added
// in ascending t (fp32) and, with round_bf16, rounded to bf16 before it is added: the same bits as a
// bf16 gradient tensor folded into the accumulator.  No atomics: one wave per token scans the ids; the
// wave of the first occurrence of an id owns that row and sums all occurrences in order, every other
// wave leaves at the first earlier occurrence it meets.  NW = 32-bit words (column pairs) per lane.
template <int NW>
__global__ __launch_bounds__(256) void embed_bwd_wte_kernel(const int64_t* __restrict__ ids,
                                                            const uint16_t* __restrict__ dy,
                                                            float* __restrict__ d_wte, int64_t n_tok,
                                                            int C, int64_t vocab, int round_bf16,
                                                            int64_t skip_id) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tok) return;
    const int64_t id = ids[t];
    // the padding row gets no gradient: its occurrences (often most of a padded batch, all owned by one
    // wave) are not summed at all
    if (id < 0 || id >= vocab || id == skip_id) return;
    const int half_c = C >> 1;
    float lo[NW], hi[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) lo[w] = hi[w] = 0.f;
    for (int64_t base = 0; base < n_tok; base += 64) {
        const int64_t idx = base + lane;
        uint64_t mask = __ballot(idx < n_tok && ids[idx] == id);
        if (base <= t) {
            // occurrences before t: another wave owns the row
            const uint64_t before = base + 64 <= t ? ~0ull : ((1ull << (t - base)) - 1ull);
            if (mask & before) return;
        }
        while (mask) {
            const int bit = __builtin_ctzll(mask);
            mask &= mask - 1;
            const uint32_t* src = reinterpret_cast<const uint32_t*>(dy + (base + bit) * C);
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const int c = w * 64 + lane;
                if (c < half_c) {
                    const uint32_t v = src[c];
                    lo[w] += bf16lo(v);
                    hi[w] += bf16hi(v);
                }
            }
        }
    }
    float* dst = d_wte + id * C;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const int c = w * 64 + lane;
        if (c < half_c) {
            float a = lo[w], b = hi[w];
            if (round_bf16) {
                const uint32_t r = pack_bf16(a, b);
                a = bf16lo(r);
                b = bf16hi(r);
            }
            float2* d2 = reinterpret_cast<float2*>(dst + 2 * c);
            const float2 old = *d2;
            *d2 = make_float2(old.x + a, old.y + b);
        }
    }
}

// d_wpe[p, :] += sum_b dy[b*seq + p, :]; each (p, column) has one owner, summed in batch order and,
// with round_bf16, rounded to bf16 before it is added.
__global__ __launch_bounds__(256) void embed_bwd_wpe_kernel(const uint16_t* __restrict__ dy,
                                                            float* __restrict__ d_wpe, int64_t n_tok,
                                                            int64_t seq, int C, int round_bf16) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // over seq * C/2
    const int half_c = C >> 1;
    if (idx >= seq * half_c) return;
    const int64_t p = idx / half_c;
    const int c = (int)(idx - p * half_c);
    float s0 = 0.f, s1 = 0.f;
    for (int64_t t = p; t < n_tok; t += seq) {
        const uint32_t w = reinterpret_cast<const uint32_t*>(dy + t * C)[c];
        s0 += bf16lo(w);
        s1 += bf16hi(w);
    }
    if (round_bf16) {
        const uint32_t r = pack_bf16(s0, s1);
        s0 = bf16lo(r);
        s1 = bf16hi(r);
    }
    float* dst = d_wpe + p * C + 2 * c;
    dst[0] += s0;
    dst[1] += s1;
}

// Positions counted over the tokens that are not padding: out[b, s] = pad for a padding token, else
// pad + the number of non-padding tokens among ids[b, 0..s].  One wave per sequence.
__global__ __launch_bounds__(64) void position_ids_kernel(const int64_t* __restrict__ ids,
                                                          int64_t* __restrict__ out, int64_t seq, int64_t pad) {
    const int lane = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.x * seq;
    int64_t running = 0;
    for (int64_t base = 0; base < seq; base += 64) {
        const int64_t s = base + lane;
        const bool real = s < seq && ids[row + s] != pad;
        const uint64_t mask = __ballot(real);
        const int upto = __builtin_popcountll(mask & ((lane == 63 ? ~0ull : ((1ull << (lane + 1)) - 1ull))));
        if (s < seq) out[row + s] = real ? pad + running + upto : pad;
        running += __builtin_popcountll(mask);
    }
}

template <int NW>
static void launch_embed_bwd_wte(const int64_t* ids, const void* dy, float* d_wte, int64_t n_tok, int C,
                                 int64_t vocab, int round_bf16, int64_t skip_id, hipStream_t st) {
    hipLaunchKernelGGL(embed_bwd_wte_kernel<NW>, dim3((uint32_t)((n_tok + 3) / 4)), dim3(256), 0, st, ids,
                       (const uint16_t*)dy, d_wte, n_tok, C, vocab, round_bf16, skip_id);
}

}  // namespace pp

using namespace pp;

extern "C" int pp_embed_fwd(const int64_t* ids, const void* wte, const void* wpe, const void* extra_row,
                            void* y, int64_t n_tok, int64_t seq, int64_t C, int64_t vocab, pp_stream stream) {
    if (n_tok < 0 || seq <= 0 || C <= 0 || vocab <= 0) return fail(PP_ERR_INVALID, "pp_embed_fwd: bad shape");
    if (C % 8) return fail(PP_ERR_UNSUPPORTED, "pp_embed_fwd: C %% 8 != 0");
    if (n_tok == 0) return PP_OK;
    if (!ids || !wte || !y) return fail(PP_ERR_INVALID, "pp_embed_fwd: null pointer");
    if (!aligned(wte, 16) || !aligned(wpe, 16) || !aligned(extra_row, 16) || !aligned(y, 16))
        return fail(PP_ERR_INVALID, "pp_embed_fwd: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(embed_fwd_kernel, dim3((uint32_t)((n_tok + 3) / 4)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), ids, (const uint16_t*)wte, (const uint16_t*)wpe,
                       (const uint16_t*)extra_row, (uint16_t*)y, n_tok, seq, (int)C, vocab,
                       (const int64_t*)nullptr, (int64_t)0);
    return check_launch("embed_fwd_kernel");
}

extern "C" int pp_embed_fwd_at(const int64_t* ids, const int64_t* pos_ids, const void* wte, const void* wpe,
                               const void* extra_row, void* y, int64_t n_tok, int64_t n_pos, int64_t C,
                               int64_t vocab, pp_stream stream) {
    if (n_tok < 0 || n_pos <= 0 || C <= 0 || vocab <= 0) return fail(PP_ERR_INVALID, "pp_embed_fwd_at: bad shape");
    if (C % 8) return fail(PP_ERR_UNSUPPORTED, "pp_embed_fwd_at: C %% 8 != 0");
    if (n_tok == 0) return PP_OK;
    if (!ids || !pos_ids || !wte || !wpe || !y) return fail(PP_ERR_INVALID, "pp_embed_fwd_at: null pointer");
    if (!aligned(wte, 16) || !aligned(wpe, 16) || !aligned(extra_row, 16) || !aligned(y, 16))
        return fail(PP_ERR_INVALID, "pp_embed_fwd_at: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(embed_fwd_kernel, dim3((uint32_t)((n_tok + 3) / 4)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), ids, (const uint16_t*)wte, (const uint16_t*)wpe,
                       (const uint16_t*)extra_row, (uint16_t*)y, n_tok, (int64_t)1, (int)C, vocab, pos_ids, n_pos);
    return check_launch("embed_fwd_kernel");
}

extern "C" int pp_position_ids_from_padding(const int64_t* ids, int64_t* out, int64_t n_seq, int64_t seq,
                                            int64_t pad, pp_stream stream) {
    if (n_seq < 0 || seq < 0) return fail(PP_ERR_INVALID, "pp_position_ids_from_padding: bad shape");
    if (n_seq == 0 || seq == 0) return PP_OK;
    if (!ids || !out) return fail(PP_ERR_INVALID, "pp_position_ids_from_padding: null pointer");
    if (n_seq > 0x7fffffff) return fail(PP_ERR_UNSUPPORTED, "pp_position_ids_from_padding: more than 2^31 - 1 sequences");
    hipLaunchKernelGGL(position_ids_kernel, dim3((uint32_t)n_seq), dim3(64), 0, static_cast<hipStream_t>(stream),
                       ids, out, seq, pad);
    return check_launch("position_ids_kernel");
}

extern "C" int pp_embed_bwd(const int64_t* ids, const void* dy, float* d_wte, float* d_wpe,
                            int64_t n_tok, int64_t seq, int64_t C, int64_t vocab, int round_bf16,
                            int64_t padding_idx, pp_stream stream) {
    if (n_tok < 0 || seq <= 0 || C <= 0 || vocab <= 0) return fail(PP_ERR_INVALID, "pp_embed_bwd: bad shape");
    if (C % 2) return fail(PP_ERR_UNSUPPORTED, "pp_embed_bwd: C %% 2 != 0");
    if (C > 8192) return fail(PP_ERR_UNSUPPORTED, "pp_embed_bwd: C > 8192");
    if (n_tok == 0) return PP_OK;
    if (!ids || !dy || !d_wte) return fail(PP_ERR_INVALID, "pp_embed_bwd: null pointer");
    if (!aligned(dy, 4) || !aligned(d_wte, 8)) return fail(PP_ERR_INVALID, "pp_embed_bwd: misaligned pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int words = (int)((C / 2 + 63) / 64);
    if (words <= 2) launch_embed_bwd_wte<2>(ids, dy, d_wte, n_tok, (int)C, vocab, round_bf16, padding_idx, st);
    else if (words <= 8) launch_embed_bwd_wte<8>(ids, dy, d_wte, n_tok, (int)C, vocab, round_bf16, padding_idx, st);
    else if (words <= 16) launch_embed_bwd_wte<16>(ids, dy, d_wte, n_tok, (int)C, vocab, round_bf16, padding_idx, st);
    else if (words <= 32) launch_embed_bwd_wte<32>(ids, dy, d_wte, n_tok, (int)C, vocab, round_bf16, padding_idx, st);
    else launch_embed_bwd_wte<64>(ids, dy, d_wte, n_tok, (int)C, vocab, round_bf16, padding_idx, st);
    if (d_wpe) {
        const int64_t work = seq * (C / 2);
        hipLaunchKernelGGL(embed_bwd_wpe_kernel, dim3((uint32_t)((work + 255) / 256)), dim3(256), 0, st,
                           (const uint16_t*)dy, d_wpe, n_tok, seq, (int)C, round_bf16);
    }
    return check_launch("embed_bwd");
}
