// Microbatch split / merge as coalesced row copies (HBM-bound, bit-exact).
//
// A split of a contiguous [outer, dim, inner] tensor along `dim`, and the concatenation that
// undoes it, both move `outer` rows per chunk where a row is a contiguous run of
// dim_chunk * inner elements.  One launch serves up to kMaxSegs such row segments; the widest
// vector (16/8/4/2/1 bytes) that divides every pointer, stride and row length is used.
#include "common.h"

namespace pp {

constexpr int kMaxSegs = 32;  // per launch; pp_copy_rows loops for longer tables
constexpr int kThreads = 256;
constexpr int kUnroll = 2;  // 8 KiB per work-group measured best for the logits merge

struct DevSeg {
    const char* src;
    char* dst;
    int64_t n_rows;
    int64_t row_bytes;
    int64_t src_stride;
    int64_t dst_stride;
    uint32_t col_blocks;      // blocks per row (>= 1); > 1 only when rows_per_block == 1
    uint32_t rows_per_block;  // rows handled by one block when a row is shorter than a tile
};

struct CopyTable {
    DevSeg seg[kMaxSegs];
    uint32_t block_start[kMaxSegs + 1];
    int n;
};

template <int V> struct VecT;
// native vector types: arrays of them stay in registers
typedef unsigned int copy_u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int copy_u32x2_t __attribute__((ext_vector_type(2)));
template <> struct VecT<16> { typedef copy_u32x4_t type; };
template <> struct VecT<8> { typedef copy_u32x2_t type; };
template <> struct VecT<4> { typedef uint32_t type; };
template <> struct VecT<2> { typedef uint16_t type; };
template <> struct VecT<1> { typedef uint8_t type; };

// Loads are unconditional (an index past the end is clamped to the last vector, whose value is then
// not stored): a load under a branch would keep the staging values out of registers.
template <int V>
__global__ __launch_bounds__(kThreads) void copy_rows_kernel(const CopyTable t) {
    typedef typename VecT<V>::type vec;
    uint32_t b = blockIdx.x;
    int s = 0;
    while (s + 1 < t.n && b >= t.block_start[s + 1]) ++s;
    b -= t.block_start[s];
    const DevSeg& g = t.seg[s];
    const int tid = threadIdx.x;

    if (g.rows_per_block == 1) {
        // long rows: this block owns one tile of one row
        const uint32_t row = b / g.col_blocks;
        const uint32_t cblk = b - row * g.col_blocks;
        const int64_t base = (int64_t)cblk * (kThreads * kUnroll * V);
        const char* sp = g.src + row * g.src_stride + base;
        char* dp = g.dst + row * g.dst_stride + base;
        const int64_t left = g.row_bytes - base;  // > 0, a multiple of V
        const int64_t last = left - V;
        vec r[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t off = (int64_t)(u * kThreads + tid) * V;
            r[u] = __builtin_nontemporal_load(reinterpret_cast<const vec*>(sp + (off < left ? off : last)));
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t off = (int64_t)(u * kThreads + tid) * V;
            if (off < left) __builtin_nontemporal_store(r[u], reinterpret_cast<vec*>(dp + off));
        }
    } else {
        // short rows: several whole rows per block
        const int64_t row0 = (int64_t)b * g.rows_per_block;
        int64_t nr = g.n_rows - row0;
        if (nr > g.rows_per_block) nr = g.rows_per_block;
        const uint32_t vpr = (uint32_t)(g.row_bytes / V);
        const uint32_t total = (uint32_t)nr * vpr;  // > 0
        for (uint32_t idx0 = 0; idx0 < total; idx0 += kThreads * kUnroll) {
            vec r[kUnroll];
            int64_t doff[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const uint32_t idx = idx0 + u * kThreads + tid;
                const uint32_t cl = idx < total ? idx : total - 1;
                const uint32_t rr = cl / vpr, cc = cl - rr * vpr;
                r[u] = *reinterpret_cast<const vec*>(g.src + (row0 + rr) * g.src_stride + (int64_t)cc * V);
                doff[u] = (row0 + rr) * g.dst_stride + (int64_t)cc * V;
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const uint32_t idx = idx0 + u * kThreads + tid;
                if (idx < total) *reinterpret_cast<vec*>(g.dst + doff[u]) = r[u];
            }
        }
    }
}

// Rows whose start is not 16-byte aligned (e.g. a row length of 50257 bf16 elements): the
// destination is aligned per row by a short scalar head, the body moves as aligned 16-byte stores
// fed by unaligned 16-byte loads, and a scalar tail finishes the row.  A = common alignment (bytes)
// of all pointers, strides and row lengths.
template <int A> struct Unaligned16;
#define PP_UNALIGNED16(A)                                                                    \
    template <> struct Unaligned16<A> {                                                      \
        typedef unsigned int type __attribute__((ext_vector_type(4), aligned(A)));          \
    };
PP_UNALIGNED16(1) PP_UNALIGNED16(2) PP_UNALIGNED16(4) PP_UNALIGNED16(8)
#undef PP_UNALIGNED16

template <int A>
__global__ __launch_bounds__(kThreads) void copy_rows_unaligned_kernel(const CopyTable t) {
    typedef typename VecT<A>::type elem;
    uint32_t b = blockIdx.x;
    int s = 0;
    while (s + 1 < t.n && b >= t.block_start[s + 1]) ++s;
    b -= t.block_start[s];
    const DevSeg& g = t.seg[s];
    const int tid = threadIdx.x;
    const int64_t row = b / g.col_blocks;
    const uint32_t cblk = b % g.col_blocks;
    const char* sp = g.src + row * g.src_stride;
    char* dp = g.dst + row * g.dst_stride;
    int64_t head = (16 - (reinterpret_cast<uintptr_t>(dp) & 15)) & 15;
    if (head > g.row_bytes) head = g.row_bytes;
    const int64_t nv = (g.row_bytes - head) >> 4;
    const int64_t v0 = (int64_t)cblk * (kThreads * kUnroll);
    uint4 r[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t vi = v0 + u * kThreads + tid;
        if (vi < nv) {
            typedef typename Unaligned16<A>::type src_vec;
            const copy_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const src_vec*>(sp + head + vi * 16));
            r[u] = make_uint4(v.x, v.y, v.z, v.w);
        }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int64_t vi = v0 + u * kThreads + tid;
        if (vi < nv) {
            const copy_u32x4_t w = {r[u].x, r[u].y, r[u].z, r[u].w};
            __builtin_nontemporal_store(w, reinterpret_cast<copy_u32x4_t*>(dp + head + vi * 16));
        }
    }
    if (cblk == 0) {
        for (int64_t i = (int64_t)tid * A; i < head; i += kThreads * A)
            *reinterpret_cast<elem*>(dp + i) = *reinterpret_cast<const elem*>(sp + i);
    }
    if (cblk == g.col_blocks - 1) {
        for (int64_t i = head + nv * 16 + (int64_t)tid * A; i < g.row_bytes; i += kThreads * A)
            *reinterpret_cast<elem*>(dp + i) = *reinterpret_cast<const elem*>(sp + i);
    }
}

template <int A>
static int launch_unaligned(const pp_copy_seg* segs, int n, hipStream_t stream) {
    CopyTable t;
    uint64_t blocks = 0;
    int m = 0;
    for (int i = 0; i < n; ++i) {
        const pp_copy_seg& s = segs[i];
        if (s.n_rows == 0 || s.row_bytes == 0) continue;
        DevSeg& d = t.seg[m];
        d.src = static_cast<const char*>(s.src);
        d.dst = static_cast<char*>(s.dst);
        d.n_rows = s.n_rows;
        d.row_bytes = s.row_bytes;
        d.src_stride = s.src_stride;
        d.dst_stride = s.dst_stride;
        d.rows_per_block = 1;
        const int64_t vecs = s.row_bytes / 16;
        const int64_t per = (int64_t)kThreads * kUnroll;
        d.col_blocks = (uint32_t)((vecs + per - 1) / per);
        if (d.col_blocks == 0) d.col_blocks = 1;
        t.block_start[m] = (uint32_t)blocks;
        blocks += (uint64_t)s.n_rows * d.col_blocks;
        if (blocks > 0x7fffffffull) return fail(PP_ERR_UNSUPPORTED, "pp_copy_rows: too many blocks");
        ++m;
    }
    if (m == 0) return PP_OK;
    t.block_start[m] = (uint32_t)blocks;
    t.n = m;
    hipLaunchKernelGGL(copy_rows_unaligned_kernel<A>, dim3((uint32_t)blocks), dim3(kThreads), 0, stream, t);
    return check_launch("copy_rows_unaligned_kernel");
}

static int pick_vec(const pp_copy_seg* segs, int n) {
    uint64_t bits = 0;
    for (int i = 0; i < n; ++i) {
        bits |= reinterpret_cast<uintptr_t>(segs[i].src) | reinterpret_cast<uintptr_t>(segs[i].dst) |
                (uint64_t)segs[i].row_bytes;
        if (segs[i].n_rows > 1) bits |= (uint64_t)segs[i].src_stride | (uint64_t)segs[i].dst_stride;
    }
    if ((bits & 15) == 0) return 16;
    if ((bits & 7) == 0) return 8;
    if ((bits & 3) == 0) return 4;
    if ((bits & 1) == 0) return 2;
    return 1;
}

template <int V>
static int launch_table(const pp_copy_seg* segs, int n, hipStream_t stream) {
    CopyTable t;
    const int64_t tile = (int64_t)kThreads * kUnroll * V;
    uint64_t blocks = 0;
    int m = 0;
    for (int i = 0; i < n; ++i) {
        const pp_copy_seg& s = segs[i];
        if (s.n_rows == 0 || s.row_bytes == 0) continue;
        DevSeg& d = t.seg[m];
        d.src = static_cast<const char*>(s.src);
        d.dst = static_cast<char*>(s.dst);
        d.n_rows = s.n_rows;
        d.row_bytes = s.row_bytes;
        d.src_stride = s.src_stride;
        d.dst_stride = s.dst_stride;
        uint64_t nb;
        if (s.row_bytes >= tile) {
            d.rows_per_block = 1;
            d.col_blocks = (uint32_t)((s.row_bytes + tile - 1) / tile);
            nb = (uint64_t)s.n_rows * d.col_blocks;
        } else {
            int64_t rpb = tile / s.row_bytes;
            if (rpb < 1) rpb = 1;
            if (rpb > 4096) rpb = 4096;
            d.rows_per_block = (uint32_t)rpb;
            d.col_blocks = 1;
            nb = (uint64_t)((s.n_rows + rpb - 1) / rpb);
            if (d.rows_per_block == 1) d.col_blocks = 1;
        }
        t.block_start[m] = (uint32_t)blocks;
        blocks += nb;
        if (blocks > 0x7fffffffull) return fail(PP_ERR_UNSUPPORTED, "pp_copy_rows: too many blocks");
        ++m;
    }
    if (m == 0) return PP_OK;
    t.block_start[m] = (uint32_t)blocks;
    t.n = m;
    hipLaunchKernelGGL(copy_rows_kernel<V>, dim3((uint32_t)blocks), dim3(kThreads), 0, stream, t);
    return check_launch("copy_rows_kernel");
}

static int copy_rows_impl(const pp_copy_seg* segs, int n_segs, hipStream_t stream) {
    for (int i = 0; i < n_segs; ++i) {
        const pp_copy_seg& s = segs[i];
        if (s.n_rows < 0 || s.row_bytes < 0)
            return fail(PP_ERR_INVALID, "pp_copy_rows: negative size in segment %d", i);
        if (s.n_rows > 0 && s.row_bytes > 0 && (!s.src || !s.dst))
            return fail(PP_ERR_INVALID, "pp_copy_rows: null pointer in segment %d", i);
        if (s.n_rows > 1 && (s.src_stride < s.row_bytes || s.dst_stride < s.row_bytes))
            return fail(PP_ERR_INVALID, "pp_copy_rows: stride shorter than row in segment %d", i);
    }
    for (int i0 = 0; i0 < n_segs; i0 += kMaxSegs) {
        const int n = (n_segs - i0 < kMaxSegs) ? n_segs - i0 : kMaxSegs;
        int rc;
        const int vec = pick_vec(segs + i0, n);
        bool long_rows = true;
        for (int i = 0; i < n; ++i)
            if (segs[i0 + i].n_rows > 0 && segs[i0 + i].row_bytes < 2048) long_rows = false;
        if (vec < 16 && long_rows) {
            switch (vec) {
                case 8: rc = launch_unaligned<8>(segs + i0, n, stream); break;
                case 4: rc = launch_unaligned<4>(segs + i0, n, stream); break;
                case 2: rc = launch_unaligned<2>(segs + i0, n, stream); break;
                default: rc = launch_unaligned<1>(segs + i0, n, stream); break;
            }
            if (rc != PP_OK) return rc;
            continue;
        }
        switch (vec) {
            case 16: rc = launch_table<16>(segs + i0, n, stream); break;
            case 8: rc = launch_table<8>(segs + i0, n, stream); break;
            case 4: rc = launch_table<4>(segs + i0, n, stream); break;
            case 2: rc = launch_table<2>(segs + i0, n, stream); break;
            default: rc = launch_table<1>(segs + i0, n, stream); break;
        }
        if (rc != PP_OK) return rc;
    }
    return PP_OK;
}

// ---- generic N-d strided gather ---------------------------------------------------------------
struct NdShape {
    int64_t size[8];
    int64_t stride[8];
    int ndim;
};

template <typename T>
__global__ __launch_bounds__(256) void strided_copy_nd_kernel(T* dst, const T* src, NdShape sh,
                                                              int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * 256) {
        int64_t rem = i, off = 0;
#pragma unroll
        for (int d = 7; d >= 0; --d) {
            if (d < sh.ndim) {
                const int64_t q = rem / sh.size[d];
                off += (rem - q * sh.size[d]) * sh.stride[d];
                rem = q;
            }
        }
        dst[i] = src[off];
    }
}

}  // namespace pp

using namespace pp;

extern "C" int pp_copy_rows(const pp_copy_seg* segs, int n_segs, pp_stream stream) {
    if (n_segs < 0 || (n_segs > 0 && !segs)) return fail(PP_ERR_INVALID, "pp_copy_rows: bad table");
    return copy_rows_impl(segs, n_segs, static_cast<hipStream_t>(stream));
}

extern "C" int pp_split_copy(const void* src, void* const* dsts, int n_chunks, int64_t outer,
                             int64_t dim, int64_t inner_bytes, pp_stream stream) {
    if (n_chunks < 1 || n_chunks > PP_COPY_MAX_SEGS)
        return fail(PP_ERR_INVALID, "pp_split_copy: n_chunks %d out of range", n_chunks);
    if (outer < 0 || dim < 0 || inner_bytes < 0 || !dsts)
        return fail(PP_ERR_INVALID, "pp_split_copy: bad shape");
    pp_copy_seg segs[PP_COPY_MAX_SEGS];
    const int64_t base = dim / n_chunks, extra = dim % n_chunks;
    int64_t lo = 0;
    for (int i = 0; i < n_chunks; ++i) {
        const int64_t d = base + (i < extra ? 1 : 0);
        segs[i].src = static_cast<const char*>(src) + lo * inner_bytes;
        segs[i].dst = dsts[i];
        segs[i].n_rows = (d > 0) ? outer : 0;
        segs[i].row_bytes = d * inner_bytes;
        segs[i].src_stride = dim * inner_bytes;
        segs[i].dst_stride = d * inner_bytes;
        lo += d;
    }
    return copy_rows_impl(segs, n_chunks, static_cast<hipStream_t>(stream));
}

extern "C" int pp_merge_copy(void* dst, const void* const* srcs, const int64_t* chunk_dims,
                             int n_chunks, int64_t outer, int64_t inner_bytes, pp_stream stream) {
    if (n_chunks < 1 || n_chunks > PP_COPY_MAX_SEGS)
        return fail(PP_ERR_INVALID, "pp_merge_copy: n_chunks %d out of range", n_chunks);
    if (outer < 0 || inner_bytes < 0 || !srcs || !chunk_dims)
        return fail(PP_ERR_INVALID, "pp_merge_copy: bad shape");
    int64_t dim = 0;
    for (int i = 0; i < n_chunks; ++i) {
        if (chunk_dims[i] < 0) return fail(PP_ERR_INVALID, "pp_merge_copy: negative chunk dim");
        dim += chunk_dims[i];
    }
    pp_copy_seg segs[PP_COPY_MAX_SEGS];
    int64_t lo = 0;
    for (int i = 0; i < n_chunks; ++i) {
        const int64_t d = chunk_dims[i];
        segs[i].src = srcs[i];
        segs[i].dst = static_cast<char*>(dst) + lo * inner_bytes;
        segs[i].n_rows = (d > 0) ? outer : 0;
        segs[i].row_bytes = d * inner_bytes;
        segs[i].src_stride = d * inner_bytes;
        segs[i].dst_stride = dim * inner_bytes;
        lo += d;
    }
    return copy_rows_impl(segs, n_chunks, static_cast<hipStream_t>(stream));
}

extern "C" int pp_strided_copy_nd(void* dst, const void* src, int ndim, const int64_t* sizes,
                                  const int64_t* src_strides, int elem_bytes, pp_stream stream) {
    if (ndim < 0 || ndim > 8) return fail(PP_ERR_INVALID, "pp_strided_copy_nd: ndim %d", ndim);
    NdShape sh;
    int64_t total = 1;
    for (int d = 0; d < 8; ++d) {
        sh.size[d] = 1;
        sh.stride[d] = 0;
    }
    for (int d = 0; d < ndim; ++d) {
        if (sizes[d] < 0) return fail(PP_ERR_INVALID, "pp_strided_copy_nd: negative size");
        sh.size[d] = sizes[d];
        sh.stride[d] = src_strides[d];
        total *= sizes[d];
    }
    sh.ndim = ndim;
    if (total == 0) return PP_OK;
    if (!dst || !src) return fail(PP_ERR_INVALID, "pp_strided_copy_nd: null pointer");
    int64_t nb = (total + 255) / 256;
    if (nb > 65536 * 16) nb = 65536 * 16;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (elem_bytes) {
        case 1: hipLaunchKernelGGL(strided_copy_nd_kernel<uint8_t>, dim3((uint32_t)nb), dim3(256), 0, st,
                                   (uint8_t*)dst, (const uint8_t*)src, sh, total); break;
        case 2: hipLaunchKernelGGL(strided_copy_nd_kernel<uint16_t>, dim3((uint32_t)nb), dim3(256), 0, st,
                                   (uint16_t*)dst, (const uint16_t*)src, sh, total); break;
        case 4: hipLaunchKernelGGL(strided_copy_nd_kernel<uint32_t>, dim3((uint32_t)nb), dim3(256), 0, st,
                                   (uint32_t*)dst, (const uint32_t*)src, sh, total); break;
        case 8: hipLaunchKernelGGL(strided_copy_nd_kernel<uint2>, dim3((uint32_t)nb), dim3(256), 0, st,
                                   (uint2*)dst, (const uint2*)src, sh, total); break;
        case 16: hipLaunchKernelGGL(strided_copy_nd_kernel<uint4>, dim3((uint32_t)nb), dim3(256), 0, st,
                                    (uint4*)dst, (const uint4*)src, sh, total); break;
        default: return fail(PP_ERR_UNSUPPORTED, "pp_strided_copy_nd: elem_bytes %d", elem_bytes);
    }
    return check_launch("strided_copy_nd_kernel");
}
