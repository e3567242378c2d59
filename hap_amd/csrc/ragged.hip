// Local halves of the uneven collectives: pad / unpad+concat / split+pad / slice /
// concat as multi-segment strided copies, and the rank-ordered float32 sum.
// All of these are HBM-bound; every thread moves 16-byte vectors, four in flight.
#include "common.h"

namespace {

struct Segment {
    const char *src;
    char *dst;
    int64_t rows;         // number of strided rows
    int64_t row_bytes;    // contiguous bytes per row
    int64_t src_stride;   // bytes between rows
    int64_t dst_stride;
};

struct SegmentList {
    int n;
    Segment seg[HAPMI_MAX_RANKS];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename V> struct ActNone {
    __device__ __forceinline__ V operator()(V v) const { return v; }
};
struct ReluBf16 {
    __device__ __forceinline__ u32x4 operator()(u32x4 v) const {
        // a bf16 is negative iff its sign bit is set; -0.0 -> +0.0 matches relu's value
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t lo = (v[i] & 0x8000u) ? 0u : (v[i] & 0xffffu);
            uint32_t hi = (v[i] & 0x80000000u) ? 0u : (v[i] & 0xffff0000u);
            r[i] = lo | hi;
        }
        return r;
    }
};
struct ReluF32 {
    __device__ __forceinline__ u32x4 operator()(u32x4 v) const {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = (v[i] & 0x80000000u) ? 0u : v[i];
        return r;
    }
};

constexpr int COPY_THREADS = 256;
constexpr int COPY_UNROLL = 4;

template <typename V, typename Act>
__global__ __launch_bounds__(COPY_THREADS) void segment_copy_kernel(SegmentList list, Act act) {
    const Segment s = list.seg[blockIdx.y];
    const uint64_t per_row = (uint64_t)s.row_bytes / sizeof(V);
    const uint64_t total = per_row * (uint64_t)s.rows;
    const uint64_t step = (uint64_t)gridDim.x * COPY_THREADS * COPY_UNROLL;
    for (uint64_t base = (uint64_t)blockIdx.x * COPY_THREADS * COPY_UNROLL + threadIdx.x; base < total; base += step) {
        V v[COPY_UNROLL];
        uint64_t doff[COPY_UNROLL];
        bool ok[COPY_UNROLL];
#pragma unroll
        for (int u = 0; u < COPY_UNROLL; ++u) {
            const uint64_t c = base + (uint64_t)u * COPY_THREADS;
            ok[u] = c < total;
            uint64_t row, col;
            if (s.rows == 1) {
                row = 0;
                col = c;
            } else if (total <= 0xffffffffull) {
                row = (uint32_t)c / (uint32_t)per_row;
                col = (uint32_t)c - (uint32_t)row * (uint32_t)per_row;
            } else {
                row = c / per_row;
                col = c - row * per_row;
            }
            doff[u] = row * (uint64_t)s.dst_stride + col * sizeof(V);
            if (ok[u]) v[u] = *(const V *)(s.src + row * (uint64_t)s.src_stride + col * sizeof(V));
        }
#pragma unroll
        for (int u = 0; u < COPY_UNROLL; ++u)
            if (ok[u]) *(V *)(s.dst + doff[u]) = act(v[u]);
    }
}

int launch_segments(const SegmentList &list, int act, int dtype, hipStream_t stream, const char *name) {
    if (list.n == 0) return HAPMI_OK;
    // widest vector that divides every address, stride and row length
    uint64_t bits = 0;
    int64_t max_chunks = 0;
    for (int i = 0; i < list.n; ++i) {
        const Segment &s = list.seg[i];
        bits |= (uint64_t)(uintptr_t)s.src | (uint64_t)(uintptr_t)s.dst | (uint64_t)s.row_bytes;
        if (s.rows > 1) bits |= (uint64_t)s.src_stride | (uint64_t)s.dst_stride;
    }
    int vec = 16;
    while (vec > 1 && (bits & (uint64_t)(vec - 1))) vec >>= 1;
    if (vec == 8) vec = 4;
    for (int i = 0; i < list.n; ++i) {
        const int64_t chunks = list.seg[i].rows * (list.seg[i].row_bytes / vec);
        if (chunks > max_chunks) max_chunks = chunks;
    }
    if (max_chunks == 0) return HAPMI_OK;
    int64_t gx = hapmi_cdiv(max_chunks, (int64_t)COPY_THREADS * COPY_UNROLL);
    const int64_t cap = hapmi_cdiv(256 * 16, list.n);   // ~16 blocks per CU over all segments
    if (gx > cap) gx = cap;
    if (gx < 1) gx = 1;
    dim3 grid((unsigned)gx, (unsigned)list.n), block(COPY_THREADS);
    if (act != HAPMI_ACT_NONE) {
        HAPMI_REQUIRE(act == HAPMI_ACT_RELU, HAPMI_EINVAL, "%s: only relu can be fused into a concat", name);
        HAPMI_REQUIRE(vec == 16, HAPMI_EALIGN, "%s: fused activation needs 16-byte aligned pieces", name);
        if (dtype == HAPMI_BF16)
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluBf16>), grid, block, 0, stream, list, ReluBf16());
        else
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluF32>), grid, block, 0, stream, list, ReluF32());
    } else if (vec == 16) {
        hipLaunchKernelGGL((segment_copy_kernel<u32x4, ActNone<u32x4>>), grid, block, 0, stream, list, ActNone<u32x4>());
    } else if (vec == 4) {
        hipLaunchKernelGGL((segment_copy_kernel<uint32_t, ActNone<uint32_t>>), grid, block, 0, stream, list,
                           ActNone<uint32_t>());
    } else if (vec == 2) {
        hipLaunchKernelGGL((segment_copy_kernel<uint16_t, ActNone<uint16_t>>), grid, block, 0, stream, list,
                           ActNone<uint16_t>());
    } else {
        hipLaunchKernelGGL((segment_copy_kernel<uint8_t, ActNone<uint8_t>>), grid, block, 0, stream, list,
                           ActNone<uint8_t>());
    }
    HAPMI_CHECK_LAUNCH(name);
    return HAPMI_OK;
}

int check_lengths(const int64_t *lengths, int n, int64_t *total, const char *name) {
    HAPMI_REQUIRE(n >= 1 && n <= HAPMI_MAX_RANKS && lengths, HAPMI_EINVAL, "%s: n_ranks %d outside 1..%d", name, n,
                  HAPMI_MAX_RANKS);
    int64_t t = 0;
    for (int i = 0; i < n; ++i) {
        HAPMI_REQUIRE(lengths[i] >= 0, HAPMI_EINVAL, "%s: negative length", name);
        t += lengths[i];
    }
    *total = t;
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_pad_rows(const void *src, void *dst, int64_t outer, int64_t len, int64_t padded_len,
                              int64_t inner_bytes, hapmi_stream_t stream) {
    HAPMI_REQUIRE(outer >= 0 && len >= 0 && padded_len >= len && inner_bytes > 0, HAPMI_EINVAL,
                  "pad_rows: bad shape outer=%lld len=%lld padded=%lld", (long long)outer, (long long)len,
                  (long long)padded_len);
    if (outer == 0 || len == 0) return HAPMI_OK;
    HAPMI_REQUIRE(src && dst, HAPMI_EINVAL, "pad_rows: null pointer");
    SegmentList list;
    list.n = 1;
    if (len == padded_len) list.seg[0] = {(const char *)src, (char *)dst, 1, outer * len * inner_bytes, 0, 0};
    else list.seg[0] = {(const char *)src, (char *)dst, outer, len * inner_bytes, len * inner_bytes, padded_len * inner_bytes};
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "pad_rows");
}

extern "C" int hapmi_slice_rows(const void *src, void *dst, int64_t outer, int64_t src_len, int64_t offset,
                                int64_t len, int64_t inner_bytes, hapmi_stream_t stream) {
    HAPMI_REQUIRE(outer >= 0 && len >= 0 && offset >= 0 && offset + len <= src_len && inner_bytes > 0, HAPMI_EINVAL,
                  "slice_rows: [%lld, %lld) outside 0..%lld", (long long)offset, (long long)(offset + len),
                  (long long)src_len);
    if (outer == 0 || len == 0) return HAPMI_OK;
    HAPMI_REQUIRE(src && dst, HAPMI_EINVAL, "slice_rows: null pointer");
    SegmentList list;
    list.n = 1;
    list.seg[0] = {(const char *)src + offset * inner_bytes, (char *)dst, outer, len * inner_bytes,
                   src_len * inner_bytes, len * inner_bytes};
    if (outer == 1) list.seg[0].rows = 1;
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "slice_rows");
}

extern "C" int hapmi_place_rows(const void *src, void *dst, int64_t outer, int64_t dst_len, int64_t offset,
                                int64_t len, int64_t inner_bytes, hapmi_stream_t stream) {
    HAPMI_REQUIRE(outer >= 0 && len >= 0 && offset >= 0 && offset + len <= dst_len && inner_bytes > 0, HAPMI_EINVAL,
                  "place_rows: [%lld, %lld) outside 0..%lld", (long long)offset, (long long)(offset + len),
                  (long long)dst_len);
    if (outer == 0 || len == 0) return HAPMI_OK;
    HAPMI_REQUIRE(src && dst, HAPMI_EINVAL, "place_rows: null pointer");
    SegmentList list;
    list.n = 1;
    list.seg[0] = {(const char *)src, (char *)dst + offset * inner_bytes, outer, len * inner_bytes,
                   len * inner_bytes, dst_len * inner_bytes};
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "place_rows");
}

extern "C" int hapmi_unpad_concat(const void *const *slices, const int64_t *lengths, int n_ranks, void *dst,
                                  int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_ranks, &total, "unpad_concat");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && slices, HAPMI_EINVAL, "unpad_concat: bad argument");
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_ranks; ++i) {
        HAPMI_REQUIRE(lengths[i] <= padded_len, HAPMI_EINVAL, "unpad_concat: length %lld above padded length %lld",
                      (long long)lengths[i], (long long)padded_len);
        if (lengths[i] > 0 && outer > 0) {
            HAPMI_REQUIRE(slices[i] && dst, HAPMI_EINVAL, "unpad_concat: null pointer");
            list.seg[list.n++] = {(const char *)slices[i], (char *)dst + off * inner_bytes, outer,
                                  lengths[i] * inner_bytes, padded_len * inner_bytes, total * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "unpad_concat");
}

extern "C" int hapmi_split_pad(const void *src, void *const *slices, const int64_t *lengths, int n_ranks,
                               int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_ranks, &total, "split_pad");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && slices, HAPMI_EINVAL, "split_pad: bad argument");
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_ranks; ++i) {
        HAPMI_REQUIRE(lengths[i] <= padded_len, HAPMI_EINVAL, "split_pad: length %lld above padded length %lld",
                      (long long)lengths[i], (long long)padded_len);
        if (lengths[i] > 0 && outer > 0) {
            HAPMI_REQUIRE(slices[i] && src, HAPMI_EINVAL, "split_pad: null pointer");
            list.seg[list.n++] = {(const char *)src + off * inner_bytes, (char *)slices[i], outer,
                                  lengths[i] * inner_bytes, total * inner_bytes, padded_len * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "split_pad");
}

extern "C" int hapmi_split_rows(const void *src, void *const *pieces, const int64_t *lengths, int n_ranks,
                                int64_t outer, int64_t inner_bytes, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_ranks, &total, "split_rows");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && pieces, HAPMI_EINVAL, "split_rows: bad argument");
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_ranks; ++i) {
        if (lengths[i] > 0 && outer > 0 && pieces[i]) {   // a NULL piece is skipped (not sent)
            HAPMI_REQUIRE(src, HAPMI_EINVAL, "split_rows: null pointer");
            list.seg[list.n++] = {(const char *)src + off * inner_bytes, (char *)pieces[i], outer,
                                  lengths[i] * inner_bytes, total * inner_bytes, lengths[i] * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "split_rows");
}

extern "C" int hapmi_concat_rows(const void *const *pieces, const int64_t *lengths, int n_ranks, void *dst,
                                 int64_t outer, int64_t inner_bytes, int act, int dtype, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_ranks, &total, "concat_rows");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && pieces, HAPMI_EINVAL, "concat_rows: bad argument");
    HAPMI_REQUIRE(act == HAPMI_ACT_NONE || hapmi_dtype_ok(dtype), HAPMI_EINVAL, "concat_rows: bad dtype");
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_ranks; ++i) {
        if (lengths[i] > 0 && outer > 0) {
            HAPMI_REQUIRE(pieces[i] && dst, HAPMI_EINVAL, "concat_rows: null pointer");
            list.seg[list.n++] = {(const char *)pieces[i], (char *)dst + off * inner_bytes, outer,
                                  lengths[i] * inner_bytes, lengths[i] * inner_bytes, total * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, act, dtype, (hipStream_t)stream, "concat_rows");
}

// ---------------------------------------------------------------------------
// rank-ordered sum with float32 accumulation
// ---------------------------------------------------------------------------
namespace {

struct ReduceArgs {
    int n;
    const void *src[HAPMI_MAX_RANKS];
};

constexpr int RED_THREADS = 256;

template <typename T, int NW>
__global__ __launch_bounds__(RED_THREADS) void ragged_reduce_kernel(ReduceArgs a, T *dst, int64_t outer,
                                                                   int64_t src_len, int64_t offset, int64_t len,
                                                                   int64_t inner, int n_dyn) {
    constexpr int EPV = Vec16<T>::N;
    const uint64_t vec_per_row = (uint64_t)(len * inner) / EPV;     // contiguous run per outer index
    const uint64_t total = vec_per_row * (uint64_t)outer;
    const uint64_t step = (uint64_t)gridDim.x * RED_THREADS;
    const int nw = NW > 0 ? NW : n_dyn;
    for (uint64_t c = (uint64_t)blockIdx.x * RED_THREADS + threadIdx.x; c < total; c += step) {
        uint64_t o = 0, col = c;
        if (outer > 1) {
            o = c / vec_per_row;
            col = c - o * vec_per_row;
        }
        const uint64_t soff = (o * (uint64_t)src_len + (uint64_t)offset) * (uint64_t)inner + col * EPV;
        float acc[EPV];
        if (NW > 0) {
            Vec16<T> v[NW > 0 ? NW : 1];
#pragma unroll
            for (int w = 0; w < NW; ++w) v[w] = *(const Vec16<T> *)((const T *)a.src[w] + soff);
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[e] = v[0].get(e);
#pragma unroll
            for (int w = 1; w < NW; ++w)
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[e] += v[w].get(e);
        } else {
            Vec16<T> v = *(const Vec16<T> *)((const T *)a.src[0] + soff);
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[e] = v.get(e);
            for (int w = 1; w < nw; ++w) {
                v = *(const Vec16<T> *)((const T *)a.src[w] + soff);
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[e] += v.get(e);
            }
        }
        Vec16<T> r;
#pragma unroll
        for (int e = 0; e < EPV; ++e) r.set(e, acc[e]);
        *(Vec16<T> *)(dst + (o * (uint64_t)len) * (uint64_t)inner + col * EPV) = r;
    }
}

template <typename T>
__global__ __launch_bounds__(RED_THREADS) void ragged_reduce_scalar_kernel(ReduceArgs a, T *dst, int64_t outer,
                                                                          int64_t src_len, int64_t offset,
                                                                          int64_t len, int64_t inner) {
    const uint64_t per = (uint64_t)(len * inner);
    const uint64_t total = per * (uint64_t)outer;
    const uint64_t step = (uint64_t)gridDim.x * RED_THREADS;
    for (uint64_t c = (uint64_t)blockIdx.x * RED_THREADS + threadIdx.x; c < total; c += step) {
        const uint64_t o = c / per, col = c - o * per;
        const uint64_t soff = (o * (uint64_t)src_len + (uint64_t)offset) * (uint64_t)inner + col;
        float acc = ld_f((const T *)a.src[0], soff);
        for (int w = 1; w < a.n; ++w) acc += ld_f((const T *)a.src[w], soff);
        st_f(dst, c, acc);
    }
}

template <typename T>
int launch_reduce(const ReduceArgs &a, void *dst, int64_t outer, int64_t src_len, int64_t offset, int64_t len,
                  int64_t inner, hipStream_t stream) {
    constexpr int EPV = Vec16<T>::N;
    const int64_t esz = sizeof(T);
    bool vec_ok = ((len * inner) % EPV == 0) && ((src_len * inner) % EPV == 0) && ((offset * inner) % EPV == 0) &&
                  ((uintptr_t)dst % 16 == 0);
    for (int w = 0; w < a.n; ++w) vec_ok = vec_ok && ((uintptr_t)a.src[w] % 16 == 0);
    (void)esz;
    if (vec_ok) {
        const int64_t total = outer * (len * inner / EPV);
        int64_t gx = hapmi_cdiv(total, RED_THREADS);
        if (gx > 256 * 16) gx = 256 * 16;
        dim3 grid((unsigned)gx), block(RED_THREADS);
        switch (a.n) {
#define HAPMI_RED_CASE(NW)                                                                                   \
    case NW:                                                                                                 \
        hipLaunchKernelGGL((ragged_reduce_kernel<T, NW>), grid, block, 0, stream, a, (T *)dst, outer, src_len, \
                           offset, len, inner, a.n);                                                         \
        break;
            HAPMI_RED_CASE(1)
            HAPMI_RED_CASE(2)
            HAPMI_RED_CASE(4)
            HAPMI_RED_CASE(8)
#undef HAPMI_RED_CASE
            default:
                hipLaunchKernelGGL((ragged_reduce_kernel<T, 0>), grid, block, 0, stream, a, (T *)dst, outer, src_len,
                                   offset, len, inner, a.n);
        }
    } else {
        const int64_t total = outer * len * inner;
        int64_t gx = hapmi_cdiv(total, RED_THREADS);
        if (gx > 256 * 16) gx = 256 * 16;
        hipLaunchKernelGGL((ragged_reduce_scalar_kernel<T>), dim3((unsigned)gx), dim3(RED_THREADS), 0, stream, a,
                           (T *)dst, outer, src_len, offset, len, inner);
    }
    HAPMI_CHECK_LAUNCH("ragged_reduce");
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_ragged_reduce(const void *const *contribs, int n_ranks, void *dst, int64_t outer,
                                   int64_t src_len, int64_t offset, int64_t len, int64_t inner, int dtype,
                                   hapmi_stream_t stream) {
    HAPMI_REQUIRE(n_ranks >= 1 && n_ranks <= HAPMI_MAX_RANKS && contribs, HAPMI_EINVAL,
                  "ragged_reduce: n_ranks %d outside 1..%d", n_ranks, HAPMI_MAX_RANKS);
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "ragged_reduce: bad dtype %d", dtype);
    HAPMI_REQUIRE(outer >= 0 && len >= 0 && inner > 0 && offset >= 0 && offset + len <= src_len, HAPMI_EINVAL,
                  "ragged_reduce: [%lld, %lld) outside 0..%lld", (long long)offset, (long long)(offset + len),
                  (long long)src_len);
    if (outer == 0 || len == 0) return HAPMI_OK;
    ReduceArgs a;
    a.n = n_ranks;
    for (int w = 0; w < n_ranks; ++w) {
        HAPMI_REQUIRE(contribs[w], HAPMI_EINVAL, "ragged_reduce: contribution %d is NULL", w);
        a.src[w] = contribs[w];
    }
    HAPMI_REQUIRE(dst, HAPMI_EINVAL, "ragged_reduce: null destination");
    if (dtype == HAPMI_F32) return launch_reduce<float>(a, dst, outer, src_len, offset, len, inner, (hipStream_t)stream);
    return launch_reduce<bf16_t>(a, dst, outer, src_len, offset, len, inner, (hipStream_t)stream);
}
