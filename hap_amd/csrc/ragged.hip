// Local halves of the uneven collectives: pad / unpad+concat / split+pad / slice /
// concat as multi-segment strided copies, and the rank-ordered float32 sum.
// All of these are HBM-bound; every thread moves 16-byte vectors, four in flight.
#include "common.h"
#include "dropout.h"

namespace {

constexpr int kGridShift = 2;   // grid cap = 4096 << shift blocks

struct Segment {
    const char *src;
    char *dst;
    int64_t rows;         // number of strided rows
    int64_t row_bytes;    // contiguous bytes per row
    int64_t src_stride;   // bytes between rows
    int64_t dst_stride;
    // for functors that need to know which element of a tensor they hold (dropout): byte offset of the segment's
    // first element in that tensor and the bytes between its rows there
    int64_t index_first = 0, index_stride = 0;
};

struct SegmentList {
    int n;
    Segment seg[HAPMI_MAX_RANKS];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename V> struct ActNone {
    static constexpr bool MASKED = false, INDEXED = false;
    __device__ __forceinline__ V operator()(V v) const { return v; }
};
// relu's backward fused into a copy: the element is kept where the forward output, which lies `delta` bytes from
// the source element, is > 0 (NaN counts as not positive, as `y > 0.f` does)
struct ReluBwdBf16 {
    static constexpr bool MASKED = true, INDEXED = false;
    int64_t delta;
    __device__ __forceinline__ u32x4 operator()(u32x4 v, u32x4 y) const {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t lo = y[i] & 0xffffu, hi = y[i] >> 16;
            const uint32_t klo = (lo - 1u) < 0x7f80u ? 0xffffu : 0u;          // 0x0001..0x7f80: positive, not NaN
            const uint32_t khi = (hi - 1u) < 0x7f80u ? 0xffff0000u : 0u;
            r[i] = v[i] & (klo | khi);
        }
        return r;
    }
};
struct ReluBwdF32 {
    static constexpr bool MASKED = true, INDEXED = false;
    int64_t delta;
    __device__ __forceinline__ u32x4 operator()(u32x4 v, u32x4 y) const {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = (y[i] - 1u) < 0x7f800000u ? v[i] : 0u;
        return r;
    }
};
struct ReluBf16 {
    static constexpr bool MASKED = false, INDEXED = false;
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
    static constexpr bool MASKED = false, INDEXED = false;
    __device__ __forceinline__ u32x4 operator()(u32x4 v) const {
        u32x4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = (v[i] & 0x80000000u) ? 0u : v[i];
        return r;
    }
};

// relu's backward times a constant: the backward of relu followed by dropout, given the DROPPED forward output (it is
// positive exactly where relu passed the element and dropout kept it; the constant is dropout's 1 / (1 - p))
template <typename T> struct ReluBwdScaled {
    static constexpr bool MASKED = true, INDEXED = false;
    int64_t delta;
    float scale;
    __device__ __forceinline__ u32x4 operator()(u32x4 v, u32x4 y) const {
        union { u32x4 u; Vec16<T> e; } g, m;
        g.u = v;
        m.u = y;
#pragma unroll
        for (int i = 0; i < Vec16<T>::N; ++i) g.e.set(i, m.e.get(i) > 0.f ? g.e.get(i) * scale : 0.f);
        return g.u;
    }
};
// relu followed by dropout on the copied elements; the decision for an element is the one the elementwise dropout
// kernel takes for its index in the tensor that the segments' index_first / index_stride refer to
template <typename T> struct ReluDrop {
    static constexpr bool MASKED = false, INDEXED = true;
    const int64_t *state;
    int64_t stream_id;
    float p;
    __device__ __forceinline__ DropKey key() const { return drop_key(state[0], state[1], stream_id, p); }
    // at: byte offset of the 16 bytes in that tensor (a multiple of 16: an even element index)
    __device__ __forceinline__ u32x4 operator()(u32x4 v, uint64_t at, const DropKey &k) const {
        union { u32x4 u; Vec16<T> e; } x;
        x.u = v;
        const uint64_t first = at / sizeof(T);
#pragma unroll
        for (int i = 0; i < Vec16<T>::N; i += 2) {
            const uint32_t bits = drop_pair_bits(k, (first + i) >> 1);
            const float a = x.e.get(i), b = x.e.get(i + 1);
            x.e.set(i, (a > 0.f && (bits & 0xffffU) >= k.thr) ? a * k.scale : 0.f);
            x.e.set(i + 1, (b > 0.f && (bits >> 16) >= k.thr) ? b * k.scale : 0.f);
        }
        return x.u;
    }
};

constexpr int COPY_THREADS = 256;
constexpr int COPY_UNROLL = 4;

template <typename V, typename Act, bool NT = false>
__global__ __launch_bounds__(COPY_THREADS) void segment_copy_kernel(SegmentList list, Act act) {
    const Segment s = list.seg[blockIdx.y];
    const uint64_t per_row = (uint64_t)s.row_bytes / sizeof(V);
    const uint64_t total = per_row * (uint64_t)s.rows;
    const uint64_t step = (uint64_t)gridDim.x * COPY_THREADS * COPY_UNROLL;
    DropKey key;
    if constexpr (Act::INDEXED) key = act.key();
    for (uint64_t base = (uint64_t)blockIdx.x * COPY_THREADS * COPY_UNROLL + threadIdx.x; base < total; base += step) {
        V v[COPY_UNROLL], y[Act::MASKED ? COPY_UNROLL : 1];
        uint64_t doff[COPY_UNROLL], ioff[Act::INDEXED ? COPY_UNROLL : 1];
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
            if constexpr (Act::INDEXED) ioff[u] = (uint64_t)s.index_first + row * (uint64_t)s.index_stride + col * sizeof(V);
            const char *from = s.src + row * (uint64_t)s.src_stride + col * sizeof(V);
            if (ok[u]) {
                if constexpr (NT) v[u] = __builtin_nontemporal_load((const V *)from);
                else v[u] = *(const V *)from;
            }
            if constexpr (Act::MASKED)
                if (ok[u]) y[u] = *(const V *)(from + act.delta);
        }
#pragma unroll
        for (int u = 0; u < COPY_UNROLL; ++u) {
            if (!ok[u]) continue;
            if constexpr (Act::MASKED) *(V *)(s.dst + doff[u]) = act(v[u], y[u]);
            else if constexpr (Act::INDEXED) *(V *)(s.dst + doff[u]) = act(v[u], ioff[u], key);
            else *(V *)(s.dst + doff[u]) = act(v[u]);
        }
    }
}

// act: HAPMI_ACT_NONE, HAPMI_ACT_RELU (applied to the copied elements), or ACT_RELU_BWD (elements kept where the
// element `mask_delta` bytes after the source element is > 0)
// ACT_RELU_BWD with scale != 1: the kept elements are multiplied by scale.  ACT_RELU_DROP: relu, then dropout as
// DropSpec describes it.
constexpr int ACT_RELU_BWD = -1, ACT_RELU_DROP = -2;
struct DropSpec {
    const int64_t *state;
    int64_t stream_id;
    float p;
};
int launch_segments(const SegmentList &list, int act, int dtype, hipStream_t stream, const char *name,
                    int64_t mask_delta = 0, float scale = 1.f, const DropSpec *drop = nullptr) {
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
    const int64_t cap = hapmi_cdiv((int64_t)(256 * 16) << kGridShift, list.n);   // blocks over all segments
    if (gx > cap) gx = cap;
    if (gx < 1) gx = 1;
    dim3 grid((unsigned)gx, (unsigned)list.n), block(COPY_THREADS);
    if (act == ACT_RELU_BWD) {
        HAPMI_REQUIRE(vec == 16 && mask_delta % 16 == 0, HAPMI_EALIGN, "%s: the fused relu backward needs 16-byte aligned pieces", name);
        if (scale != 1.f && dtype == HAPMI_BF16)
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluBwdScaled<bf16_t>>), grid, block, 0, stream, list,
                               ReluBwdScaled<bf16_t>{mask_delta, scale});
        else if (scale != 1.f)
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluBwdScaled<float>>), grid, block, 0, stream, list,
                               ReluBwdScaled<float>{mask_delta, scale});
        else if (dtype == HAPMI_BF16)
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluBwdBf16>), grid, block, 0, stream, list, ReluBwdBf16{mask_delta});
        else
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluBwdF32>), grid, block, 0, stream, list, ReluBwdF32{mask_delta});
    } else if (act == ACT_RELU_DROP) {
        bool idx_ok = drop != nullptr;
        for (int i = 0; i < list.n; ++i) idx_ok = idx_ok && ((list.seg[i].index_first | list.seg[i].index_stride) & 15) == 0;
        HAPMI_REQUIRE(vec == 16 && idx_ok, HAPMI_EALIGN, "%s: relu + dropout needs 16-byte aligned pieces", name);
        if (dtype == HAPMI_BF16)
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluDrop<bf16_t>>), grid, block, 0, stream, list,
                               ReluDrop<bf16_t>{drop->state, drop->stream_id, drop->p});
        else
            hipLaunchKernelGGL((segment_copy_kernel<u32x4, ReluDrop<float>>), grid, block, 0, stream, list,
                               ReluDrop<float>{drop->state, drop->stream_id, drop->p});
    } else if (act != HAPMI_ACT_NONE) {
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
            // a slice that was received at its place in dst (outer = 1: one contiguous range) stays where it is
            if (outer == 1 && (const char *)slices[i] == (const char *)dst + off * inner_bytes) {
                off += lengths[i];
                continue;
            }
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
        if (lengths[i] > 0 && outer > 0 && slices[i]) {       // a NULL slice is skipped (a piece nobody needs)
            HAPMI_REQUIRE(src, HAPMI_EINVAL, "split_pad: null pointer");
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

namespace {
int split_rows_relu_bwd(const void *src, const void *fwd_out, void *const *pieces, const int64_t *lengths, int n_ranks,
                        int64_t outer, int64_t inner_bytes, float scale, int dtype, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_ranks, &total, "split_rows_relu_bwd");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && pieces, HAPMI_EINVAL, "split_rows_relu_bwd: bad argument");
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "split_rows_relu_bwd: bad dtype %d", dtype);
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_ranks; ++i) {
        if (lengths[i] > 0 && outer > 0 && pieces[i]) {
            HAPMI_REQUIRE(src && fwd_out, HAPMI_EINVAL, "split_rows_relu_bwd: null pointer");
            list.seg[list.n++] = {(const char *)src + off * inner_bytes, (char *)pieces[i], outer,
                                  lengths[i] * inner_bytes, total * inner_bytes, lengths[i] * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, ACT_RELU_BWD, dtype, (hipStream_t)stream, "split_rows_relu_bwd",
                           (int64_t)((const char *)fwd_out - (const char *)src), scale);
}
}  // namespace

extern "C" int hapmi_split_rows_relu_bwd(const void *src, const void *fwd_out, void *const *pieces,
                                         const int64_t *lengths, int n_ranks, int64_t outer, int64_t inner_bytes,
                                         int dtype, hapmi_stream_t stream) {
    return split_rows_relu_bwd(src, fwd_out, pieces, lengths, n_ranks, outer, inner_bytes, 1.f, dtype, stream);
}

extern "C" int hapmi_split_rows_relu_bwd_scaled(const void *src, const void *fwd_out, void *const *pieces,
                                                const int64_t *lengths, int n_ranks, int64_t outer, int64_t inner_bytes,
                                                float scale, int dtype, hapmi_stream_t stream) {
    return split_rows_relu_bwd(src, fwd_out, pieces, lengths, n_ranks, outer, inner_bytes, scale, dtype, stream);
}

namespace {
int concat_rows(const void *const *pieces, const int64_t *lengths, int n_ranks, void *dst, int64_t outer, int64_t inner_bytes,
                int act, int dtype, const DropSpec *drop, hapmi_stream_t stream) {
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
            // a piece that was produced at its place in dst (outer = 1: the place is one contiguous range) stays
            const bool in_place = act == HAPMI_ACT_NONE && outer == 1 &&
                                  (const char *)pieces[i] == (const char *)dst + off * inner_bytes;
            if (!in_place)      // index_*: the piece's place in dst, for a dropout that rides on the copy
                list.seg[list.n++] = {(const char *)pieces[i], (char *)dst + off * inner_bytes, outer,
                                      lengths[i] * inner_bytes, lengths[i] * inner_bytes, total * inner_bytes,
                                      off * inner_bytes, total * inner_bytes};
        }
        off += lengths[i];
    }
    return launch_segments(list, act, dtype, (hipStream_t)stream, "concat_rows", 0, 1.f, drop);
}
}  // namespace

extern "C" int hapmi_concat_rows(const void *const *pieces, const int64_t *lengths, int n_ranks, void *dst,
                                 int64_t outer, int64_t inner_bytes, int act, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(act == HAPMI_ACT_NONE || act == HAPMI_ACT_RELU, HAPMI_EINVAL, "concat_rows: only relu can be fused into a concat");
    return concat_rows(pieces, lengths, n_ranks, dst, outer, inner_bytes, act, dtype, nullptr, stream);
}

extern "C" int hapmi_concat_rows_relu_dropout(const void *const *pieces, const int64_t *lengths, int n_ranks, void *dst,
                                              int64_t outer, int64_t inner_bytes, float p, const int64_t *rng_state_dev,
                                              int64_t stream_id, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(p >= 0.f && p <= 1.f && rng_state_dev && ((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EINVAL,
                  "concat_rows_relu_dropout: bad probability %g or RNG state", (double)p);
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "concat_rows_relu_dropout: bad dtype %d", dtype);
    const DropSpec drop = {rng_state_dev, stream_id, p};
    return concat_rows(pieces, lengths, n_ranks, dst, outer, inner_bytes, ACT_RELU_DROP, dtype, &drop, stream);
}

extern "C" int hapmi_relu_dropout_pieces(const void *const *src, void *const *dst, const int64_t *widths, int n_pieces,
                                         int64_t rows, float p, const int64_t *rng_state_dev, int64_t stream_id,
                                         int dtype, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(widths, n_pieces, &total, "relu_dropout_pieces");
    if (rc) return rc;
    HAPMI_REQUIRE(rows >= 0 && src && dst && hapmi_dtype_ok(dtype), HAPMI_EINVAL, "relu_dropout_pieces: bad argument");
    HAPMI_REQUIRE(p >= 0.f && p <= 1.f && rng_state_dev && ((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EINVAL,
                  "relu_dropout_pieces: bad probability %g or RNG state", (double)p);
    const int64_t es = hapmi_elem_size(dtype);
    SegmentList list;
    list.n = 0;
    int64_t off = 0;
    for (int i = 0; i < n_pieces; ++i) {
        if (widths[i] > 0 && rows > 0) {
            HAPMI_REQUIRE(src[i] && dst[i], HAPMI_EINVAL, "relu_dropout_pieces: null pointer");
            list.seg[list.n++] = {(const char *)src[i], (char *)dst[i], rows, widths[i] * es, widths[i] * es, widths[i] * es,
                                  off * es, total * es};
        }
        off += widths[i];
    }
    const DropSpec drop = {rng_state_dev, stream_id, p};
    return launch_segments(list, ACT_RELU_DROP, dtype, (hipStream_t)stream, "relu_dropout_pieces", 0, 1.f, &drop);
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

// bit0 nontemporal loads, bit1 nontemporal store, bit2 two vectors per thread.  Measured on eight contributions of
// 131 MB: plain 5.2 TB/s, streaming loads 5.7-6.0, with two vectors per thread 6.1; streaming stores lose 0.2
constexpr int RED_VARIANT = 5;

struct ReduceOut {
    void *dst;
    int64_t offset, len;       // rows [offset, offset + len) of the sharded dimension
    const void *addend;        // optional, dst's layout: added to the sum last (dst may be the addend itself)
};
struct ReduceOuts {
    int n;
    ReduceOut out[HAPMI_MAX_RANKS];
};

// NT is a template parameter on purpose: a run-time choice between the two kinds of access compiles to the plain one
template <typename T, bool NT> __device__ __forceinline__ Vec16<T> ldv(const T *p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    union { u32x4 u; Vec16<T> v; } x;
    if constexpr (NT) x.u = __builtin_nontemporal_load((const u32x4 *)p);
    else x.u = *(const u32x4 *)p;
    return x.v;
}
template <typename T, bool NT> __device__ __forceinline__ void stv(T *p, const Vec16<T> &v) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    union { u32x4 u; Vec16<T> v; } x;
    x.v = v;
    if constexpr (NT) __builtin_nontemporal_store(x.u, (u32x4 *)p);
    else *(u32x4 *)p = x.u;
}

// blockIdx.y selects the output shard; every output is outs.out[y].len rows of the rank-ordered float32 sum
template <typename T, int NW, int VAR>
__global__ __launch_bounds__(RED_THREADS) void ragged_reduce_kernel(ReduceArgs a, ReduceOuts outs, int64_t outer,
                                                                   int64_t src_len, int64_t inner, int n_dyn) {
    constexpr int EPV = Vec16<T>::N;
    constexpr int U = (VAR & 4) ? 2 : 1;
    constexpr bool NTL = VAR & 1, NTS = VAR & 2;
    const ReduceOut od = outs.out[blockIdx.y];
    T *dst = (T *)od.dst;
    const T *addend = (const T *)od.addend;
    const int64_t offset = od.offset, len = od.len;
    const uint64_t vec_per_row = (uint64_t)(len * inner) / EPV;     // contiguous run per outer index
    const uint64_t total = vec_per_row * (uint64_t)outer;
    const uint64_t step = (uint64_t)gridDim.x * RED_THREADS * U;
    const int nw = NW > 0 ? NW : n_dyn;
    for (uint64_t c0 = (uint64_t)blockIdx.x * RED_THREADS * U + threadIdx.x; c0 < total; c0 += step) {
        uint64_t soff[U], doff[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t c = c0 + (uint64_t)u * RED_THREADS;
            ok[u] = c < total;
            uint64_t o = 0, col = c;
            if (outer > 1) {
                o = c / vec_per_row;
                col = c - o * vec_per_row;
            }
            soff[u] = (o * (uint64_t)src_len + (uint64_t)offset) * (uint64_t)inner + col * EPV;
            doff[u] = (o * (uint64_t)len) * (uint64_t)inner + col * EPV;
        }
        float acc[U][EPV];
        if (NW > 0) {
            Vec16<T> v[U][NW > 0 ? NW : 1];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int w = 0; w < NW; ++w)
                    if (ok[u]) v[u][w] = ldv<T, NTL>((const T *)a.src[w] + soff[u]);
#pragma unroll
            for (int u = 0; u < U; ++u) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[u][e] = v[u][0].get(e);
#pragma unroll
                for (int w = 1; w < NW; ++w)
#pragma unroll
                    for (int e = 0; e < EPV; ++e) acc[u][e] += v[u][w].get(e);
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (!ok[u]) continue;
                Vec16<T> v = ldv<T, NTL>((const T *)a.src[0] + soff[u]);
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[u][e] = v.get(e);
                for (int w = 1; w < nw; ++w) {
                    v = ldv<T, NTL>((const T *)a.src[w] + soff[u]);
#pragma unroll
                    for (int e = 0; e < EPV; ++e) acc[u][e] += v.get(e);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (!ok[u]) continue;
            if (addend) {
                const Vec16<T> g = ldv<T, NTL>(addend + doff[u]);
#pragma unroll
                for (int e = 0; e < EPV; ++e) acc[u][e] += g.get(e);
            }
            Vec16<T> r;
#pragma unroll
            for (int e = 0; e < EPV; ++e) r.set(e, acc[u][e]);
            stv<T, NTS>(dst + doff[u], r);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(RED_THREADS) void ragged_reduce_scalar_kernel(ReduceArgs a, T *dst, const T *addend,
                                                                          int64_t outer, int64_t src_len,
                                                                          int64_t offset, int64_t len, int64_t inner) {
    const uint64_t per = (uint64_t)(len * inner);
    const uint64_t total = per * (uint64_t)outer;
    const uint64_t step = (uint64_t)gridDim.x * RED_THREADS;
    for (uint64_t c = (uint64_t)blockIdx.x * RED_THREADS + threadIdx.x; c < total; c += step) {
        const uint64_t o = c / per, col = c - o * per;
        const uint64_t soff = (o * (uint64_t)src_len + (uint64_t)offset) * (uint64_t)inner + col;
        float acc = ld_f((const T *)a.src[0], soff);
        for (int w = 1; w < a.n; ++w) acc += ld_f((const T *)a.src[w], soff);
        if (addend) acc += ld_f(addend, c);
        st_f(dst, c, acc);
    }
}

template <typename T, int VAR>
void launch_reduce_var(const ReduceArgs &a, const ReduceOuts &outs, int64_t outer, int64_t src_len, int64_t inner,
                       dim3 grid, hipStream_t stream) {
    dim3 block(RED_THREADS);
    switch (a.n) {
#define HAPMI_RED_CASE(NW)                                                                                        \
    case NW:                                                                                                      \
        hipLaunchKernelGGL((ragged_reduce_kernel<T, NW, VAR>), grid, block, 0, stream, a, outs, outer, src_len, inner, \
                           a.n);                                                                                  \
        break;
        HAPMI_RED_CASE(1)
        HAPMI_RED_CASE(2)
        HAPMI_RED_CASE(4)
        HAPMI_RED_CASE(8)
#undef HAPMI_RED_CASE
        default:
            hipLaunchKernelGGL((ragged_reduce_kernel<T, 0, VAR>), grid, block, 0, stream, a, outs, outer, src_len, inner,
                               a.n);
    }
}

template <typename T>
int launch_reduce(const ReduceArgs &a, const ReduceOuts &outs, int64_t outer, int64_t src_len, int64_t inner,
                  hipStream_t stream) {
    constexpr int EPV = Vec16<T>::N;
    bool vec_ok = ((src_len * inner) % EPV == 0);
    int64_t max_len = 0;
    for (int r = 0; r < outs.n; ++r) {
        const ReduceOut &o = outs.out[r];
        vec_ok = vec_ok && ((o.len * inner) % EPV == 0) && ((o.offset * inner) % EPV == 0) && ((uintptr_t)o.dst % 16 == 0) &&
                 ((uintptr_t)o.addend % 16 == 0);
        if (o.len > max_len) max_len = o.len;
    }
    for (int w = 0; w < a.n; ++w) vec_ok = vec_ok && ((uintptr_t)a.src[w] % 16 == 0);
    if (vec_ok) {
        const int u = (RED_VARIANT & 4) ? 2 : 1;
        const int64_t total = outer * (max_len * inner / EPV);
        int64_t gx = hapmi_cdiv(total, (int64_t)RED_THREADS * u);
        const int64_t cap = hapmi_cdiv((int64_t)(256 * 16) << kGridShift, outs.n);
        if (gx > cap) gx = cap;
        if (gx < 1) gx = 1;
        dim3 grid((unsigned)gx, (unsigned)outs.n);
        launch_reduce_var<T, RED_VARIANT>(a, outs, outer, src_len, inner, grid, stream);
    } else {
        for (int r = 0; r < outs.n; ++r) {
            const ReduceOut &o = outs.out[r];
            const int64_t total = outer * o.len * inner;
            if (total == 0) continue;
            int64_t gx = hapmi_cdiv(total, RED_THREADS);
            if (gx > 256 * 16) gx = 256 * 16;
            hipLaunchKernelGGL((ragged_reduce_scalar_kernel<T>), dim3((unsigned)gx), dim3(RED_THREADS), 0, stream, a,
                               (T *)o.dst, (const T *)o.addend, outer, src_len, o.offset, o.len, inner);
        }
    }
    HAPMI_CHECK_LAUNCH("ragged_reduce");
    return HAPMI_OK;
}

}  // namespace

namespace {
int reduce_multi(const void *const *contribs, int n_ranks, void *const *dsts, const void *const *addends,
                 const int64_t *offsets, const int64_t *lengths, int n_outputs, int64_t outer, int64_t src_len,
                 int64_t inner, int dtype, hapmi_stream_t stream);
}

extern "C" int hapmi_ragged_reduce(const void *const *contribs, int n_ranks, void *dst, int64_t outer,
                                   int64_t src_len, int64_t offset, int64_t len, int64_t inner, int dtype,
                                   hapmi_stream_t stream) {
    void *dsts[1] = {dst};
    const int64_t offs[1] = {offset}, lens[1] = {len};
    return reduce_multi(contribs, n_ranks, dsts, nullptr, offs, lens, 1, outer, src_len, inner, dtype, stream);
}

extern "C" int hapmi_ragged_reduce_add(const void *const *contribs, int n_ranks, void *dst, const void *addend,
                                       int64_t outer, int64_t src_len, int64_t offset, int64_t len, int64_t inner,
                                       int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(addend, HAPMI_EINVAL, "ragged_reduce_add: null addend");
    void *dsts[1] = {dst};
    const void *adds[1] = {addend};
    const int64_t offs[1] = {offset}, lens[1] = {len};
    return reduce_multi(contribs, n_ranks, dsts, adds, offs, lens, 1, outer, src_len, inner, dtype, stream);
}

extern "C" int hapmi_ragged_reduce_multi(const void *const *contribs, int n_ranks, void *const *dsts,
                                         const int64_t *offsets, const int64_t *lengths, int n_outputs,
                                         int64_t outer, int64_t src_len, int64_t inner, int dtype,
                                         hapmi_stream_t stream) {
    return reduce_multi(contribs, n_ranks, dsts, nullptr, offsets, lengths, n_outputs, outer, src_len, inner, dtype,
                        stream);
}

namespace {
int reduce_multi(const void *const *contribs, int n_ranks, void *const *dsts, const void *const *addends,
                 const int64_t *offsets, const int64_t *lengths, int n_outputs, int64_t outer, int64_t src_len,
                 int64_t inner, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n_ranks >= 1 && n_ranks <= HAPMI_MAX_RANKS && contribs, HAPMI_EINVAL,
                  "ragged_reduce: n_ranks %d outside 1..%d", n_ranks, HAPMI_MAX_RANKS);
    HAPMI_REQUIRE(n_outputs >= 1 && n_outputs <= HAPMI_MAX_RANKS && dsts && offsets && lengths, HAPMI_EINVAL,
                  "ragged_reduce: n_outputs %d outside 1..%d", n_outputs, HAPMI_MAX_RANKS);
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "ragged_reduce: bad dtype %d", dtype);
    HAPMI_REQUIRE(outer >= 0 && inner > 0 && src_len >= 0, HAPMI_EINVAL, "ragged_reduce: bad shape");
    ReduceOuts outs;
    outs.n = 0;
    for (int r = 0; r < n_outputs; ++r) {
        HAPMI_REQUIRE(lengths[r] >= 0 && offsets[r] >= 0 && offsets[r] + lengths[r] <= src_len, HAPMI_EINVAL,
                      "ragged_reduce: [%lld, %lld) outside 0..%lld", (long long)offsets[r],
                      (long long)(offsets[r] + lengths[r]), (long long)src_len);
        if (lengths[r] == 0 || outer == 0) continue;
        HAPMI_REQUIRE(dsts[r], HAPMI_EINVAL, "ragged_reduce: null destination");
        outs.out[outs.n++] = ReduceOut{dsts[r], offsets[r], lengths[r], addends ? addends[r] : nullptr};
    }
    if (outs.n == 0) return HAPMI_OK;
    ReduceArgs a;
    a.n = n_ranks;
    for (int w = 0; w < n_ranks; ++w) {
        HAPMI_REQUIRE(contribs[w], HAPMI_EINVAL, "ragged_reduce: contribution %d is NULL", w);
        a.src[w] = contribs[w];
    }
    if (dtype == HAPMI_F32) return launch_reduce<float>(a, outs, outer, src_len, inner, (hipStream_t)stream);
    return launch_reduce<bf16_t>(a, outs, outer, src_len, inner, (hipStream_t)stream);
}
}  // namespace

extern "C" int hapmi_pad_rows_multi(const void *const *srcs, void *const *dsts, const int64_t *lengths, int n_shards,
                                    int64_t outer, int64_t padded_len, int64_t inner_bytes, hapmi_stream_t stream) {
    int64_t total;
    int rc = check_lengths(lengths, n_shards, &total, "pad_rows_multi");
    if (rc) return rc;
    HAPMI_REQUIRE(outer >= 0 && inner_bytes > 0 && srcs && dsts, HAPMI_EINVAL, "pad_rows_multi: bad argument");
    SegmentList list;
    list.n = 0;
    for (int i = 0; i < n_shards; ++i) {
        HAPMI_REQUIRE(lengths[i] <= padded_len, HAPMI_EINVAL, "pad_rows_multi: length %lld above padded length %lld",
                      (long long)lengths[i], (long long)padded_len);
        if (lengths[i] > 0 && outer > 0) {
            HAPMI_REQUIRE(srcs[i] && dsts[i], HAPMI_EINVAL, "pad_rows_multi: null pointer");
            list.seg[list.n++] = {(const char *)srcs[i], (char *)dsts[i], outer, lengths[i] * inner_bytes,
                                  lengths[i] * inner_bytes, padded_len * inner_bytes};
        }
    }
    return launch_segments(list, HAPMI_ACT_NONE, 0, (hipStream_t)stream, "pad_rows_multi");
}

