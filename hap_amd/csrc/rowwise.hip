// Row-wise HBM-bound kernels: residual-add + LayerNorm (no affine), softmax with
// additive mask, and log-softmax + NLL with its gradient.  Statistics are float32.
#include "common.h"
#include "dropout.h"

namespace {

constexpr int ROW_WAVES = 4;                 // rows per block, one wave per row
constexpr int ROW_MAXE = 32;                 // most elements per lane -> width <= 2048
// The kernels are instantiated for 8, 16 and 32 elements per lane (widths up to 512, 1024, 2048): the loops over a
// lane's elements are unrolled over registers, so a row of 1024 on the 32-element instance would do twice the
// arithmetic and hold twice the registers.

// A row of `width` elements held across one wave: element e of lane l is
// column (e / EPV) * 64 * EPV + l * EPV + (e % EPV).
template <typename T, int EPV, int MAXE> struct RowRegs {
    float v[MAXE];
    __device__ __forceinline__ static int col(int e, int lane) { return (e / EPV) * 64 * EPV + lane * EPV + (e % EPV); }

    __device__ __forceinline__ void load(const T *row, int width, int lane, float fill) {
#pragma unroll
        for (int g = 0; g < MAXE / EPV; ++g) {
            const int c0 = g * 64 * EPV + lane * EPV;
            if (EPV * sizeof(T) == 16) {
                if (c0 < width) {
                    Vec16<T> x = *(const Vec16<T> *)(row + c0);
#pragma unroll
                    for (int k = 0; k < EPV; ++k) v[g * EPV + k] = x.get(k);
                } else {
#pragma unroll
                    for (int k = 0; k < EPV; ++k) v[g * EPV + k] = fill;
                }
            } else {
#pragma unroll
                for (int k = 0; k < EPV; ++k) v[g * EPV + k] = (c0 + k < width) ? ld_f(row, c0 + k) : fill;
            }
        }
    }
    __device__ __forceinline__ void store(T *row, int width, int lane) const {
#pragma unroll
        for (int g = 0; g < MAXE / EPV; ++g) {
            const int c0 = g * 64 * EPV + lane * EPV;
            if (EPV * sizeof(T) == 16) {
                if (c0 < width) {
                    Vec16<T> x;
#pragma unroll
                    for (int k = 0; k < EPV; ++k) x.set(k, v[g * EPV + k]);
                    *(Vec16<T> *)(row + c0) = x;
                }
            } else {
#pragma unroll
                for (int k = 0; k < EPV; ++k)
                    if (c0 + k < width) st_f(row, c0 + k, v[g * EPV + k]);
            }
        }
    }
};

// F.dropout on a row held in registers: element (row, column c) takes the decision of flat index row * width + c, as
// the elementwise dropout kernel does for the whole tensor.  The vector layouts hold an element pair (even column,
// next column) in one lane and have an even width, so one hash serves the pair; the scalar layout asks per element.
// Kept elements are scaled and, for the 2-byte storage type, rounded as the stored dropout output would be.
template <typename T, int EPV, int MAXE>
__device__ __forceinline__ void drop_row(RowRegs<T, EPV, MAXE> &a, const DropKey &key, int64_t row_first, int width, int lane) {
    auto kept = [&](float v) {
        v *= key.scale;
        return sizeof(T) == 2 ? (float)(bf16_t)v : v;
    };
    if constexpr (EPV % 2 == 0) {
#pragma unroll
        for (int e = 0; e < MAXE; e += 2) {
            const int c = RowRegs<T, EPV, MAXE>::col(e, lane);
            if (c < width) {
                const uint32_t bits = drop_pair_bits(key, (uint64_t)(row_first + c) >> 1);
                a.v[e] = (bits & 0xffffU) >= key.thr ? kept(a.v[e]) : 0.f;
                a.v[e + 1] = (bits >> 16) >= key.thr ? kept(a.v[e + 1]) : 0.f;
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < MAXE; ++e) {
            const int c = RowRegs<T, EPV, MAXE>::col(e, lane);
            if (c < width) a.v[e] = drop_keep(key, (uint64_t)(row_first + c)) ? kept(a.v[e]) : 0.f;
        }
    }
}

// y = LN(x + res), or with DROP y = LN(dropout(x) + res): F.dropout -> operator.add -> F.layer_norm in one pass
template <typename T, int EPV, int MAXE, bool DROP>
__device__ __forceinline__ void add_layernorm_fwd_row(const T *x, const T *res, T *y, float *rstd, int64_t rows, int width,
                                                      float eps, float p, const int64_t *state, int64_t stream_id) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (r >= rows) return;
    RowRegs<T, EPV, MAXE> a;
    a.load(x + r * width, width, lane, 0.f);
    if constexpr (DROP) drop_row(a, drop_key(state[0], state[1], stream_id, p), r * width, width, lane);
    if (res) {
        RowRegs<T, EPV, MAXE> b;
        b.load(res + r * width, width, lane, 0.f);
#pragma unroll
        for (int e = 0; e < MAXE; ++e) {
            a.v[e] += b.v[e];
            // the sum is a tensor of the storage type in the unfused program: round it the same way
            if (sizeof(T) == 2) a.v[e] = (float)(bf16_t)a.v[e];
        }
    }
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) s += a.v[e];
    const float mean = wave_sum(s) / (float)width;
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) {
        const float d = (RowRegs<T, EPV, MAXE>::col(e, lane) < width) ? a.v[e] - mean : 0.f;
        q += d * d;
    }
    const float var = wave_sum(q) / (float)width;
    const float rs = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int e = 0; e < MAXE; ++e) a.v[e] = (a.v[e] - mean) * rs;
    a.store(y + r * width, width, lane);
    if (lane == 0) rstd[r] = rs;
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void add_layernorm_fwd_kernel(const T *x, const T *res, T *y, float *rstd,
                                                                         int64_t rows, int width, float eps) {
    add_layernorm_fwd_row<T, EPV, MAXE, false>(x, res, y, rstd, rows, width, eps, 0.f, nullptr, 0);
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void dropout_add_layernorm_fwd_kernel(const T *x, const T *res, T *y, float *rstd,
                                                                                 int64_t rows, int width, float eps, float p,
                                                                                 const int64_t *state, int64_t stream_id) {
    add_layernorm_fwd_row<T, EPV, MAXE, true>(x, res, y, rstd, rows, width, eps, p, state, stream_id);
}

// dx = rstd * (dy - mean(dy) - y * mean(dy * y)) (+ dx_add); with DROP also dx_drop = dropout's backward of dx (the
// gradient of the operand that went through F.dropout before the add), from the same decisions as forward
template <typename T, int EPV, int MAXE, bool DROP>
__device__ __forceinline__ void layernorm_bwd_row(const T *dy, const T *y, const float *rstd, const T *dx_add, T *dx, T *dx_drop,
                                                  int64_t rows, int width, float p, const int64_t *state, int64_t stream_id) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (r >= rows) return;
    RowRegs<T, EPV, MAXE> g, o;
    g.load(dy + r * width, width, lane, 0.f);
    o.load(y + r * width, width, lane, 0.f);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) {
        s1 += g.v[e];
        s2 += g.v[e] * o.v[e];
    }
    const float c1 = wave_sum(s1) / (float)width, c2 = wave_sum(s2) / (float)width;
    const float rs = rstd[r];
#pragma unroll
    for (int e = 0; e < MAXE; ++e) g.v[e] = rs * (g.v[e] - c1 - o.v[e] * c2);
    if (dx_add) {
        o.load(dx_add + r * width, width, lane, 0.f);
#pragma unroll
        for (int e = 0; e < MAXE; ++e) g.v[e] += o.v[e];
    }
    g.store(dx + r * width, width, lane);
    if constexpr (DROP) {
        if (sizeof(T) == 2) {                                      // dropout's backward reads the stored gradient
#pragma unroll
            for (int e = 0; e < MAXE; ++e) g.v[e] = (float)(bf16_t)g.v[e];
        }
        drop_row(g, drop_key(state[0], state[1], stream_id, p), r * width, width, lane);
        g.store(dx_drop + r * width, width, lane);
    }
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void layernorm_bwd_kernel(const T *dy, const T *y, const float *rstd,
                                                                     const T *dx_add, T *dx, int64_t rows, int width) {
    layernorm_bwd_row<T, EPV, MAXE, false>(dy, y, rstd, dx_add, dx, nullptr, rows, width, 0.f, nullptr, 0);
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void layernorm_bwd_dropout_kernel(const T *dy, const T *y, const float *rstd,
                                                                             const T *dx_add, T *dx, T *dx_drop, int64_t rows,
                                                                             int width, float p, const int64_t *state,
                                                                             int64_t stream_id) {
    layernorm_bwd_row<T, EPV, MAXE, true>(dy, y, rstd, dx_add, dx, dx_drop, rows, width, p, state, stream_id);
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void softmax_fwd_kernel(const T *x, const float *mask, T *p, int64_t rows,
                                                                   int width, int64_t ld, int64_t mask_rows) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (r >= rows) return;
    RowRegs<T, EPV, MAXE> a;
    a.load(x + r * ld, width, lane, -INFINITY);
    if (mask) {
        const float *mrow = mask + (r % mask_rows) * width;
#pragma unroll
        for (int e = 0; e < MAXE; ++e) {
            const int c = RowRegs<T, EPV, MAXE>::col(e, lane);
            if (c < width) a.v[e] += mrow[c];
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) m = fmaxf(m, a.v[e]);
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) {
        a.v[e] = __expf(a.v[e] - m);
        s += a.v[e];
    }
    const float inv = 1.0f / wave_sum(s);
#pragma unroll
    for (int e = 0; e < MAXE; ++e) a.v[e] *= inv;
    a.store(p + r * ld, width, lane);
}

template <typename T, int EPV, int MAXE>
__global__ __launch_bounds__(ROW_WAVES * 64) void softmax_bwd_kernel(const T *dp, const T *p, T *ds, int64_t rows,
                                                                   int width, int64_t ld) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + (threadIdx.x >> 6);
    if (r >= rows) return;
    RowRegs<T, EPV, MAXE> g, o;
    g.load(dp + r * ld, width, lane, 0.f);
    o.load(p + r * ld, width, lane, 0.f);
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < MAXE; ++e) s += g.v[e] * o.v[e];
    s = wave_sum(s);
#pragma unroll
    for (int e = 0; e < MAXE; ++e) g.v[e] = o.v[e] * (g.v[e] - s);
    g.store(ds + r * ld, width, lane);
}

template <typename T> int row_epv(const void *const *ptrs, int n, int64_t width) {
    constexpr int EPV = 16 / sizeof(T);
    bool ok = width % EPV == 0;
    for (int i = 0; i < n; ++i) ok = ok && (((uintptr_t)ptrs[i]) % 16 == 0);
    return ok ? EPV : 1;
}

#define HAPMI_ROW_LAUNCH(KERNEL, T, EPV_, MAXE_, grid, stream, ...) \
    hipLaunchKernelGGL((KERNEL<T, EPV_, MAXE_>), grid, dim3(ROW_WAVES * 64), 0, stream, __VA_ARGS__)

// `width` picks the instance with the fewest elements per lane that holds a row
#define HAPMI_ROW_DISPATCH(KERNEL, T, epv, width, grid, stream, ...)                                        \
    do {                                                                                                    \
        constexpr int V_ = 16 / sizeof(T);                                                                  \
        const int me_ = (width) <= 8 * 64 ? 8 : ((width) <= 16 * 64 ? 16 : 32);                             \
        if ((epv) == 1) {                                                                                   \
            if (me_ == 8) HAPMI_ROW_LAUNCH(KERNEL, T, 1, 8, grid, stream, __VA_ARGS__);                     \
            else if (me_ == 16) HAPMI_ROW_LAUNCH(KERNEL, T, 1, 16, grid, stream, __VA_ARGS__);              \
            else HAPMI_ROW_LAUNCH(KERNEL, T, 1, 32, grid, stream, __VA_ARGS__);                             \
        } else {                                                                                            \
            if (me_ == 8) HAPMI_ROW_LAUNCH(KERNEL, T, V_, 8, grid, stream, __VA_ARGS__);                    \
            else if (me_ == 16) HAPMI_ROW_LAUNCH(KERNEL, T, V_, 16, grid, stream, __VA_ARGS__);             \
            else HAPMI_ROW_LAUNCH(KERNEL, T, V_, 32, grid, stream, __VA_ARGS__);                            \
        }                                                                                                   \
    } while (0)

int check_rows(const char *name, int64_t rows, int64_t width, int dtype) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "%s: bad dtype %d", name, dtype);
    HAPMI_REQUIRE(rows >= 0 && width >= 1, HAPMI_EINVAL, "%s: bad shape [%lld, %lld]", name, (long long)rows,
                  (long long)width);
    const int64_t maxw = (int64_t)ROW_MAXE * 64;
    HAPMI_REQUIRE(width <= maxw, HAPMI_ELIMIT, "%s: width %lld above the limit %lld", name, (long long)width,
                  (long long)maxw);
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_add_layernorm_fwd(const void *x, const void *res, void *y, float *rstd, int64_t rows,
                                       int64_t width, float eps, int dtype, hapmi_stream_t stream) {
    int rc = check_rows("add_layernorm_fwd", rows, width, dtype);
    if (rc) return rc;
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(x && y && rstd, HAPMI_EINVAL, "add_layernorm_fwd: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[3] = {x, y, res};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(add_layernorm_fwd_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)x,
                           (const float *)res, (float *)y, rstd, rows, (int)width, eps);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(add_layernorm_fwd_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)x,
                           (const bf16_t *)res, (bf16_t *)y, rstd, rows, (int)width, eps);
    }
    HAPMI_CHECK_LAUNCH("add_layernorm_fwd");
    return HAPMI_OK;
}

extern "C" int hapmi_layernorm_bwd(const void *dy, const void *y, const float *rstd, const void *dx_add, void *dx,
                                   int64_t rows, int64_t width, int dtype, hapmi_stream_t stream) {
    int rc = check_rows("layernorm_bwd", rows, width, dtype);
    if (rc) return rc;
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(dy && y && rstd && dx, HAPMI_EINVAL, "layernorm_bwd: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[4] = {dy, y, dx, dx_add};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 4, width);
        HAPMI_ROW_DISPATCH(layernorm_bwd_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)dy,
                           (const float *)y, rstd, (const float *)dx_add, (float *)dx, rows, (int)width);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 4, width);
        HAPMI_ROW_DISPATCH(layernorm_bwd_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)dy,
                           (const bf16_t *)y, rstd, (const bf16_t *)dx_add, (bf16_t *)dx, rows, (int)width);
    }
    HAPMI_CHECK_LAUNCH("layernorm_bwd");
    return HAPMI_OK;
}

extern "C" int hapmi_dropout_add_layernorm_fwd(const void *x, const void *res, void *y, float *rstd, int64_t rows,
                                               int64_t width, float eps, float p, const int64_t *rng_state_dev,
                                               int64_t stream_id, int dtype, hapmi_stream_t stream) {
    int rc = check_rows("dropout_add_layernorm_fwd", rows, width, dtype);
    if (rc) return rc;
    HAPMI_REQUIRE(p >= 0.f && p <= 1.f, HAPMI_EINVAL, "dropout_add_layernorm_fwd: bad probability %g", (double)p);
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(x && y && rstd && rng_state_dev, HAPMI_EINVAL, "dropout_add_layernorm_fwd: null pointer");
    HAPMI_REQUIRE(((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EALIGN, "dropout_add_layernorm_fwd: misaligned RNG state");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[3] = {x, y, res};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(dropout_add_layernorm_fwd_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)x,
                           (const float *)res, (float *)y, rstd, rows, (int)width, eps, p, rng_state_dev, stream_id);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(dropout_add_layernorm_fwd_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)x,
                           (const bf16_t *)res, (bf16_t *)y, rstd, rows, (int)width, eps, p, rng_state_dev, stream_id);
    }
    HAPMI_CHECK_LAUNCH("dropout_add_layernorm_fwd");
    return HAPMI_OK;
}

extern "C" int hapmi_layernorm_bwd_dropout(const void *dy, const void *y, const float *rstd, const void *dx_add, void *dx,
                                           void *dx_drop, int64_t rows, int64_t width, float p,
                                           const int64_t *rng_state_dev, int64_t stream_id, int dtype,
                                           hapmi_stream_t stream) {
    int rc = check_rows("layernorm_bwd_dropout", rows, width, dtype);
    if (rc) return rc;
    HAPMI_REQUIRE(p >= 0.f && p <= 1.f, HAPMI_EINVAL, "layernorm_bwd_dropout: bad probability %g", (double)p);
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(dy && y && rstd && dx && dx_drop && rng_state_dev, HAPMI_EINVAL, "layernorm_bwd_dropout: null pointer");
    HAPMI_REQUIRE(((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EALIGN, "layernorm_bwd_dropout: misaligned RNG state");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[5] = {dy, y, dx, dx_add, dx_drop};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 5, width);
        HAPMI_ROW_DISPATCH(layernorm_bwd_dropout_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)dy,
                           (const float *)y, rstd, (const float *)dx_add, (float *)dx, (float *)dx_drop, rows, (int)width, p,
                           rng_state_dev, stream_id);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 5, width);
        HAPMI_ROW_DISPATCH(layernorm_bwd_dropout_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)dy,
                           (const bf16_t *)y, rstd, (const bf16_t *)dx_add, (bf16_t *)dx, (bf16_t *)dx_drop, rows, (int)width, p,
                           rng_state_dev, stream_id);
    }
    HAPMI_CHECK_LAUNCH("layernorm_bwd_dropout");
    return HAPMI_OK;
}

extern "C" int hapmi_softmax_fwd(const void *x, const float *mask, void *p, int64_t rows, int64_t width, int64_t ld,
                                 int64_t mask_rows, int dtype, hapmi_stream_t stream) {
    int rc = check_rows("softmax_fwd", rows, width, dtype);
    if (rc) return rc;
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(x && p, HAPMI_EINVAL, "softmax_fwd: null pointer");
    HAPMI_REQUIRE(!mask || mask_rows >= 1, HAPMI_EINVAL, "softmax_fwd: mask_rows must be >= 1");
    HAPMI_REQUIRE(ld >= width, HAPMI_EINVAL, "softmax_fwd: ld below width");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[3] = {x, p, (const void *)(uintptr_t)(ld * hapmi_elem_size(dtype))};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(softmax_fwd_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)x, mask,
                           (float *)p, rows, (int)width, ld, mask_rows);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 3, width);
        HAPMI_ROW_DISPATCH(softmax_fwd_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)x, mask,
                           (bf16_t *)p, rows, (int)width, ld, mask_rows);
    }
    HAPMI_CHECK_LAUNCH("softmax_fwd");
    return HAPMI_OK;
}

extern "C" int hapmi_softmax_bwd(const void *dp, const void *p, void *ds, int64_t rows, int64_t width, int64_t ld,
                                 int dtype, hapmi_stream_t stream) {
    int rc = check_rows("softmax_bwd", rows, width, dtype);
    if (rc) return rc;
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(dp && p && ds, HAPMI_EINVAL, "softmax_bwd: null pointer");
    HAPMI_REQUIRE(ld >= width, HAPMI_EINVAL, "softmax_bwd: ld below width");
    dim3 grid((unsigned)hapmi_cdiv(rows, ROW_WAVES));
    const void *ptrs[4] = {dp, p, ds, (const void *)(uintptr_t)(ld * hapmi_elem_size(dtype))};
    if (dtype == HAPMI_F32) {
        int epv = row_epv<float>(ptrs, 4, width);
        HAPMI_ROW_DISPATCH(softmax_bwd_kernel, float, epv, width, grid, (hipStream_t)stream, (const float *)dp,
                           (const float *)p, (float *)ds, rows, (int)width, ld);
    } else {
        int epv = row_epv<bf16_t>(ptrs, 4, width);
        HAPMI_ROW_DISPATCH(softmax_bwd_kernel, bf16_t, epv, width, grid, (hipStream_t)stream, (const bf16_t *)dp,
                           (const bf16_t *)p, (bf16_t *)ds, rows, (int)width, ld);
    }
    HAPMI_CHECK_LAUNCH("softmax_bwd");
    return HAPMI_OK;
}

// ---------------------------------------------------------------------------
// log-softmax + NLL(sum) + gradient, one block per row of the logits
// ---------------------------------------------------------------------------
namespace {

constexpr int NLL_THREADS = 512;

template <typename T, int EPV> struct alignas(EPV * sizeof(T)) SmallVec {
    T e[EPV];
};

template <typename T, int EPV>
__global__ __launch_bounds__(NLL_THREADS) void logsoftmax_nll_kernel(const T *logits, const int64_t *targets,
                                                                   int64_t ignore_index, float *row_loss, T *dlogits,
                                                                   int64_t width, int64_t ld, float grad_scale) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    const T *row = logits + r * ld;
    typedef SmallVec<T, EPV> V;
    const int64_t nvec = width / EPV;           // tail elements are handled after the vector body
    // pass 1: running maximum and sum of exponentials per thread
    float m = -INFINITY, s = 0.f;
    for (int64_t i = threadIdx.x; i < nvec; i += NLL_THREADS) {
        V v = ((const V *)row)[i];
        float f[EPV], vm = -INFINITY;
#pragma unroll
        for (int k = 0; k < EPV; ++k) {
            f[k] = (float)v.e[k];
            vm = fmaxf(vm, f[k]);
        }
        if (vm > m) {
            s *= __expf(m - vm);
            m = vm;
        }
#pragma unroll
        for (int k = 0; k < EPV; ++k) s += __expf(f[k] - m);
    }
    for (int64_t c = nvec * EPV + threadIdx.x; c < width; c += NLL_THREADS) {
        const float f = (float)row[c];
        if (f > m) {
            s *= __expf(m - f);
            m = f;
        }
        s += __expf(f - m);
    }
    const float bm = block_max(m, red);
    s = (m == -INFINITY) ? 0.f : s * __expf(m - bm);
    const float bs = block_sum(s, red);
    const float lse = bm + __logf(bs);
    const int64_t t = targets[r];
    const bool in_range = t >= 0 && t < width;       // an out-of-range class poisons the loss instead of faulting
    const bool counted = t != ignore_index && in_range;
    if (threadIdx.x == 0) row_loss[r] = counted ? lse - (float)row[t] : ((t != ignore_index) ? NAN : 0.f);
    if (!dlogits) return;
    __syncthreads();                                  // dlogits may alias logits: row[t] is read before any write
    T *drow = dlogits + r * ld;
    const float inv = 1.0f / bs;
    for (int64_t i = threadIdx.x; i < nvec; i += NLL_THREADS) {
        V v = ((const V *)row)[i], o;
#pragma unroll
        for (int k = 0; k < EPV; ++k) {
            float g = 0.f;
            if (counted) {
                g = __expf((float)v.e[k] - bm) * inv;
                if (i * EPV + k == t) g -= 1.0f;
                g *= grad_scale;
            }
            o.e[k] = (T)g;
        }
        ((V *)drow)[i] = o;
    }
    for (int64_t c = nvec * EPV + threadIdx.x; c < width; c += NLL_THREADS) {
        float g = 0.f;
        if (counted) {
            g = __expf((float)row[c] - bm) * inv;
            if (c == t) g -= 1.0f;
            g *= grad_scale;
        }
        drow[c] = (T)g;
    }
}

__global__ __launch_bounds__(1024) void sum_f32_kernel(const float *x, int64_t n, float *out) {
    __shared__ float red[16];
    // fixed association: thread-strided partials, then wave tree, then wave order
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) s += x[i];
    s = block_sum(s, red);
    if (threadIdx.x == 0) out[0] = s;
}

}  // namespace

extern "C" int hapmi_logsoftmax_nll(const void *logits, const int64_t *targets, int64_t ignore_index,
                                    float *row_loss, void *dlogits, int64_t rows, int64_t width, int64_t ld,
                                    float grad_scale, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype), HAPMI_EINVAL, "logsoftmax_nll: bad dtype %d", dtype);
    HAPMI_REQUIRE(rows >= 0 && width >= 1, HAPMI_EINVAL, "logsoftmax_nll: bad shape");
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(logits && targets && row_loss, HAPMI_EINVAL, "logsoftmax_nll: null pointer");
    const int64_t esz = hapmi_elem_size(dtype);
    HAPMI_REQUIRE(ld >= width, HAPMI_EINVAL, "logsoftmax_nll: ld below width");
    uint64_t bits = (uint64_t)(uintptr_t)logits | (uint64_t)(uintptr_t)dlogits | (uint64_t)(ld * esz);
    int vb = 16;
    while (vb > esz && (bits & (uint64_t)(vb - 1))) vb >>= 1;
    const int epv = (int)(vb / esz);
    dim3 grid((unsigned)rows), block(NLL_THREADS);
    hipStream_t st = (hipStream_t)stream;
#define HAPMI_NLL(T, E)                                                                                          \
    hipLaunchKernelGGL((logsoftmax_nll_kernel<T, E>), grid, block, 0, st, (const T *)logits, targets, ignore_index, \
                       row_loss, (T *)dlogits, width, ld, grad_scale)
    if (dtype == HAPMI_F32) {
        if (epv == 4) HAPMI_NLL(float, 4);
        else if (epv == 2) HAPMI_NLL(float, 2);
        else HAPMI_NLL(float, 1);
    } else {
        if (epv == 8) HAPMI_NLL(bf16_t, 8);
        else if (epv == 4) HAPMI_NLL(bf16_t, 4);
        else if (epv == 2) HAPMI_NLL(bf16_t, 2);
        else HAPMI_NLL(bf16_t, 1);
    }
#undef HAPMI_NLL
    HAPMI_CHECK_LAUNCH("logsoftmax_nll");
    return HAPMI_OK;
}

extern "C" int hapmi_sum_f32(const float *x, int64_t n, float *out, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0 && out && (x || n == 0), HAPMI_EINVAL, "sum_f32: bad argument");
    hipLaunchKernelGGL(sum_f32_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, x, n, out);
    HAPMI_CHECK_LAUNCH("sum_f32");
    return HAPMI_OK;
}
