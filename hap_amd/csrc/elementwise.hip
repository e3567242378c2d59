// Elementwise, gather/scatter and optimizer kernels (all HBM-bound).
#include "common.h"
#include <mutex>

namespace {

constexpr int EW_THREADS = 256;

inline unsigned ew_grid(int64_t n_items) {
    int64_t g = hapmi_cdiv(n_items, EW_THREADS);
    if (g > 256 * 32) g = 256 * 32;
    if (g < 1) g = 1;
    return (unsigned)g;
}

// Optimizer updates stream four to eight arrays at once; measured on 300 M parameters they run fastest with one
// 16-byte vector per thread (no grid-stride loop until the grid limit) and streaming (non-temporal) accesses:
// 6.0 TB/s against 4.4 TB/s for a capped grid of looping blocks with cached accesses.
inline unsigned stream_grid(int64_t n_items) {
    int64_t g = hapmi_cdiv(n_items, EW_THREADS);
    if (g > 0x7fffffffLL) g = 0x7fffffffLL;
    if (g < 1) g = 1;
    return (unsigned)g;
}
template <typename V>
__device__ __forceinline__ V ld_stream(const V *p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void st_stream(V v, V *p) { __builtin_nontemporal_store(v, p); }

__device__ __forceinline__ float gelu_f(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752f)); }
__device__ __forceinline__ float gelu_grad_f(float x) {
    const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752f));
    const float pdf = 0.3989422804014327f * __expf(-0.5f * x * x);
    return cdf + x * pdf;
}

// Generic vectorised map over n elements: F(float...)->float, inputs/outputs of type T.
template <typename T, typename F> __global__ __launch_bounds__(EW_THREADS) void map1_kernel(const T *a, T *o, int64_t n, F f) {
    constexpr int EPV = Vec16<T>::N;
    const int64_t nv = n / EPV, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < nv; i += step) {
        Vec16<T> x = ((const Vec16<T> *)a)[i], r;
#pragma unroll
        for (int k = 0; k < EPV; ++k) r.set(k, f(x.get(k)));
        ((Vec16<T> *)o)[i] = r;
    }
    for (int64_t i = nv * EPV + (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step) st_f(o, i, f(ld_f(a, i)));
}
template <typename T, typename F>
__global__ __launch_bounds__(EW_THREADS) void map2_kernel(const T *a, const T *b, T *o, int64_t n, F f) {
    constexpr int EPV = Vec16<T>::N;
    const int64_t nv = n / EPV, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < nv; i += step) {
        Vec16<T> x = ((const Vec16<T> *)a)[i], y = ((const Vec16<T> *)b)[i], r;
#pragma unroll
        for (int k = 0; k < EPV; ++k) r.set(k, f(x.get(k), y.get(k)));
        ((Vec16<T> *)o)[i] = r;
    }
    for (int64_t i = nv * EPV + (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step)
        st_f(o, i, f(ld_f(a, i), ld_f(b, i)));
}

struct FRelu { __device__ float operator()(float x) const { return x > 0.f ? x : 0.f; } };
struct FGelu { __device__ float operator()(float x) const { return gelu_f(x); } };
struct FReluBwd { __device__ float operator()(float dy, float y) const { return y > 0.f ? dy : 0.f; } };
struct FGeluBwd { __device__ float operator()(float dy, float x) const { return dy * gelu_grad_f(x); } };
struct FSigmoid { __device__ float operator()(float x) const { return 1.0f / (1.0f + __expf(-x)); } };
struct FSigmoidBwd { __device__ float operator()(float dy, float y) const { return dy * y * (1.0f - y); } };
struct FAdd { __device__ float operator()(float a, float b) const { return a + b; } };
struct FConst {
    float v;
    __device__ float operator()(float) const { return v; }
};
struct FScale {
    float s;
    __device__ float operator()(float a) const { return a * s; }
};

bool aligned16(const void *p) { return ((uintptr_t)p % 16) == 0; }

template <typename F> int run_map1(const void *a, void *o, int64_t n, int dtype, F f, hipStream_t st, const char *name) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && n >= 0, HAPMI_EINVAL, "%s: bad argument", name);
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(a && o, HAPMI_EINVAL, "%s: null pointer", name);
    HAPMI_REQUIRE(aligned16(a) && aligned16(o), HAPMI_EALIGN, "%s: pointers must be 16-byte aligned", name);
    const int epv = dtype == HAPMI_F32 ? 4 : 8;
    dim3 grid(ew_grid(hapmi_cdiv(n, epv)));
    if (dtype == HAPMI_F32) hipLaunchKernelGGL((map1_kernel<float, F>), grid, dim3(EW_THREADS), 0, st, (const float *)a, (float *)o, n, f);
    else hipLaunchKernelGGL((map1_kernel<bf16_t, F>), grid, dim3(EW_THREADS), 0, st, (const bf16_t *)a, (bf16_t *)o, n, f);
    HAPMI_CHECK_LAUNCH(name);
    return HAPMI_OK;
}
template <typename F>
int run_map2(const void *a, const void *b, void *o, int64_t n, int dtype, F f, hipStream_t st, const char *name) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && n >= 0, HAPMI_EINVAL, "%s: bad argument", name);
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(a && b && o, HAPMI_EINVAL, "%s: null pointer", name);
    HAPMI_REQUIRE(aligned16(a) && aligned16(b) && aligned16(o), HAPMI_EALIGN, "%s: pointers must be 16-byte aligned", name);
    const int epv = dtype == HAPMI_F32 ? 4 : 8;
    dim3 grid(ew_grid(hapmi_cdiv(n, epv)));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((map2_kernel<float, F>), grid, dim3(EW_THREADS), 0, st, (const float *)a, (const float *)b, (float *)o, n, f);
    else
        hipLaunchKernelGGL((map2_kernel<bf16_t, F>), grid, dim3(EW_THREADS), 0, st, (const bf16_t *)a, (const bf16_t *)b, (bf16_t *)o, n, f);
    HAPMI_CHECK_LAUNCH(name);
    return HAPMI_OK;
}

}  // namespace

extern "C" int hapmi_act_fwd(const void *x, void *y, int64_t n, int act, int dtype, hapmi_stream_t stream) {
    if (act == HAPMI_ACT_RELU) return run_map1(x, y, n, dtype, FRelu(), (hipStream_t)stream, "act_fwd(relu)");
    if (act == HAPMI_ACT_GELU) return run_map1(x, y, n, dtype, FGelu(), (hipStream_t)stream, "act_fwd(gelu)");
    if (act == HAPMI_ACT_SIGMOID) return run_map1(x, y, n, dtype, FSigmoid(), (hipStream_t)stream, "act_fwd(sigmoid)");
    return hapmi_set_error(HAPMI_EINVAL, "act_fwd: unknown activation %d", act);
}
extern "C" int hapmi_act_bwd(const void *dy, const void *ref, void *dx, int64_t n, int act, int dtype,
                             hapmi_stream_t stream) {
    if (act == HAPMI_ACT_RELU) return run_map2(dy, ref, dx, n, dtype, FReluBwd(), (hipStream_t)stream, "act_bwd(relu)");
    if (act == HAPMI_ACT_GELU) return run_map2(dy, ref, dx, n, dtype, FGeluBwd(), (hipStream_t)stream, "act_bwd(gelu)");
    if (act == HAPMI_ACT_SIGMOID) return run_map2(dy, ref, dx, n, dtype, FSigmoidBwd(), (hipStream_t)stream, "act_bwd(sigmoid)");
    return hapmi_set_error(HAPMI_EINVAL, "act_bwd: unknown activation %d", act);
}
extern "C" int hapmi_add(const void *a, const void *b, void *out, int64_t n, int dtype, hapmi_stream_t stream) {
    return run_map2(a, b, out, n, dtype, FAdd(), (hipStream_t)stream, "add");
}
extern "C" int hapmi_fill_value(void *out, float value, int64_t n, int dtype, hapmi_stream_t stream) {
    return run_map1(out, out, n, dtype, FConst{value}, (hipStream_t)stream, "fill_value");
}
extern "C" int hapmi_scale(const void *a, float s, void *out, int64_t n, int dtype, hapmi_stream_t stream) {
    return run_map1(a, out, n, dtype, FScale{s}, (hipStream_t)stream, "scale");
}

// ---------------------------------------------------------------------------
namespace {

template <typename T>
__global__ __launch_bounds__(EW_THREADS) void add_bcast_rows_kernel(const T *a, const T *b, T *o, int64_t rows,
                                                                   int64_t b_rows, int64_t width) {
    const int64_t n = rows * width, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step) {
        const int64_t r = i / width, c = i - r * width;
        st_f(o, i, ld_f(a, i) + ld_f(b, (r % b_rows) * width + c));
    }
}

// column sums of x[M, N] (row stride ldx): each block owns 64 columns and a slab of `rows_per_slab` rows and writes
// its sum to dst[slab][N] (dst = the output itself when there is one slab, else the workspace, whose slabs
// colsum_final_kernel adds in order): no atomics, so the same call gives the same bits every time
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(const T *x, float *dst, int64_t M, int64_t N, int64_t ldx,
                                                   int64_t rows_per_slab, int add_to_dst) {
    __shared__ float part[4][64];
    const int c = threadIdx.x & 63, rg = threadIdx.x >> 6;
    const int64_t col = (int64_t)blockIdx.x * 64 + c;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_slab;
    const int64_t r1 = r0 + rows_per_slab < M ? r0 + rows_per_slab : M;
    float s = 0.f;
    if (col < N)
        for (int64_t r = r0 + rg; r < r1; r += 4) s += ld_f(x, r * ldx + col);
    part[rg][c] = s;
    __syncthreads();
    if (rg == 0 && col < N) {
        const float t = part[0][c] + part[1][c] + part[2][c] + part[3][c];
        float *o = dst + (int64_t)blockIdx.y * N + col;
        *o = add_to_dst ? *o + t : t;
    }
}

// vectorised form: 32 column groups of one 16-byte vector x 8 row groups per block
template <typename T>
__global__ __launch_bounds__(256) void colsum_vec_kernel(const T *x, float *dst, int64_t M, int64_t N, int64_t ldx,
                                                       int64_t rows_per_slab, int add_to_dst) {
    constexpr int EPV = Vec16<T>::N;
    __shared__ float part[8][32 * EPV + 1];
    const int cg = threadIdx.x & 31, rg = threadIdx.x >> 5;
    const int64_t col = ((int64_t)blockIdx.x * 32 + cg) * EPV;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_slab;
    const int64_t r1 = r0 + rows_per_slab < M ? r0 + rows_per_slab : M;
    float s[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) s[e] = 0.f;
    if (col < N)                                              // N is a multiple of EPV on this path
        for (int64_t r = r0 + rg; r < r1; r += 8) {
            const Vec16<T> v = *(const Vec16<T> *)(x + r * ldx + col);
#pragma unroll
            for (int e = 0; e < EPV; ++e) s[e] += v.get(e);
        }
#pragma unroll
    for (int e = 0; e < EPV; ++e) part[rg][cg * EPV + e] = s[e];
    __syncthreads();
    for (int c = threadIdx.x; c < 32 * EPV; c += 256) {
        const int64_t gc = (int64_t)blockIdx.x * 32 * EPV + c;
        if (gc < N) {
            float t = 0.f;
#pragma unroll
            for (int g = 0; g < 8; ++g) t += part[g][c];
            float *o = dst + (int64_t)blockIdx.y * N + gc;
            *o = add_to_dst ? *o + t : t;
        }
    }
}

__global__ __launch_bounds__(256) void colsum_final_kernel(const float *slabs, float *out, int64_t N, int64_t n_slabs,
                                                         int accumulate) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= N) return;
    float s = accumulate ? out[c] : 0.f;
    for (int64_t i = 0; i < n_slabs; ++i) s += slabs[i * N + c];
    out[c] = s;
}

template <typename TS, typename TD>
__global__ __launch_bounds__(EW_THREADS) void cast_kernel(const TS *s, TD *d, int64_t n) {
    const int64_t step = (int64_t)gridDim.x * EW_THREADS * 4;
    for (int64_t i = ((int64_t)blockIdx.x * EW_THREADS + threadIdx.x) * 4; i < n; i += step) {
#pragma unroll
        for (int k = 0; k < 4; ++k)
            if (i + k < n) st_f(d, i + k, ld_f(s, i + k));
    }
}

__global__ __launch_bounds__(EW_THREADS) void zero_f32_kernel(float *p, int64_t n) {
    const int64_t step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step) p[i] = 0.f;
}

__global__ __launch_bounds__(EW_THREADS) void fill_zero_kernel(uint32_t *p, int64_t n_words) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int64_t nv = n_words / 4, step = (int64_t)gridDim.x * EW_THREADS;
    const u32x4 z = {0, 0, 0, 0};
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < nv; i += step) ((u32x4 *)p)[i] = z;
    for (int64_t i = nv * 4 + (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n_words; i += step) p[i] = 0;
}

}  // namespace

extern "C" int hapmi_add_bcast_rows(const void *a, const void *b, void *out, int64_t rows, int64_t b_rows,
                                    int64_t width, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && rows >= 0 && b_rows >= 1 && width >= 1, HAPMI_EINVAL, "add_bcast_rows: bad argument");
    if (rows == 0) return HAPMI_OK;
    HAPMI_REQUIRE(a && b && out, HAPMI_EINVAL, "add_bcast_rows: null pointer");
    dim3 grid(ew_grid(rows * width));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((add_bcast_rows_kernel<float>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, (const float *)a, (const float *)b, (float *)out, rows, b_rows, width);
    else
        hipLaunchKernelGGL((add_bcast_rows_kernel<bf16_t>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t *)a, (const bf16_t *)b, (bf16_t *)out, rows, b_rows, width);
    HAPMI_CHECK_LAUNCH("add_bcast_rows");
    return HAPMI_OK;
}

extern "C" int hapmi_fill_zero(void *p, int64_t bytes, hapmi_stream_t stream) {
    HAPMI_REQUIRE(bytes >= 0 && bytes % 4 == 0, HAPMI_EINVAL, "fill_zero: byte count must be a multiple of 4");
    if (bytes == 0) return HAPMI_OK;
    HAPMI_REQUIRE(p && aligned16(p), HAPMI_EALIGN, "fill_zero: pointer must be 16-byte aligned");
    hipLaunchKernelGGL(fill_zero_kernel, dim3(ew_grid(bytes / 16 + 1)), dim3(EW_THREADS), 0, (hipStream_t)stream, (uint32_t *)p, bytes / 4);
    HAPMI_CHECK_LAUNCH("fill_zero");
    return HAPMI_OK;
}

extern "C" int hapmi_colsum(const void *x, float *out, int64_t M, int64_t N, int64_t ldx, int accumulate, int dtype,
                            float *workspace, int64_t workspace_elems, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && M >= 0 && N >= 0 && ldx >= N && workspace_elems >= 0, HAPMI_EINVAL, "colsum: bad argument");
    if (N == 0) return HAPMI_OK;
    HAPMI_REQUIRE(out && (x || M == 0), HAPMI_EINVAL, "colsum: null pointer");
    // out may be 4-byte aligned only (a view into a flat gradient buffer)
    HAPMI_REQUIRE(((uintptr_t)out % 4) == 0 && ((uintptr_t)workspace % 4) == 0, HAPMI_EALIGN, "colsum: out / workspace must be 4-byte aligned");
    if (M == 0) {
        if (!accumulate) hipLaunchKernelGGL(zero_f32_kernel, dim3(ew_grid(N)), dim3(EW_THREADS), 0, (hipStream_t)stream, out, N);
        return HAPMI_OK;
    }
    // slabs of at least 128 rows, as many as the workspace holds ([slab][N]); one slab writes the result itself
    int64_t n_slabs = hapmi_cdiv(M, 128);
    if (!workspace || n_slabs * N > workspace_elems) n_slabs = workspace ? workspace_elems / N : 1;
    if (n_slabs < 2) n_slabs = 1;
    if (n_slabs > 65535) n_slabs = 65535;
    const int64_t rows_per_slab = hapmi_cdiv(M, n_slabs);
    n_slabs = hapmi_cdiv(M, rows_per_slab);
    float *dst = n_slabs > 1 ? workspace : out;
    const int add = n_slabs > 1 ? 0 : accumulate;
    const int64_t epv = dtype == HAPMI_F32 ? 4 : 8;
    if (aligned16(x) && ldx % epv == 0 && N % epv == 0) {
        dim3 vgrid((unsigned)hapmi_cdiv(N, 32 * epv), (unsigned)n_slabs);
        if (dtype == HAPMI_F32) hipLaunchKernelGGL((colsum_vec_kernel<float>), vgrid, dim3(256), 0, (hipStream_t)stream, (const float *)x, dst, M, N, ldx, rows_per_slab, add);
        else hipLaunchKernelGGL((colsum_vec_kernel<bf16_t>), vgrid, dim3(256), 0, (hipStream_t)stream, (const bf16_t *)x, dst, M, N, ldx, rows_per_slab, add);
    } else {
        dim3 grid((unsigned)hapmi_cdiv(N, 64), (unsigned)n_slabs);
        if (dtype == HAPMI_F32) hipLaunchKernelGGL((colsum_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, (const float *)x, dst, M, N, ldx, rows_per_slab, add);
        else hipLaunchKernelGGL((colsum_kernel<bf16_t>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16_t *)x, dst, M, N, ldx, rows_per_slab, add);
    }
    if (n_slabs > 1)
        hipLaunchKernelGGL(colsum_final_kernel, dim3((unsigned)hapmi_cdiv(N, 256)), dim3(256), 0, (hipStream_t)stream,
                           (const float *)workspace, out, N, n_slabs, accumulate);
    HAPMI_CHECK_LAUNCH("colsum");
    return HAPMI_OK;
}

extern "C" int hapmi_cast(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(src_dtype) && hapmi_dtype_ok(dst_dtype) && n >= 0, HAPMI_EINVAL, "cast: bad argument");
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(src && dst, HAPMI_EINVAL, "cast: null pointer");
    dim3 grid(ew_grid(hapmi_cdiv(n, 4))), block(EW_THREADS);
    hipStream_t st = (hipStream_t)stream;
    if (src_dtype == HAPMI_F32 && dst_dtype == HAPMI_BF16) hipLaunchKernelGGL((cast_kernel<float, bf16_t>), grid, block, 0, st, (const float *)src, (bf16_t *)dst, n);
    else if (src_dtype == HAPMI_BF16 && dst_dtype == HAPMI_F32) hipLaunchKernelGGL((cast_kernel<bf16_t, float>), grid, block, 0, st, (const bf16_t *)src, (float *)dst, n);
    else if (src_dtype == HAPMI_F32) hipLaunchKernelGGL((cast_kernel<float, float>), grid, block, 0, st, (const float *)src, (float *)dst, n);
    else hipLaunchKernelGGL((cast_kernel<bf16_t, bf16_t>), grid, block, 0, st, (const bf16_t *)src, (bf16_t *)dst, n);
    HAPMI_CHECK_LAUNCH("cast");
    return HAPMI_OK;
}

// ---------------------------------------------------------------------------
// embedding
// ---------------------------------------------------------------------------
namespace {

template <typename T>
__global__ __launch_bounds__(256) void embedding_fwd_kernel(const int64_t *ids, const T *table, const T *pe, T *out,
                                                          int64_t n_tokens, int64_t d, int64_t S, int64_t vocab,
                                                          float scale) {
    // one wave per token row
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const int64_t id = ids[t];
    const bool ok = id >= 0 && id < vocab;
    const T *row = table + (ok ? id : 0) * d;
    const T *prow = pe ? pe + (t % S) * d : nullptr;
    for (int64_t c = lane; c < d; c += 64) {
        float v = ok ? ld_f(row, c) : NAN;       // an id outside the table poisons the row instead of faulting
        v *= scale;
        if (sizeof(T) == 2) v = (float)(bf16_t)v;   // `* scale` is its own node: round like the unfused program
        if (prow) v += ld_f(prow, c);
        st_f(out + t * d, c, v);
    }
}

// dtable[id, :] += sum over the tokens t with ids[t] == id of dout[t, :] * scale, added in token order.  One wave per
// token; the wave of the FIRST token of an id (no earlier token has the same id) gathers all of that id's rows in
// registers and adds the sum to the table row, the other waves leave.  No atomics and one writer per table row, so
// the same call gives the same bits every time.  A wave holds 64 * EB_COLS columns of a row; wider rows are cut into
// column blocks over blockIdx.y.  Cost: every wave reads all earlier ids (n_tokens^2 / 2 id loads per call and column
// block, 64 per instruction): 19 M for the 6144 tokens of a [12, 512] shard, negligible next to the rows moved; a batch
// of far more tokens per call would want a sort by id first.
constexpr int EB_COLS = 32;
template <typename T>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int64_t *ids, const T *dout, float *dtable,
                                                          int64_t n_tokens, int64_t d, int64_t vocab, float scale) {
    const int lane = threadIdx.x & 63;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const int64_t id = ids[t];
    if (id < 0 || id >= vocab) return;
    const int64_t col0 = (int64_t)blockIdx.y * (64 * EB_COLS);   // this block's columns: col0 .. col0 + 64 * EB_COLS
    // is an earlier token of the same id?  (wave-uniform)
    for (int64_t u0 = 0; u0 < t; u0 += 64) {
        const int64_t u = u0 + lane;
        const bool hit = u < t && ids[u] == id;
        if (__ballot(hit) != 0ull) return;
    }
    float acc[EB_COLS];
#pragma unroll
    for (int j = 0; j < EB_COLS; ++j) acc[j] = 0.f;
    for (int64_t u0 = t / 64 * 64; u0 < n_tokens; u0 += 64) {
        const int64_t u = u0 + lane;
        unsigned long long hits = __ballot(u >= t && u < n_tokens && ids[u] == id);
        while (hits) {                                            // ascending token order
            const int b = __ffsll((long long)hits) - 1;
            hits &= hits - 1;
            const T *row = dout + (u0 + b) * d;
#pragma unroll
            for (int j = 0; j < EB_COLS; ++j) {
                const int64_t c = col0 + (int64_t)j * 64 + lane;
                if (col0 + (int64_t)j * 64 < d && c < d) {
                    float g = ld_f(row, c) * scale;
                    if (sizeof(T) == 2) g = (float)(bf16_t)g;
                    acc[j] += g;
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < EB_COLS; ++j) {
        const int64_t c = col0 + (int64_t)j * 64 + lane;
        if (col0 + (int64_t)j * 64 < d && c < d) dtable[id * d + c] += acc[j];
    }
}

}  // namespace

extern "C" int hapmi_embedding_fwd(const int64_t *ids, const void *table, const void *pe, void *out,
                                   int64_t n_tokens, int64_t d, int64_t S, int64_t vocab, float scale, int dtype,
                                   hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && n_tokens >= 0 && d >= 1 && vocab >= 1 && S >= 1, HAPMI_EINVAL, "embedding_fwd: bad argument");
    if (n_tokens == 0) return HAPMI_OK;
    HAPMI_REQUIRE(ids && table && out, HAPMI_EINVAL, "embedding_fwd: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(n_tokens, 4));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((embedding_fwd_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, ids, (const float *)table, (const float *)pe, (float *)out, n_tokens, d, S, vocab, scale);
    else
        hipLaunchKernelGGL((embedding_fwd_kernel<bf16_t>), grid, dim3(256), 0, (hipStream_t)stream, ids, (const bf16_t *)table, (const bf16_t *)pe, (bf16_t *)out, n_tokens, d, S, vocab, scale);
    HAPMI_CHECK_LAUNCH("embedding_fwd");
    return HAPMI_OK;
}

extern "C" int hapmi_embedding_bwd(const int64_t *ids, const void *dout, float *dtable, int64_t n_tokens, int64_t d,
                                   int64_t vocab, float scale, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && n_tokens >= 0 && d >= 1 && vocab >= 1, HAPMI_EINVAL, "embedding_bwd: bad argument");
    HAPMI_REQUIRE(hapmi_cdiv(d, 64 * EB_COLS) <= 65535, HAPMI_ELIMIT, "embedding_bwd: rows of at most %d elements", 65535 * 64 * EB_COLS);
    if (n_tokens == 0) return HAPMI_OK;
    HAPMI_REQUIRE(ids && dout && dtable, HAPMI_EINVAL, "embedding_bwd: null pointer");
    dim3 grid((unsigned)hapmi_cdiv(n_tokens, 4), (unsigned)hapmi_cdiv(d, 64 * EB_COLS));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((embedding_bwd_kernel<float>), grid, dim3(256), 0, (hipStream_t)stream, ids, (const float *)dout, dtable, n_tokens, d, vocab, scale);
    else
        hipLaunchKernelGGL((embedding_bwd_kernel<bf16_t>), grid, dim3(256), 0, (hipStream_t)stream, ids, (const bf16_t *)dout, dtable, n_tokens, d, vocab, scale);
    HAPMI_CHECK_LAUNCH("embedding_bwd");
    return HAPMI_OK;
}

// ---------------------------------------------------------------------------
// ViT leaves
// ---------------------------------------------------------------------------
namespace {

template <typename T>
__global__ __launch_bounds__(EW_THREADS) void patchify_kernel(const float *x, T *cols, int64_t b, int64_t C, int64_t gh,
                                                            int64_t gw, int64_t ph, int64_t pw) {
    // cols[(n, gy, gx), (c, py, px)] = x[n, c, gy*ph + py, gx*pw + px]; threads run along px (contiguous in x)
    const int64_t K = C * ph * pw, total = b * gh * gw * K, step = (int64_t)gridDim.x * EW_THREADS;
    const int64_t H = gh * ph, W = gw * pw;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += step) {
        const int64_t row = i / K, k = i - row * K;
        const int64_t n = row / (gh * gw), g = row - n * gh * gw, gy = g / gw, gx = g - gy * gw;
        const int64_t c = k / (ph * pw), q = k - c * ph * pw, py = q / pw, px = q - py * pw;
        st_f(cols, i, x[((n * C + c) * H + gy * ph + py) * W + gx * pw + px]);
    }
}

template <typename T>
__global__ __launch_bounds__(EW_THREADS) void append_cls_pos_kernel(const T *patches, const T *cls, const T *pos, T *out,
                                                                  int64_t b, int64_t T1, int64_t d) {
    // out[b, T1, d] with T1 = T + 1
    const int64_t total = b * T1 * d, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < total; i += step) {
        const int64_t n = i / (T1 * d), r = i - n * T1 * d, t = r / d, c = r - t * d;
        const float v = t == 0 ? ld_f(cls, c) : ld_f(patches, (n * (T1 - 1) + (t - 1)) * d + c);
        st_f(out, i, pos ? v + ld_f(pos, t * d + c) : v);
    }
}

}  // namespace

extern "C" int hapmi_patchify(const float *x, void *cols, int64_t b, int64_t C, int64_t gh, int64_t gw, int64_t ph,
                              int64_t pw, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && b >= 0 && C >= 1 && gh >= 1 && gw >= 1 && ph >= 1 && pw >= 1, HAPMI_EINVAL, "patchify: bad argument");
    if (b == 0) return HAPMI_OK;
    HAPMI_REQUIRE(x && cols, HAPMI_EINVAL, "patchify: null pointer");
    dim3 grid(ew_grid(b * gh * gw * C * ph * pw));
    if (dtype == HAPMI_F32) hipLaunchKernelGGL((patchify_kernel<float>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, x, (float *)cols, b, C, gh, gw, ph, pw);
    else hipLaunchKernelGGL((patchify_kernel<bf16_t>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, x, (bf16_t *)cols, b, C, gh, gw, ph, pw);
    HAPMI_CHECK_LAUNCH("patchify");
    return HAPMI_OK;
}

extern "C" int hapmi_append_cls_pos(const void *patches, const void *cls, const void *pos, void *out, int64_t b,
                                    int64_t T, int64_t d, int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && b >= 0 && T >= 0 && d >= 1, HAPMI_EINVAL, "append_cls_pos: bad argument");
    if (b == 0) return HAPMI_OK;
    HAPMI_REQUIRE(patches && cls && out, HAPMI_EINVAL, "append_cls_pos: null pointer");
    dim3 grid(ew_grid(b * (T + 1) * d));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((append_cls_pos_kernel<float>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, (const float *)patches, (const float *)cls, (const float *)pos, (float *)out, b, T + 1, d);
    else
        hipLaunchKernelGGL((append_cls_pos_kernel<bf16_t>), grid, dim3(EW_THREADS), 0, (hipStream_t)stream, (const bf16_t *)patches, (const bf16_t *)cls, (const bf16_t *)pos, (bf16_t *)out, b, T + 1, d);
    HAPMI_CHECK_LAUNCH("append_cls_pos");
    return HAPMI_OK;
}

// ---------------------------------------------------------------------------
// optimizer
// ---------------------------------------------------------------------------
namespace {

__global__ __launch_bounds__(EW_THREADS) void sgd_kernel(float *p, const float *g, bf16_t *shadow, int64_t n, float lr,
                                                       const float *gscale) {
    const float gs = gscale ? gscale[0] : 1.0f;
    const int64_t nv = n / 4, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < nv; i += step) {
        f32x4 pv = ld_stream((const f32x4 *)p + i);
        const f32x4 gv = ld_stream((const f32x4 *)g + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) pv[k] = pv[k] - lr * (gv[k] * gs);
        st_stream(pv, (f32x4 *)p + i);
        if (shadow) {
            bf16x4 s;
#pragma unroll
            for (int k = 0; k < 4; ++k) s[k] = (bf16_t)pv[k];
            st_stream(s, (bf16x4 *)shadow + i);
        }
    }
    for (int64_t i = nv * 4 + (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step) {
        const float v = p[i] - lr * (g[i] * gs);
        p[i] = v;
        if (shadow) shadow[i] = (bf16_t)v;
    }
}

struct AdamHyper {
    float lr, beta1, beta2, eps, bc1, bc2;
};

__device__ __forceinline__ float adam_one(float p, float g, float &m, float &v, const AdamHyper &h) {
    // same order of operations as torch.optim.Adam's single-tensor path
    m = m + (g - m) * (1.0f - h.beta1);                       // lerp
    v = v * h.beta2 + (1.0f - h.beta2) * g * g;
    const float denom = sqrtf(v) / sqrtf(h.bc2) + h.eps;
    return p - (h.lr / h.bc1) * (m / denom);
}

// state = {step count, 1 - beta1^step, 1 - beta2^step}: advanced on the device so that a captured HIP graph,
// whose kernel arguments are frozen, still sees the right bias corrections on every replay
__global__ void adam_advance_kernel(float *state, float beta1, float beta2) {
    const double step = (double)state[0] + 1.0;
    state[0] = (float)step;
    state[1] = (float)(1.0 - pow((double)beta1, step));
    state[2] = (float)(1.0 - pow((double)beta2, step));
}

__global__ __launch_bounds__(EW_THREADS) void adam_kernel(float *p, const float *g, float *m, float *v, bf16_t *shadow,
                                                        int64_t n, AdamHyper h, const float *gscale,
                                                        const float *state) {
    if (state) {
        h.bc1 = state[1];
        h.bc2 = state[2];
    }
    const float gs = gscale ? gscale[0] : 1.0f;
    const int64_t nv = n / 4, step = (int64_t)gridDim.x * EW_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < nv; i += step) {
        f32x4 pv = ld_stream((const f32x4 *)p + i), mv = ld_stream((const f32x4 *)m + i), vv = ld_stream((const f32x4 *)v + i);
        const f32x4 gv = ld_stream((const f32x4 *)g + i);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            float mk = mv[k], vk = vv[k];
            pv[k] = adam_one(pv[k], gv[k] * gs, mk, vk, h);
            mv[k] = mk;
            vv[k] = vk;
        }
        st_stream(pv, (f32x4 *)p + i);
        st_stream(mv, (f32x4 *)m + i);
        st_stream(vv, (f32x4 *)v + i);
        if (shadow) {
            bf16x4 s;
#pragma unroll
            for (int k = 0; k < 4; ++k) s[k] = (bf16_t)pv[k];
            st_stream(s, (bf16x4 *)shadow + i);
        }
    }
    for (int64_t i = nv * 4 + (int64_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += step) {
        float mk = m[i], vk = v[i];
        const float pn = adam_one(p[i], g[i] * gs, mk, vk, h);
        p[i] = pn;
        m[i] = mk;
        v[i] = vk;
        if (shadow) shadow[i] = (bf16_t)pn;
    }
}

// Sum of squares in two deterministic stages: the input is cut into chunks of SUMSQ_CHUNK elements (a partition
// that does not depend on the grid), partials[c] is chunk c's sum in a fixed order, and one block adds the
// partials in a fixed order.  No atomics: the same call gives the same bits every time.
constexpr int64_t SUMSQ_CHUNK = 16384;
__global__ __launch_bounds__(EW_THREADS) void sumsq_partial_kernel(const float *g, int64_t n, float *partials, int64_t n_chunks) {
    __shared__ float red[16];
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const int64_t i0 = c * SUMSQ_CHUNK, i1 = i0 + SUMSQ_CHUNK < n ? i0 + SUMSQ_CHUNK : n;
        float s = 0.f;
        for (int64_t i = i0 + threadIdx.x; i < i1; i += EW_THREADS) s += g[i] * g[i];
        s = block_sum(s, red);
        if (threadIdx.x == 0) partials[c] = s;
    }
}
__global__ __launch_bounds__(EW_THREADS) void sumsq_final_kernel(const float *partials, int64_t n_chunks, float *out) {
    __shared__ float red[16];
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n_chunks; i += EW_THREADS) s += partials[i];
    s = block_sum(s, red);
    if (threadIdx.x == 0) out[0] = s;
}

__global__ void clip_coef_kernel(const float *sumsq, float max_norm, float *coef) {
    const float c = max_norm / (sqrtf(sumsq[0]) + 1e-6f);
    coef[0] = c < 1.0f ? c : 1.0f;
}

}  // namespace

extern "C" int hapmi_sgd_step(float *param, const float *grad, void *shadow, int64_t n, float lr,
                              const float *grad_scale_dev, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0, HAPMI_EINVAL, "sgd_step: negative size");
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(param && grad, HAPMI_EINVAL, "sgd_step: null pointer");
    HAPMI_REQUIRE(aligned16(param) && aligned16(grad) && (!shadow || ((uintptr_t)shadow % 8) == 0), HAPMI_EALIGN, "sgd_step: misaligned buffer");
    hipLaunchKernelGGL(sgd_kernel, dim3(stream_grid(hapmi_cdiv(n, 4))), dim3(EW_THREADS), 0, (hipStream_t)stream, param, grad, (bf16_t *)shadow, n, lr, grad_scale_dev);
    HAPMI_CHECK_LAUNCH("sgd_step");
    return HAPMI_OK;
}

extern "C" int hapmi_adam_step(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow,
                               int64_t n, float lr, float beta1, float beta2, float eps, float bias_corr1,
                               float bias_corr2, const float *grad_scale_dev, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0, HAPMI_EINVAL, "adam_step: negative size");
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(param && grad && exp_avg && exp_avg_sq, HAPMI_EINVAL, "adam_step: null pointer");
    HAPMI_REQUIRE(aligned16(param) && aligned16(grad) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                      (!shadow || ((uintptr_t)shadow % 8) == 0),
                  HAPMI_EALIGN, "adam_step: misaligned buffer");
    AdamHyper h{lr, beta1, beta2, eps, bias_corr1, bias_corr2};
    hipLaunchKernelGGL(adam_kernel, dim3(stream_grid(hapmi_cdiv(n, 4))), dim3(EW_THREADS), 0, (hipStream_t)stream, param, grad, exp_avg, exp_avg_sq, (bf16_t *)shadow, n, h, grad_scale_dev, (const float *)nullptr);
    HAPMI_CHECK_LAUNCH("adam_step");
    return HAPMI_OK;
}

extern "C" int hapmi_adam_step_dev(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow,
                                   int64_t n, float lr, float beta1, float beta2, float eps, float *state_dev,
                                   const float *grad_scale_dev, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0, HAPMI_EINVAL, "adam_step_dev: negative size");
    HAPMI_REQUIRE(state_dev, HAPMI_EINVAL, "adam_step_dev: null state");
    hipLaunchKernelGGL(adam_advance_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, state_dev, beta1, beta2);
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(param && grad && exp_avg && exp_avg_sq, HAPMI_EINVAL, "adam_step_dev: null pointer");
    HAPMI_REQUIRE(aligned16(param) && aligned16(grad) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                      (!shadow || ((uintptr_t)shadow % 8) == 0),
                  HAPMI_EALIGN, "adam_step_dev: misaligned buffer");
    AdamHyper h{lr, beta1, beta2, eps, 1.f, 1.f};
    hipLaunchKernelGGL(adam_kernel, dim3(stream_grid(hapmi_cdiv(n, 4))), dim3(EW_THREADS), 0, (hipStream_t)stream, param, grad, exp_avg, exp_avg_sq, (bf16_t *)shadow, n, h, grad_scale_dev, (const float *)state_dev);
    HAPMI_CHECK_LAUNCH("adam_step_dev");
    return HAPMI_OK;
}

extern "C" int hapmi_adam_advance(float *state_dev, float beta1, float beta2, hapmi_stream_t stream) {
    HAPMI_REQUIRE(state_dev, HAPMI_EINVAL, "adam_advance: null state");
    hipLaunchKernelGGL(adam_advance_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, state_dev, beta1, beta2);
    HAPMI_CHECK_LAUNCH("adam_advance");
    return HAPMI_OK;
}

extern "C" int hapmi_adam_apply_dev(float *param, const float *grad, float *exp_avg, float *exp_avg_sq, void *shadow,
                                    int64_t n, float lr, float beta1, float beta2, float eps, const float *state_dev,
                                    const float *grad_scale_dev, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0, HAPMI_EINVAL, "adam_apply_dev: negative size");
    HAPMI_REQUIRE(state_dev, HAPMI_EINVAL, "adam_apply_dev: null state");
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(param && grad && exp_avg && exp_avg_sq, HAPMI_EINVAL, "adam_apply_dev: null pointer");
    HAPMI_REQUIRE(aligned16(param) && aligned16(grad) && aligned16(exp_avg) && aligned16(exp_avg_sq) &&
                      (!shadow || ((uintptr_t)shadow % 8) == 0),
                  HAPMI_EALIGN, "adam_apply_dev: misaligned buffer");
    AdamHyper h{lr, beta1, beta2, eps, 1.f, 1.f};
    hipLaunchKernelGGL(adam_kernel, dim3(stream_grid(hapmi_cdiv(n, 4))), dim3(EW_THREADS), 0, (hipStream_t)stream, param, grad, exp_avg, exp_avg_sq, (bf16_t *)shadow, n, h, grad_scale_dev, state_dev);
    HAPMI_CHECK_LAUNCH("adam_apply_dev");
    return HAPMI_OK;
}

namespace {
int sumsq_launch(const float *g, int64_t n, float *out, float *partials, hipStream_t st) {
    const int64_t n_chunks = hapmi_cdiv(n, SUMSQ_CHUNK);
    int64_t gx = n_chunks < 2048 ? n_chunks : 2048;
    hipLaunchKernelGGL(sumsq_partial_kernel, dim3((unsigned)gx), dim3(EW_THREADS), 0, st, g, n, partials, n_chunks);
    hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(EW_THREADS), 0, st, (const float *)partials, n_chunks, out);
    HAPMI_CHECK_LAUNCH("sumsq");
    return HAPMI_OK;
}
}  // namespace

extern "C" int hapmi_sumsq_workspace_elems(int64_t n, int64_t *elems_host) {
    HAPMI_REQUIRE(n >= 0 && elems_host, HAPMI_EINVAL, "sumsq_workspace_elems: bad argument");
    *elems_host = hapmi_cdiv(n, SUMSQ_CHUNK);
    return HAPMI_OK;
}

extern "C" int hapmi_sumsq(const float *g, int64_t n, float *out, float *workspace, int64_t workspace_elems,
                           hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0 && out, HAPMI_EINVAL, "sumsq: bad argument");
    if (n == 0) {
        hipLaunchKernelGGL(zero_f32_kernel, dim3(1), dim3(EW_THREADS), 0, (hipStream_t)stream, out, (int64_t)1);
        return HAPMI_OK;
    }
    HAPMI_REQUIRE(g && workspace, HAPMI_EINVAL, "sumsq: null pointer");
    HAPMI_REQUIRE(workspace_elems >= hapmi_cdiv(n, SUMSQ_CHUNK), HAPMI_ELIMIT,
                  "sumsq: %lld elements need a workspace of %lld floats, %lld given", (long long)n,
                  (long long)hapmi_cdiv(n, SUMSQ_CHUNK), (long long)workspace_elems);
    return sumsq_launch(g, n, out, workspace, (hipStream_t)stream);
}

// ---- hapmi_sumsq_static: the same sum for callers that cannot allocate -------------------------------------
// The partial sums live in a file-scope device array instead of a caller workspace.  Each GPU holds its own copy
// of the array at its own address: the address is looked up once per device (with that device current) and only
// that pointer is ever handed to kernels -- the array's name is not a device address in host code.
constexpr int64_t SUMSQ_STATIC_CHUNKS = 65536;                    // 256 KiB per GPU; 2^30 elements at most
static __device__ __align__(256) float g_sumsq_scratch[SUMSQ_STATIC_CHUNKS];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float *g_scratch_ptr[kMaxDevices] = {nullptr};

// the device a stream belongs to (the current device for the null stream)
int device_of_stream(hipStream_t st, int *dev) {
    hipError_t e = st ? hipStreamGetDevice(st, dev) : hipGetDevice(dev);
    if (e != hipSuccess) return hapmi_set_error(HAPMI_ELAUNCH, "sumsq_static: device of the stream: %s", hipGetErrorString(e));
    HAPMI_REQUIRE(*dev >= 0 && *dev < kMaxDevices, HAPMI_ELIMIT, "sumsq_static: device index %d beyond %d", *dev, kMaxDevices);
    return HAPMI_OK;
}
}  // namespace

// Looks up the address of the current device's copy of the scratch array (hapmi_init calls this, so that a later
// hapmi_sumsq_static is a pure enqueue: no symbol lookup, no lazy module load, nothing a stream capture would record
// or refuse).
int hapmi_sumsq_static_setup() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hapmi_set_error(HAPMI_ELAUNCH, "sumsq_static: hipGetDevice: %s", hipGetErrorString(e));
    HAPMI_REQUIRE(dev >= 0 && dev < kMaxDevices, HAPMI_ELIMIT, "sumsq_static: device index %d beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_sumsq_scratch));
        if (e != hipSuccess || !p)
            return hapmi_set_error(HAPMI_ELAUNCH, "sumsq_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = (float *)p;
    }
    return HAPMI_OK;
}

extern "C" int hapmi_sumsq_static(const float *g, int64_t n, float *out, hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0 && out, HAPMI_EINVAL, "sumsq_static: bad argument");
    if (n == 0) {
        hipLaunchKernelGGL(zero_f32_kernel, dim3(1), dim3(EW_THREADS), 0, (hipStream_t)stream, out, (int64_t)1);
        HAPMI_CHECK_LAUNCH("sumsq_static");
        return HAPMI_OK;
    }
    HAPMI_REQUIRE(g, HAPMI_EINVAL, "sumsq_static: null pointer");
    HAPMI_REQUIRE(hapmi_cdiv(n, SUMSQ_CHUNK) <= SUMSQ_STATIC_CHUNKS, HAPMI_ELIMIT,
                  "sumsq_static: %lld elements exceed the built-in scratch (at most %lld elements; use hapmi_sumsq "
                  "with a workspace)", (long long)n, (long long)(SUMSQ_STATIC_CHUNKS * SUMSQ_CHUNK));
    int dev = -1;
    const int rc = device_of_stream((hipStream_t)stream, &dev);
    if (rc) return rc;
    float *scratch = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        scratch = g_scratch_ptr[dev];
    }
    HAPMI_REQUIRE(scratch, HAPMI_EINVAL,
                  "sumsq_static: hapmi_init() has not run with device %d current (it looks up that device's scratch "
                  "array; this call only enqueues kernels)", dev);
    // every partial sum that the final kernel reads is written by the first kernel of this call: nothing in the
    // array has to start at zero, whatever an earlier call left there
    return sumsq_launch(g, n, out, scratch, (hipStream_t)stream);
}

extern "C" int hapmi_clip_coef(const float *sumsq, float max_norm, float *coef, hapmi_stream_t stream) {
    HAPMI_REQUIRE(sumsq && coef, HAPMI_EINVAL, "clip_coef: null pointer");
    hipLaunchKernelGGL(clip_coef_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, sumsq, max_norm, coef);
    HAPMI_CHECK_LAUNCH("clip_coef");
    return HAPMI_OK;
}
