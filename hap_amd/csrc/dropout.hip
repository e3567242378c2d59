// F.dropout in training mode (hap.rs:1464): y = x * keep / (1 - p) with counter-based keep decisions (dropout.h).
#include "common.h"
#include "dropout.h"

namespace {

constexpr int DR_THREADS = 256;

inline unsigned dr_grid(int64_t n_items) {
    int64_t g = hapmi_cdiv(n_items, DR_THREADS);
    if (g > 256 * 32) g = 256 * 32;
    if (g < 1) g = 1;
    return (unsigned)g;
}

template <typename T>
__global__ __launch_bounds__(DR_THREADS) void dropout_kernel(const T *x, T *y, int64_t n, float p, const int64_t *state,
                                                          int64_t stream_id) {
    constexpr int EPV = Vec16<T>::N;
    const DropKey key = drop_key(state[0], state[1], stream_id, p);
    const int64_t nv = n / EPV, step = (int64_t)gridDim.x * DR_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * DR_THREADS + threadIdx.x; i < nv; i += step) {
        Vec16<T> v = ((const Vec16<T> *)x)[i], r;
#pragma unroll
        for (int k = 0; k < EPV; k += 2) {
            const uint32_t bits = drop_pair_bits(key, (uint64_t)(i * EPV + k) >> 1);
            r.set(k, (bits & 0xffffU) >= key.thr ? v.get(k) * key.scale : 0.f);
            r.set(k + 1, (bits >> 16) >= key.thr ? v.get(k + 1) * key.scale : 0.f);
        }
        ((Vec16<T> *)y)[i] = r;
    }
    for (int64_t i = nv * EPV + (int64_t)blockIdx.x * DR_THREADS + threadIdx.x; i < n; i += step)
        st_f(y, i, drop_keep(key, (uint64_t)i) ? ld_f(x, i) * key.scale : 0.f);
}

__global__ __launch_bounds__(DR_THREADS) void dropout_mask_kernel(uint8_t *mask, int64_t n, float p, const int64_t *state,
                                                               int64_t stream_id) {
    const DropKey key = drop_key(state[0], state[1], stream_id, p);
    const int64_t step = (int64_t)gridDim.x * DR_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * DR_THREADS + threadIdx.x; i < n; i += step)
        mask[i] = drop_keep(key, (uint64_t)i) ? 1 : 0;
}

__global__ void rng_advance_kernel(int64_t *state) { state[1] += 1; }

}  // namespace

extern "C" int hapmi_dropout(const void *x, void *y, int64_t n, float p, const int64_t *rng_state_dev, int64_t stream_id,
                             int dtype, hapmi_stream_t stream) {
    HAPMI_REQUIRE(hapmi_dtype_ok(dtype) && n >= 0 && p >= 0.f && p <= 1.f, HAPMI_EINVAL, "dropout: bad argument (p = %g)", (double)p);
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(x && y && rng_state_dev, HAPMI_EINVAL, "dropout: null pointer");
    HAPMI_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EALIGN,
                  "dropout: x and y must be 16-byte aligned");
    const int64_t epv = dtype == HAPMI_F32 ? 4 : 8;
    dim3 grid(dr_grid(hapmi_cdiv(n, epv)));
    if (dtype == HAPMI_F32)
        hipLaunchKernelGGL((dropout_kernel<float>), grid, dim3(DR_THREADS), 0, (hipStream_t)stream, (const float *)x, (float *)y, n, p, rng_state_dev, stream_id);
    else
        hipLaunchKernelGGL((dropout_kernel<bf16_t>), grid, dim3(DR_THREADS), 0, (hipStream_t)stream, (const bf16_t *)x, (bf16_t *)y, n, p, rng_state_dev, stream_id);
    HAPMI_CHECK_LAUNCH("dropout");
    return HAPMI_OK;
}

extern "C" int hapmi_dropout_mask(uint8_t *mask, int64_t n, float p, const int64_t *rng_state_dev, int64_t stream_id,
                                  hapmi_stream_t stream) {
    HAPMI_REQUIRE(n >= 0 && p >= 0.f && p <= 1.f, HAPMI_EINVAL, "dropout_mask: bad argument (p = %g)", (double)p);
    if (n == 0) return HAPMI_OK;
    HAPMI_REQUIRE(mask && rng_state_dev, HAPMI_EINVAL, "dropout_mask: null pointer");
    hipLaunchKernelGGL(dropout_mask_kernel, dim3(dr_grid(n)), dim3(DR_THREADS), 0, (hipStream_t)stream, mask, n, p, rng_state_dev, stream_id);
    HAPMI_CHECK_LAUNCH("dropout_mask");
    return HAPMI_OK;
}

extern "C" int hapmi_rng_advance(int64_t *rng_state_dev, hapmi_stream_t stream) {
    HAPMI_REQUIRE(rng_state_dev && ((uintptr_t)rng_state_dev % 8) == 0, HAPMI_EINVAL, "rng_advance: bad state pointer");
    hipLaunchKernelGGL(rng_advance_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, rng_state_dev);
    HAPMI_CHECK_LAUNCH("rng_advance");
    return HAPMI_OK;
}
