// Kernels of GEMM tile configuration 0: 128 x 128 block tile, 2 x 2 waves.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(0) {
    if (in_dtype == HAPMI_BF16 && out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 128, 128, 2, 2>(p, transA, transB, batch, st);
    if (in_dtype == HAPMI_BF16) return launch_cfg<bf16_t, float, 128, 128, 2, 2>(p, transA, transB, batch, st);
    if (out_dtype == HAPMI_F32) return launch_cfg<float, float, 128, 128, 2, 2>(p, transA, transB, batch, st);
    return launch_cfg<float, bf16_t, 128, 128, 2, 2>(p, transA, transB, batch, st);
}
