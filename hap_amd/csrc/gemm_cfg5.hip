// Kernels of GEMM tile configuration 5: 256 x 128 block tile, 4 x 2 waves.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(5) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 5 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 256, 128, 4, 2, 3>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 256, 128, 4, 2, 3>(p, transA, transB, batch, st);
}
