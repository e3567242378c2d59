// Kernels of GEMM tile configuration 6: 128 x 256 block tile, 2 x 4 waves.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(6) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 6 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 128, 256, 2, 4, 3>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 128, 256, 2, 4, 3>(p, transA, transB, batch, st);
}
