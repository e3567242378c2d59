// Kernels of GEMM tile configuration 9: 128 x 192 block tile, 4 x 2 waves (wave tile 32 x 96), three stages.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(9) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 9 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 128, 192, 4, 2, 3>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 128, 192, 4, 2, 3>(p, transA, transB, batch, st);
}
