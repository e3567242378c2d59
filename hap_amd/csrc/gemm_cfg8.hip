// Kernels of GEMM tile configuration 8: 256 x 128 block tile, 2 x 2 waves (wave tile 128 x 64), one block per CU.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(8) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 8 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 256, 128, 2, 2, 3>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 256, 128, 2, 2, 3>(p, transA, transB, batch, st);
}
