// Kernels of GEMM tile configuration 3: 192 x 256 block tile, 2 x 4 waves.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(3) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 3 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 192, 256, 2, 4>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 192, 256, 2, 4>(p, transA, transB, batch, st);
}
