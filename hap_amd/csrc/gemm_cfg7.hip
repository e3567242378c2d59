// Kernels of GEMM tile configuration 7: 192 x 128 block tile, 2 x 4 waves (wave tile 96 x 32): a [6144, 1024]
// output is 256 such tiles, one per compute unit.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(7) {
    if (in_dtype != HAPMI_BF16) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 7 takes bf16 operands only");
    if (out_dtype == HAPMI_BF16) return launch_cfg<bf16_t, bf16_t, 192, 128, 2, 4, 3>(p, transA, transB, batch, st);
    return launch_cfg<bf16_t, float, 192, 128, 2, 4, 3>(p, transA, transB, batch, st);
}
