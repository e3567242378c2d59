// Kernels of GEMM tile configuration 11: 64 x 128 block tile, 2 x 2 waves (wave tile 32 x 64), float32 operands.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(11) {
    if (in_dtype != HAPMI_F32) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 11 takes float32 operands only");
    if (out_dtype == HAPMI_F32) return launch_cfg<float, float, 64, 128, 2, 2>(p, transA, transB, batch, st);
    return launch_cfg<float, bf16_t, 64, 128, 2, 2>(p, transA, transB, batch, st);
}
