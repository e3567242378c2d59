// Kernels of GEMM tile configuration 10: 64 x 64 block tile, 2 x 2 waves (wave tile 32 x 32), float32 operands:
// the float32 MFMA is an eighth of the bf16 rate, so a [384, 512] output needs small tiles to spread over the chip.
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(10) {
    if (in_dtype != HAPMI_F32) return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 10 takes float32 operands only");
    if (out_dtype == HAPMI_F32) return launch_cfg<float, float, 64, 64, 2, 2>(p, transA, transB, batch, st);
    return launch_cfg<float, bf16_t, 64, 64, 2, 2>(p, transA, transB, batch, st);
}
