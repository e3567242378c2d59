// GEMM tile configuration 12: a measurement build of configuration 7 (192 x 128 block tile, 2 x 4 waves, three LDS
// stages) that moves every k-tile's operands from memory into LDS and waits for them as configuration 7 does, but
// reads no fragments and issues no MFMA.  Its result is zeros; only hapmi_gemm_tuning selects it.  The time of a
// launch is what the operand movement alone costs (bench.py --gemm-table prints it next to the real launch).
#include "gemm_kernel.h"

HAPMI_GEMM_DECLARE_CFG(12) {
    if (in_dtype != HAPMI_BF16 || out_dtype != HAPMI_BF16)
        return hapmi_set_error(HAPMI_EINVAL, "gemm: tile configuration 12 (operand movement only) takes bf16 operands and results");
    return launch_cfg<bf16_t, bf16_t, 192, 128, 2, 4, 3, 8>(p, transA, transB, batch, st);
}
