/* A C99 caller of the backend, the way the engine's own translation units are: includes both public headers,
 * takes the address of entry points of every group and asks the GPU-free questions.  Built and run by
 * tests/test_abi_exports.py with gcc -std=c99 -pedantic -Wall -Wextra -Werror; exits 0 when every answer is as
 * documented.  No compute call is made. */
#include <stdio.h>
#include <string.h>

#include "salt_gpu_mi355.h"
#include "salt_gpu_mi355_engine.h"

int main(void) {
    SaltGpuStartupRequirements req;
    SaltGpuExactCell cell;
    SaltMi355FfnLayer layer;
    SaltMi355Cell dev_cell;
    const void *entry[] = {
        (const void *)salt_gpu_q4_matvec, (const void *)salt_gpu_q4_batch, (const void *)salt_gpu_q4_moe_chain,
        (const void *)salt_gpu_nvfp4_matvec, (const void *)salt_gpu_q8_batch, (const void *)salt_gpu_bf16_matvec,
        (const void *)salt_gpu_exact_cells, (const void *)salt_mi355_moe_decode_step_dev,
        (const void *)salt_mi355_ffn_block_dev, (const void *)salt_mi355_bf16_matvec_dev,
        (const void *)salt_mi355_cells_dev};
    size_t k;
    memset(&cell, 0, sizeof cell);
    memset(&layer, 0, sizeof layer);
    memset(&dev_cell, 0, sizeof dev_cell);
    for (k = 0; k < sizeof entry / sizeof entry[0]; k++)
        if (!entry[k]) return 10;
    if (salt_gpu_rocm_present() != 1 || salt_gpu_cuda_present() != 0) return 11;
    if (salt_gpu_startup_requirements(&req, sizeof req) != 0) return 12;
    if (salt_gpu_startup_requirements(&req, sizeof req - 1) != -1) return 13;
    if (cell.kind != 0 || SALT_GPU_EXACT_ROUTER_INPUT != 6) return 14;
    if (salt_mi355_ffn_block_workspace_bytes(&layer) != 0) return 15;      /* an empty description is refused */
    if (salt_gpu_residency_backend_ops() == NULL || salt_gpu_residency_backend_ops()->abi_version != 1u) return 16;
    printf("c99 consumer ok\n");
    return 0;
}
