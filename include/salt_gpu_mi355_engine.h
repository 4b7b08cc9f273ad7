/* salt_gpu_mi355_engine.h -- the engine-facing half of the C ABI: the
 * salt_gpu_* entry points of the reference's include/salt/gpu.h that lie on
 * the quantized decode path, with identical names, argument order and
 * structure layouts. */
#ifndef SALT_GPU_MI355_ENGINE_H
#define SALT_GPU_MI355_ENGINE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* reference gpu.h:26-27 */
int salt_gpu_init(void);
int salt_gpu_free(void);

#ifdef __cplusplus
}
#endif

#endif /* SALT_GPU_MI355_ENGINE_H */
