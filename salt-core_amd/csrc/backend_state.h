// Process-wide state of libsalt_gpu_mi355.so (one owner thread, no locks, as
// the reference backends: reference gpu_hip.cpp keeps file-scope statics).
#pragma once

#include <vector>

#include "../../include/salt_gpu_mi355.h"
#include "mi355_internal.h"

namespace mi355 {

struct State {
    int ready = 0;
    int compute_units = 0;
    hipStream_t stream = nullptr;
    float code_scale = 0.0f;            // 1 / fp8_table[1]
    int fp8_is_ocp = 0;                 // the converter decodes every byte as OCP E4M3FN
    float fp8_table[256] = {0};
    float fp4_table[512] = {0};
    char last_error[256] = {0};
    // device + pinned copies of the most recent multi-job table
    void *table_device = nullptr;
    void *table_pinned = nullptr;
    size_t table_capacity = 0;
};

extern State g_state;

void set_error(const char *format, ...) __attribute__((format(printf, 1, 2)));
int hip_ok(hipError_t status, const char *what);
void *stage_table(const void *host_table, size_t nbytes, hipStream_t stream);

}  // namespace mi355
