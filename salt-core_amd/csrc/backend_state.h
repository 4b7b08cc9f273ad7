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
    hipStream_t side = nullptr;         // second branch of a forked sequence (default priority, like every stream)
    hipEvent_t fork = nullptr, join = nullptr;
    int tolerance_class = 0;            // policy: the engine entry points may run the tolerance-class kernels
    float code_scale = 0.0f;            // 1 / fp8_table[1]
    int fp8_is_ocp = 0;                 // the converter decodes every byte as OCP E4M3FN
    float fp8_table[256] = {0};
    float fp4_table[512] = {0};
    char last_error[256] = {0};
    char last_kernel[96] = {0};
    // Ring of device + pinned copies of multi-job tables.  A slot is reused
    // only after the event recorded behind its last consumer has completed.
    struct TableSlot {
        void *device = nullptr;
        void *pinned = nullptr;
        size_t capacity = 0;
        size_t valid_bytes = 0;         // bytes of `pinned` that the device copy mirrors (0: none)
        hipStream_t stream = nullptr;   // the stream that carried the upload
        hipEvent_t done = nullptr;
        int busy = 0;
    };
    static constexpr int kTableSlots = 8;
    TableSlot tables[kTableSlots];
    int next_table = 0;
};

extern State g_state;

void set_error(const char *format, ...) __attribute__((format(printf, 1, 2)));
int hip_ok(hipError_t status, const char *what);
// Copies a host job table to the device on `stream`; after the consuming
// launch has been enqueued the caller hands the slot back with table_release.
State::TableSlot *table_acquire(const void *host_table, size_t nbytes, hipStream_t stream);
void table_release(State::TableSlot *slot, hipStream_t stream);

}  // namespace mi355
