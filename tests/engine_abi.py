"""ctypes mirrors of the engine-facing structures declared in
include/salt_gpu_mi355_engine.h, and argument types for the entry points the
tests drive.  Test-side only."""
import ctypes as C

vp, i32, u32, u64, sz, f32 = C.c_void_p, C.c_int, C.c_uint32, C.c_uint64, C.c_size_t, C.c_float


class BatchStats(C.Structure):
    _fields_ = [(n, u64) for n in ("arena_batches", "trunk_batches", "expert_layer_batches", "mapped_only_misses",
                                   "direct_output_batches", "direct_output_jobs")]


class BatchStatsV2(C.Structure):
    _fields_ = BatchStats._fields_ + [(n, u64) for n in (
        "nvfp4_logical_packed_weight_bytes", "nvfp4_logical_weight_scale_bytes", "nvfp4_activation_input_bytes",
        "nvfp4_activation_qdq_bytes", "nvfp4_projection_output_bytes", "nvfp4_kernel_launches",
        "nvfp4_completion_fences", "nvfp4_h2d_ns", "nvfp4_qdq_ns", "nvfp4_projection_ns", "nvfp4_d2h_ns",
        "q4_weight_stationary_batches")]


class StartupRequirements(C.Structure):
    _fields_ = [("fixed_device_bytes", u64), ("fixed_pinned_host_bytes", u64), ("descriptor_bytes", u64),
                ("device_copied_weight_bytes", u64), ("max_output_floats", u32), ("max_batch_jobs", u32),
                ("shared_buffer_slots", u32), ("reserved", u32)]


class ResourceUsage(C.Structure):
    _fields_ = [("described_bytes", u64), ("registered_bytes", u64), ("pageable_bytes", u64),
                ("active_window_bytes", u64), ("peak_window_bytes", u64), ("device_copied_weight_bytes", u64),
                ("described_resources", u32), ("active_resources", u32), ("active_windows", u32), ("reserved", u32)]


class SharedBuffer(C.Structure):
    _fields_ = [("contents", vp), ("nbytes", sz), ("backend", vp)]


class MoeExpert(C.Structure):
    _fields_ = [("gate_vals", vp), ("gate_scales", vp), ("gate_biases", vp), ("gate_id", vp),
                ("up_vals", vp), ("up_scales", vp), ("up_biases", vp), ("up_id", vp),
                ("down_vals", vp), ("down_scales", vp), ("down_biases", vp), ("down_id", vp),
                ("group", i32), ("resource_slot", i32), ("logical_resource_id", u64)]


class SelectedJob(C.Structure):
    _fields_ = [("vals", vp), ("scales", vp), ("biases", vp), ("id", vp), ("inputs", vp), ("outputs", vp),
                ("rows", i32), ("cols", i32), ("batch", i32), ("resource_slot", i32), ("logical_resource_id", u64)]


class ResidencyPlan(C.Structure):
    _fields_ = [("device_budget_bytes", u64), ("permanent_bytes", u64), ("slot_base_offset", u64),
                ("slot_bytes", u64), ("staging_bytes", u64), ("slot_count", u32), ("staging_count", u32),
                ("device_alignment", u32), ("flags", u32)]


class PermanentLayout(C.Structure):
    _fields_ = [("permanent_bytes", u64), ("maximum_span_bytes", u64), ("span_count", u32), ("alignment", u32)]


RESIDENCY_READ = C.CFUNCTYPE(i32, vp, u64, vp, sz)


class PermanentSpan(C.Structure):      # reference gpu_residency.h:40-62
    _fields_ = [("kind", u32), ("resource_id", u32), ("value_offset", u64), ("scale_offset", u64), ("bias_offset", u64),
                ("logical_resource_id", u64), ("source_offset", u64), ("nbytes", u64), ("read", RESIDENCY_READ),
                ("read_context", vp), ("device_offset", u64)]


class ResidencyOps(C.Structure):
    _fields_ = [("abi_version", u32), ("ops_size", sz),
                ("create", C.CFUNCTYPE(i32, vp, C.POINTER(ResidencyPlan))),
                ("staging", C.CFUNCTYPE(i32, vp, u32, C.POINTER(vp), C.POINTER(sz))),
                ("populate", C.CFUNCTYPE(i32, vp, u32, u64, u32, sz, u64)),
                ("poll", C.CFUNCTYPE(i32, vp, u32, u64, C.POINTER(i32))),
                ("resolve", C.CFUNCTYPE(i32, vp, u64, sz, C.POINTER(C.c_size_t))),
                ("retire", C.CFUNCTYPE(i32, vp, u32, u64)),
                ("destroy", C.CFUNCTYPE(i32, vp)),
                ("permanent_layout", C.CFUNCTYPE(i32, vp, C.POINTER(PermanentLayout), sz)),
                ("permanent_span", C.CFUNCTYPE(i32, vp, u32, C.POINTER(PermanentSpan), sz)),
                ("permanent_copy", C.CFUNCTYPE(i32, vp, u32, u64, u32, sz, u64)),
                ("permanent_publish", C.CFUNCTYPE(i32, vp))]


class ExactCell(C.Structure):
    _fields_ = [("kind", C.c_int), ("views", C.POINTER(SharedBuffer) * 8), ("offsets", C.c_size_t * 8), ("n", u32),
                ("aux", u32), ("eps", C.c_float), ("scalar", C.c_float)]


def bind(lib):
    """Sets argument and result types of the engine entry points used by tests."""
    def sig(name, res, *args):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, list(args)
    for name in ("salt_gpu_init", "salt_gpu_free", "salt_gpu_cuda_present", "salt_gpu_rocm_present",
                 "salt_gpu_pageable_mmap_active", "salt_gpu_mapped_only", "salt_gpu_defer", "salt_gpu_sync",
                 "salt_gpu_selected_resources_fence", "salt_gpu_resident_trunk_unmap"):
        sig(name, i32)
    sig("salt_gpu_set_mapped_only", None, i32)
    sig("salt_gpu_set_defer", i32, i32)
    sig("salt_gpu_batch_stats_get", None, C.POINTER(BatchStats))
    sig("salt_gpu_batch_stats_get_v2", i32, C.POINTER(BatchStatsV2), sz)
    sig("salt_gpu_startup_requirements", i32, C.POINTER(StartupRequirements), sz)
    sig("salt_gpu_weight_resource_describe", i32, u32, u32, vp, sz)
    sig("salt_gpu_weight_resource_activate", i32, u32, u32, i32)
    sig("salt_gpu_weight_resource_pool_bind", i32, u32, u32)
    sig("salt_gpu_weight_resource_deactivate", i32, u32, u32)
    sig("salt_gpu_weight_resource_usage", i32, C.POINTER(ResourceUsage), sz)
    sig("salt_gpu_weight_resource_bind", i32, u32, u32, vp, sz)
    sig("salt_gpu_weight_resource_unbind", i32, u32, u32)
    sig("salt_gpu_weight_window_bind", i32, u32, u32, u64, sz)
    sig("salt_gpu_weight_window_unbind", i32, u32, u32)
    sig("salt_gpu_weight_resource_slot", i32, u32, u32, vp, vp, vp, vp, i32, i32, i32)
    sig("salt_gpu_nvfp4_resource_slot", i32, u32, u32, vp, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_expert_resource_bind", i32, u32, vp, sz)
    sig("salt_gpu_expert_resource_slot", i32, u32, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_expert_resource_unbind", i32, u32)
    sig("salt_gpu_resident_slot", i32, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_shared_buffer_alloc", i32, C.POINTER(SharedBuffer), sz)
    sig("salt_gpu_shared_buffer_free", i32, C.POINTER(SharedBuffer))
    sig("salt_gpu_q4_matvec", i32, vp, vp, vp, i32, i32, vp, vp)
    sig("salt_gpu_q4_batch", i32, vp, vp, vp, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_proj_batch", i32, vp, vp, vp, i32, i32, i32, vp, vp, vp)
    sig("salt_gpu_proj_batch_indexed", i32, vp, vp, vp, i32, i32, i32, i32, i32, vp, C.POINTER(SharedBuffer), sz, vp)
    sig("salt_gpu_q4_moe_chain", i32, C.POINTER(MoeExpert), i32, i32, i32, vp, vp, vp, vp, sz)
    sig("salt_gpu_q4_moe_chain_selected", i32, C.POINTER(MoeExpert), i32, i32, i32, vp, vp, vp, vp, sz)
    sig("salt_gpu_q4_selected_shared", i32, C.POINTER(SelectedJob), i32, C.POINTER(SharedBuffer))
    sig("salt_gpu_selected_resources_prepare", i32, i32, i32)
    sig("salt_gpu_selected_resource_bind", i32, i32, u64, vp, sz, vp)
    sig("salt_gpu_selected_resource_bind_resident", i32, i32, u64, vp, sz, C.c_size_t, u64)
    sig("salt_gpu_selected_resource_unbind", i32, i32, u64)
    sig("salt_gpu_nvfp4_qdq", i32, vp, i32, f32, vp, vp, vp)
    sig("salt_gpu_nvfp4_matvec", i32, vp, i32, i32, vp, vp)
    sig("salt_gpu_nvfp4_matvec_batch", i32, vp, i32, i32, i32, vp, vp)
    sig("salt_gpu_nvfp4_batch", i32, vp, vp, vp, vp, i32, i32, i32)
    sig("salt_gpu_nvfp4_mixed_batch", i32, vp, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_residency_backend_ops", C.POINTER(ResidencyOps))
    sig("salt_gpu_q8_matvec", i32, vp, vp, vp, i32, i32, vp, vp)
    sig("salt_gpu_q8_batch", i32, vp, vp, vp, vp, vp, vp, vp, i32, i32)
    sig("salt_gpu_bf16_resource_slot", i32, u32, u32, vp, vp, i32, i32)
    sig("salt_gpu_bf16_matvec", i32, vp, i32, i32, vp, vp)
    sig("salt_gpu_bf16_matvec_batch", i32, vp, i32, i32, i32, vp, vp)
    sig("salt_gpu_exact_cells", i32, C.POINTER(ExactCell), i32)
    sig("salt_dispatch_get", vp)
    sig("salt_gpu_tensor_program_ops", vp)
    sig("salt_gpu_resident_trunk_map", i32, vp, sz)
    sig("salt_gpu_resident_pool_map", i32, vp, sz)
    return lib


def ptr_array(items):
    arr = (vp * len(items))()
    for k, a in enumerate(items):
        arr[k] = a if isinstance(a, int) or a is None else a.ctypes.data
    return arr
