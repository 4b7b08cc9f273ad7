"""The C-ABI library loads without a GPU, exports every symbol its headers
declare and every backend symbol the reference's null backend defines, and
answers the GPU-free queries.  No compute call is made here."""
import ctypes as C
import re
import subprocess
from pathlib import Path

import pytest

import engine_abi as abi

ROOT = Path(__file__).resolve().parent.parent

# every symbol reference src/gpu_stub.c defines (the complete backend link surface)
REFERENCE_BACKEND_SYMBOLS = """
salt_dispatch_get salt_gpu_attention_batch salt_gpu_attention_bind_kv salt_gpu_attention_import
salt_gpu_attention_materialize salt_gpu_attention_prepare salt_gpu_attention_rewind salt_gpu_attention_transform
salt_gpu_batch_stats_get salt_gpu_batch_stats_get_v2 salt_gpu_bf16_matvec salt_gpu_bf16_matvec_batch
salt_gpu_bf16_resource_slot salt_gpu_cuda_present salt_gpu_defer salt_gpu_exact_cells salt_gpu_expert_resource_bind
salt_gpu_expert_resource_slot salt_gpu_expert_resource_unbind salt_gpu_free salt_gpu_init salt_gpu_mapped_only
salt_gpu_nvfp4_batch salt_gpu_nvfp4_matvec salt_gpu_nvfp4_matvec_batch salt_gpu_nvfp4_mixed_batch salt_gpu_nvfp4_qdq
salt_gpu_nvfp4_resource_slot salt_gpu_pageable_mmap_active salt_gpu_proj_batch salt_gpu_proj_batch_indexed
salt_gpu_proj_batch_indexed_exact_views salt_gpu_q4_batch salt_gpu_q4_matvec salt_gpu_q4_moe_chain
salt_gpu_q4_moe_chain_selected salt_gpu_q4_selected_shared salt_gpu_q8_batch salt_gpu_q8_matvec
salt_gpu_resident_pool_map salt_gpu_resident_slot salt_gpu_resident_trunk_map salt_gpu_resident_trunk_unmap
salt_gpu_residency_backend_ops salt_gpu_rocm_present salt_gpu_selected_resource_bind
salt_gpu_selected_resource_bind_resident salt_gpu_selected_resource_unbind salt_gpu_selected_resources_fence
salt_gpu_selected_resources_prepare salt_gpu_set_defer salt_gpu_set_mapped_only salt_gpu_shared_buffer_alloc
salt_gpu_shared_buffer_free salt_gpu_startup_requirements salt_gpu_sync salt_gpu_tensor_program_ops
salt_gpu_weight_resource_activate salt_gpu_weight_resource_bind salt_gpu_weight_resource_deactivate
salt_gpu_weight_resource_describe salt_gpu_weight_resource_pool_bind salt_gpu_weight_resource_slot
salt_gpu_weight_resource_unbind salt_gpu_weight_resource_usage salt_gpu_weight_window_bind
salt_gpu_weight_window_unbind
""".split()


@pytest.fixture(scope="module")
def lib(pkg):
    return abi.bind(pkg.lib.load())


def test_every_declared_symbol_is_exported(pkg, lib):
    names = pkg.lib.declared_symbols()
    assert len(names) > 80
    assert [n for n in names if not hasattr(lib, n)] == []


def test_every_reference_backend_symbol_is_exported(lib):
    assert [n for n in REFERENCE_BACKEND_SYMBOLS if not hasattr(lib, n)] == []
    stub = Path("/root/reference/src/gpu_stub.c")
    if stub.exists():       # the list above is the stub's definition list; re-derive it when the tree is mounted
        text = re.sub(r"/\*.*?\*/", " ", stub.read_text(), flags=re.S)
        found = set(re.findall(r"^(?:const\s+\w[\w\s\*]*?|int|void)\s*\*?\s*(salt_\w+)\s*\(", text, flags=re.M))
        assert found and found <= set(REFERENCE_BACKEND_SYMBOLS)


def test_library_has_no_cpu_fallback_dependencies():
    # the product must not link or load the CPU checker
    out = subprocess.check_output(["ldd", str(ROOT / "salt-core_amd" / "libsalt_gpu_mi355.so")], text=True)
    assert "oracle" not in out and "saltref" not in out and "amdhip64" in out


def test_gpu_free_queries(lib):
    req = abi.StartupRequirements()
    assert lib.salt_gpu_startup_requirements(C.byref(req), C.sizeof(req)) == 0
    assert req.max_output_floats == 4096 * 2816 and req.max_batch_jobs == 4096 and req.shared_buffer_slots == 8
    assert lib.salt_gpu_startup_requirements(C.byref(req), C.sizeof(req) - 1) == -1
    assert lib.salt_gpu_rocm_present() == 1 and lib.salt_gpu_cuda_present() == 0
    assert lib.salt_gpu_pageable_mmap_active() == 0
    lib.salt_gpu_set_mapped_only(5)
    assert lib.salt_gpu_mapped_only() == 1
    lib.salt_gpu_set_mapped_only(0)
    stats = abi.BatchStatsV2()
    assert lib.salt_gpu_batch_stats_get_v2(C.byref(stats), C.sizeof(stats)) == 0
    assert lib.salt_gpu_batch_stats_get_v2(C.byref(stats), 8) == -1
    ops = lib.salt_gpu_residency_backend_ops()
    assert ops.contents.abi_version == 1 and ops.contents.ops_size == C.sizeof(abi.ResidencyOps)
    assert lib.salt_dispatch_get() is None and lib.salt_gpu_tensor_program_ops() is None


def test_a_c99_translation_unit_consumes_both_headers(tmp_path):
    """The engine is C99: its compiler must accept the public headers as they are, and a C99 program linked against the
    library must get the documented answers to the GPU-free queries."""
    exe = tmp_path / "c99_consumer"
    libdir = ROOT / "salt-core_amd"
    # taking a function's address as a data pointer is the one thing -pedantic would flag in the consumer itself
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-Wno-pedantic",
                           "-I", str(ROOT / "include"), str(ROOT / "tests" / "c99_consumer.c"), "-o", str(exe),
                           "-L", str(libdir), "-lsalt_gpu_mi355", f"-Wl,-rpath,{libdir}"])
    for header in ("salt_gpu_mi355.h", "salt_gpu_mi355_engine.h"):
        subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c",
                               "-I", str(ROOT / "include"), str(ROOT / "include" / header)])
    out = subprocess.check_output([str(exe)], text=True)
    assert "c99 consumer ok" in out
