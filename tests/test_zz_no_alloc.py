"""salt_mi355_moe_decode_step_static_dev: the MoE decode layer-step with the library's static workspace instead of a
caller-supplied one.  It must give the bits of salt_mi355_moe_decode_step_dev, call after call, also when a smaller
geometry follows a larger one in the same (shared) workspace."""
import numpy as np
import pytest

from golden import cases

pytestmark = pytest.mark.gpu
synth = cases.synth


def free_device_bytes():
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def run_both(pkg, E, K, H, F, pool_seed, logit_seed, x_seed, status_word=True):
    gpu = pkg.lib
    lib = gpu.init()
    pool = synth.expert_pool(E, H, F, pool_seed)
    layer = gpu.MoeLayer(pool, E, H, F, K)
    logits, scale = synth.router_logits(E, logit_seed), np.ones(E, np.float32)
    x = synth.activations(H, 1, x_seed)[0]
    want = layer.step(logits, scale, x)                                   # (status, sel, w, expert_out, out)
    sel, w = gpu.DeviceBuffer(K * 4, fill=0xEE), gpu.DeviceBuffer(K * 4, fill=0xEE)
    eo, out = gpu.DeviceBuffer(K * H * 4, fill=0xEE), gpu.DeviceBuffer(H * 4, fill=0xEE)
    status = gpu.DeviceBuffer(4, fill=0x7F)
    stream = lib.salt_mi355_stream()

    def call():
        rc = lib.salt_mi355_moe_decode_step_static_dev(layer.pool.at(0), layer.stride, H, F, E, K, layer.logits.ptr,
                                                       layer.scale.ptr, layer.x.ptr, sel.ptr, w.ptr, eo.ptr, out.ptr,
                                                       status.ptr if status_word else None, stream)
        assert rc == 0, lib.salt_mi355_last_error().decode()
        gpu.check(lib.salt_mi355_stream_sync(stream), "sync")

    call()                                                                # warm: code objects are loaded
    before = free_device_bytes()
    call()
    assert free_device_bytes() == before, "the static step changed the amount of free device memory"
    got = (int(status.to_host(np.int32)[0]) if status_word else 0, sel.to_host(np.int32), w.to_host(np.float32),
           eo.to_host(np.float32).reshape(K, H), out.to_host(np.float32))
    assert got[0] == want[0] == 0
    assert np.array_equal(got[1], want[1])
    for a, b in zip(got[2:], want[2:]):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_static_workspace_step_equals_the_workspace_step(pkg):
    print("static step: gemma geometry, 16 experts", flush=True)
    run_both(pkg, 16, 8, 2816, 704, 11, 611, 612)
    print("static step: a smaller geometry right after it", flush=True)
    run_both(pkg, 8, 3, 256, 128, 13, 615, 616)
    print("static step: five-launch plan (more experts than the router prologue holds)", flush=True)
    run_both(pkg, 520, 4, 128, 64, 14, 617, 618)
    print("static step: status word inside the static workspace", flush=True)
    run_both(pkg, 16, 8, 2816, 704, 15, 619, 620, status_word=False)


def test_static_workspace_step_refuses_what_does_not_fit(pkg):
    lib = pkg.lib.init()
    buf = pkg.lib.DeviceBuffer(1 << 12)
    # 64 selected experts of 8192 x 4096: far beyond the static workspace
    assert lib.salt_mi355_moe_workspace_bytes(8192, 4096, 128, 64) > (1 << 20)
    assert lib.salt_mi355_moe_decode_step_static_dev(buf.ptr, 1 << 30, 8192, 4096, 128, 64, buf.ptr, buf.ptr, buf.ptr,
                                                     buf.ptr, buf.ptr, None, buf.ptr, None, None) == -1
    assert b"static" in lib.salt_mi355_last_error()
