"""The engine-facing entry points (salt_gpu_*) driven the way the engine drives
its physical backend: host pointers in and out, weights named inside described
resources, expert seats filled through the residency operations.  Outputs are
compared bit-for-bit with the CPU checker."""
import ctypes as C

import numpy as np
import pytest

import engine_abi as abi
from golden import cases
from oracle_lib import ExpertGeometry, bits, host_threads, ptr

pytestmark = pytest.mark.gpu
synth = cases.synth
TRUNK, EXPERT_LAYER = 1, 2


@pytest.fixture(scope="module")
def eng(pkg):
    lib = abi.bind(pkg.lib.load())
    assert lib.salt_gpu_init() == 0 and lib.salt_gpu_init() == 0      # idempotent
    yield lib
    assert lib.salt_gpu_sync() == 0


def err(pkg):
    return pkg.lib.load().salt_mi355_last_error().decode()


def q4_want(oracle, vals, scales, biases, R, Cc, xs):
    xs = xs.reshape(-1, Cc)
    ys = np.zeros((xs.shape[0], R), np.float32)
    for t in range(xs.shape[0]):
        assert oracle.orc_q4_matvec_threads(ptr(vals), ptr(scales), ptr(biases), R, Cc, ptr(np.ascontiguousarray(xs[t])),
                                            ptr(ys[t]), host_threads()) == 0
    return ys


class Trunk:
    """Several Q4 tensors laid out back to back in one host byte range, the way
    a model file maps them."""

    def __init__(self, shapes, seed):
        parts, self.views = [], []
        at = 0
        for k, (R, Cc) in enumerate(shapes):
            vals, scales, biases = synth.q4_tensor(R, Cc, seed + k)
            offs = []
            for a in (vals, scales, biases):
                offs.append(at); parts.append(a.view(np.uint8)); at += a.nbytes
                pad = (-at) % 16
                parts.append(np.zeros(pad, np.uint8)); at += pad
            self.views.append((R, Cc, offs, vals, scales, biases))
        self.blob = np.concatenate(parts)
        self.base = self.blob.ctypes.data

    def pointers(self, k):
        R, Cc, offs, *_ = self.views[k]
        return self.base + offs[0], self.base + offs[1], self.base + offs[2]


def test_resource_lifecycle_matvec_batch_and_stats(eng, oracle, pkg):
    trunk = Trunk([(704, 2816), (2816, 704), (130, 2816)], 11)
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 7, trunk.base, trunk.blob.nbytes) == 0
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 7, trunk.base, trunk.blob.nbytes) == 0       # same again is fine
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 7, trunk.base, trunk.blob.nbytes - 1) == -1  # conflicting
    assert eng.salt_gpu_weight_resource_activate(TRUNK, 7, 3) == -1                                  # pageable refused
    assert eng.salt_gpu_weight_resource_activate(TRUNK, 7, 2) == 0, err(pkg)
    usage = abi.ResourceUsage()
    assert eng.salt_gpu_weight_resource_usage(C.byref(usage), C.sizeof(usage)) == 0
    assert usage.described_resources == 1 and usage.active_resources == 1
    assert usage.device_copied_weight_bytes == trunk.blob.nbytes == usage.registered_bytes
    keys = [0x1000 + k for k in range(3)]
    for k in range(3):
        R, Cc, *_ = trunk.views[k]
        v, s, b = trunk.pointers(k)
        assert eng.salt_gpu_weight_resource_slot(TRUNK, 7, keys[k], v, s, b, 4, R, Cc) == 0, err(pkg)
        assert eng.salt_gpu_weight_resource_slot(TRUNK, 7, keys[k], v, s, b, 4, R, Cc) == 0          # identical re-registration
    v0, s0, b0 = trunk.pointers(0)
    assert eng.salt_gpu_weight_resource_slot(TRUNK, 7, keys[0], v0 + 16, s0, b0, 4, 704, 2816) == -1  # conflicting key
    assert eng.salt_gpu_weight_resource_slot(TRUNK, 7, 0x2000, v0, s0, b0, 3, 704, 2816) == -1        # neither 4 nor 8 bits
    assert eng.salt_gpu_weight_resource_slot(TRUNK, 9, 0x2000, v0, s0, b0, 4, 704, 2816) == -1        # unknown resource
    assert eng.salt_gpu_weight_resource_slot(TRUNK, 7, 0x2000, v0, s0, b0, 4, 70400, 2816) == -1      # outside the range

    eng.salt_gpu_set_mapped_only(1)
    before = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(before))
    # one matvec by pointers that lie inside the active resource
    R, Cc, _, vals, scales, biases = trunk.views[0]
    x = synth.activations(Cc, 1, 5)[0]; y = np.full(R, np.nan, np.float32)
    assert eng.salt_gpu_q4_matvec(v0, s0, b0, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
    assert np.array_equal(bits(y), bits(q4_want(oracle, vals, scales, biases, R, Cc, x)[0]))
    # batch: two tensors sharing C = 2816, distinct inputs
    xs = synth.activations(2816, 2, 6)
    y0 = np.zeros(704, np.float32); y2 = np.zeros(130, np.float32)
    v2, s2, b2 = trunk.pointers(2)
    rc = eng.salt_gpu_q4_batch(abi.ptr_array([v0, v2]), abi.ptr_array([s0, s2]), abi.ptr_array([b0, b2]),
                               abi.ptr_array([xs[0], xs[1]]), abi.ptr_array([y0, y2]), abi.ptr_array(keys[0:3:2]),
                               (C.c_int * 2)(704, 130), 2816, 2)
    assert rc == 0, err(pkg)
    assert np.array_equal(bits(y0), bits(q4_want(oracle, *trunk.views[0][3:], 704, 2816, xs[0])[0]))
    assert np.array_equal(bits(y2), bits(q4_want(oracle, *trunk.views[2][3:], 130, 2816, xs[1])[0]))
    # a key that does not match the pointers it travels with is refused
    assert eng.salt_gpu_q4_batch(abi.ptr_array([v0]), abi.ptr_array([s0]), abi.ptr_array([b0]), abi.ptr_array([xs[0]]),
                                 abi.ptr_array([y0]), abi.ptr_array([keys[2]]), (C.c_int * 1)(704), 2816, 1) == -1
    # projection adapter: B = 6 contiguous tokens through the down-shaped tensor
    R, Cc, _, vals, scales, biases = trunk.views[1]
    v1, s1, b1 = trunk.pointers(1)
    xb = synth.activations(Cc, 6, 8); yb = np.zeros((6, R), np.float32)
    rc = eng.salt_gpu_proj_batch(v1, s1, b1, R, Cc, 6, abi.ptr_array([xb[t] for t in range(6)]),
                                 abi.ptr_array([yb[t] for t in range(6)]), keys[1])
    assert rc == 0, err(pkg)
    assert np.array_equal(bits(yb), bits(q4_want(oracle, vals, scales, biases, R, Cc, xb)))
    scattered = [xb[t] for t in (0, 2, 1, 3, 4, 5)]
    assert eng.salt_gpu_proj_batch(v1, s1, b1, R, Cc, 6, abi.ptr_array(scattered),
                                   abi.ptr_array([yb[t] for t in range(6)]), keys[1]) == -1
    after = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(after))
    assert after.trunk_batches == before.trunk_batches + 3 and after.arena_batches == before.arena_batches

    # weights outside any resource: refused under mapped-only (and counted), copied per call otherwise
    lv, ls, lb = synth.q4_tensor(64, 128, 3)
    lx = synth.activations(128, 1, 4)[0]; ly = np.zeros(64, np.float32)
    assert eng.salt_gpu_q4_matvec(ptr(lv), ptr(ls), ptr(lb), 64, 128, ptr(lx), ptr(ly)) == -1
    miss = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(miss))
    assert miss.mapped_only_misses == after.mapped_only_misses + 1
    eng.salt_gpu_set_mapped_only(0)
    assert eng.salt_gpu_q4_matvec(ptr(lv), ptr(ls), ptr(lb), 64, 128, ptr(lx), ptr(ly)) == 0, err(pkg)
    assert np.array_equal(bits(ly), bits(q4_want(oracle, lv, ls, lb, 64, 128, lx)[0]))
    assert eng.salt_gpu_q4_matvec(ptr(lv), ptr(ls), None, 64, 128, ptr(lx), ptr(ly)) == 0          # NULL biases
    assert np.array_equal(bits(ly), bits(q4_want(oracle, lv, ls, None, 64, 128, lx)[0]))
    legacy = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(legacy))
    assert legacy.arena_batches == miss.arena_batches + 2

    # deferred publication: outputs appear at salt_gpu_sync()
    assert eng.salt_gpu_set_defer(1) == 0 and eng.salt_gpu_defer() == 1
    R, Cc, _, vals, scales, biases = trunk.views[0]
    y = np.full(R, 7.0, np.float32)
    assert eng.salt_gpu_q4_matvec(v0, s0, b0, R, Cc, ptr(x), ptr(y)) == 0
    assert (y == 7.0).all()
    assert eng.salt_gpu_set_defer(0) == 0 and eng.salt_gpu_defer() == 0
    assert np.array_equal(bits(y), bits(q4_want(oracle, vals, scales, biases, R, Cc, x)[0]))

    assert eng.salt_gpu_weight_resource_deactivate(TRUNK, 7) == 0
    eng.salt_gpu_set_mapped_only(1)
    assert eng.salt_gpu_q4_matvec(v0, s0, b0, R, Cc, ptr(x), ptr(y)) == -1       # no longer resident
    eng.salt_gpu_set_mapped_only(0)
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, 7) == 0
    assert eng.salt_gpu_weight_resource_usage(C.byref(usage), C.sizeof(usage)) == 0
    assert usage.described_resources == 0 and usage.device_copied_weight_bytes == 0


def test_batch_of_unregistered_matrices_larger_than_one_copy_chunk(eng, oracle, pkg):
    """Three matrices outside every resource, 78 MB together: each is copied for the call, and the copy of the first
    must still be in place when the launch runs although the third does not fit the chunk that holds the first."""
    R, Cc = 16384, 2816
    eng.salt_gpu_set_mapped_only(0)
    tensors = [synth.q4_tensor(R, Cc, 300 + j) for j in range(3)]
    xs = synth.activations(Cc, 3, 310)
    ys = [np.zeros(R, np.float32) for _ in range(3)]
    rc = eng.salt_gpu_q4_batch(abi.ptr_array([t[0] for t in tensors]), abi.ptr_array([t[1] for t in tensors]),
                               abi.ptr_array([t[2] for t in tensors]), abi.ptr_array([xs[j] for j in range(3)]),
                               abi.ptr_array(ys), abi.ptr_array([t[0] for t in tensors]), (C.c_int * 3)(R, R, R), Cc, 3)
    assert rc == 0, err(pkg)
    for j, (vals, scales, biases) in enumerate(tensors):
        assert np.array_equal(bits(ys[j]), bits(q4_want(oracle, vals, scales, biases, R, Cc, xs[j])[0])), j
    # the next call starts over in the copy memory and still computes from its own weights
    lv, ls, lb = synth.q4_tensor(64, 128, 3)
    lx = synth.activations(128, 1, 4)[0]; ly = np.zeros(64, np.float32)
    assert eng.salt_gpu_q4_matvec(ptr(lv), ptr(ls), ptr(lb), 64, 128, ptr(lx), ptr(ly)) == 0, err(pkg)
    assert np.array_equal(bits(ly), bits(q4_want(oracle, lv, ls, lb, 64, 128, lx)[0]))


def test_bounded_window_and_expert_layer_resource(eng, oracle, pkg):
    trunk = Trunk([(128, 256), (64, 256)], 21)
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 3, trunk.base, trunk.blob.nbytes) == 0
    assert eng.salt_gpu_weight_resource_activate(TRUNK, 3, 1) == 0
    eng.salt_gpu_set_mapped_only(1)
    R, Cc, offs, vals, scales, biases = trunk.views[1]
    v, s, b = trunk.pointers(1)
    x = synth.activations(Cc, 1, 2)[0]; y = np.zeros(R, np.float32)
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == -1          # no window bound yet
    assert eng.salt_gpu_weight_window_bind(TRUNK, 3, offs[0], trunk.blob.nbytes - offs[0]) == 0, err(pkg)
    assert eng.salt_gpu_weight_window_bind(TRUNK, 3, 0, 64) == -1                # one window at a time
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
    assert np.array_equal(bits(y), bits(q4_want(oracle, vals, scales, biases, R, Cc, x)[0]))
    usage = abi.ResourceUsage()
    assert eng.salt_gpu_weight_resource_usage(C.byref(usage), C.sizeof(usage)) == 0
    assert usage.active_windows == 1 and usage.active_window_bytes == trunk.blob.nbytes - offs[0]
    assert eng.salt_gpu_weight_window_unbind(TRUNK, 3) == 0
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == -1
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, 3) == 0
    # command-scoped expert layer (reference src/gpu_layer.c:17-81): bind, slot, run, unbind
    layer = Trunk([(64, 128)], 31)
    assert eng.salt_gpu_expert_resource_bind(55, layer.base, layer.blob.nbytes) == 0
    v, s, b = layer.pointers(0)
    assert eng.salt_gpu_expert_resource_slot(55, 0xABC, v, s, b, 64, 128) == 0
    assert eng.salt_gpu_resident_slot(0xABD, v, s, b, 64, 128) == 0
    x = synth.activations(128, 1, 3)[0]; y = np.zeros(64, np.float32)
    before = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(before))
    assert eng.salt_gpu_q4_matvec(v, s, b, 64, 128, ptr(x), ptr(y)) == 0
    after = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(after))
    assert after.expert_layer_batches == before.expert_layer_batches + 1
    assert np.array_equal(bits(y), bits(q4_want(oracle, *layer.views[0][3:], 64, 128, x)[0]))
    assert eng.salt_gpu_expert_resource_unbind(55) == 0
    assert eng.salt_gpu_q4_matvec(v, s, b, 64, 128, ptr(x), ptr(y)) == -1
    eng.salt_gpu_set_mapped_only(0)


def expert_record(pool, e, H, F, group, slot=-1, logical=0):
    base = pool.ctypes.data + e * synth.expert_slot_bytes(H, F)
    proj = synth.expert_proj_bytes(H, F)
    n = H * F
    rec = abi.MoeExpert()
    for p, name in enumerate(("gate", "up", "down")):
        at = base + p * proj
        setattr(rec, name + "_vals", at)
        setattr(rec, name + "_scales", at + n // 2)
        setattr(rec, name + "_biases", at + n // 2 + (n // 64) * 2)
        setattr(rec, name + "_id", at)
    rec.group, rec.resource_slot, rec.logical_resource_id = group, slot, logical
    return rec


def chain_want(oracle, pool, H, F, experts, groups, inputs):
    g = ExpertGeometry(H, F)
    slot = synth.expert_slot_bytes(H, F)
    out = np.zeros_like(inputs)
    row = 0
    for e, n in zip(experts, groups):
        for _ in range(n):
            gate = np.zeros(F, np.float32); up = np.zeros(F, np.float32)
            assert oracle.orc_expert_ffn(C.byref(g), ptr(pool[e * slot:]), ptr(inputs[row]), ptr(gate), ptr(up),
                                         ptr(out[row])) == 0
            row += 1
    return out


def test_moe_chain_from_a_layer_resource(eng, oracle, pkg):
    E, H, F = 6, 256, 128
    pool = synth.expert_pool(E, H, F, 41)
    assert eng.salt_gpu_expert_resource_bind(9, pool.ctypes.data, pool.nbytes) == 0, err(pkg)
    experts, groups = [1, 3, 4], [2, 5, 1]              # prefill-shaped: several rows per expert
    recs = (abi.MoeExpert * 3)(*[expert_record(pool, e, H, F, n) for e, n in zip(experts, groups)])
    rows = sum(groups)
    inputs = synth.activations(H, rows, 42); outputs = np.zeros((rows, H), np.float32)
    scratch = np.zeros((2, rows * F), np.float32)
    eng.salt_gpu_set_mapped_only(1)
    rc = eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(inputs), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), rows * F)
    assert rc == 0, err(pkg)
    assert np.array_equal(bits(outputs), bits(chain_want(oracle, pool, H, F, experts, groups, inputs)))
    # rejected: too little scratch, zero-row expert, not resident
    assert eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(inputs), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), rows * F - 1) == -1
    recs[1].group = 0
    assert eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(inputs), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), rows * F) == -1
    recs[1].group = 5
    assert eng.salt_gpu_expert_resource_unbind(9) == 0
    assert eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(inputs), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), rows * F) == -1
    eng.salt_gpu_set_mapped_only(0)


def test_tolerance_class_policy_reaches_the_engine_entry_points(eng, oracle, pkg):
    """salt_mi355_set_tolerance_class(1): salt_gpu_q4_matvec and the decode-shaped salt_gpu_q4_moe_chain run the
    tolerance-class kernels (salt_mi355_last_kernel says so) inside their stated bounds; switched off again, the same
    calls are bit-identical to the CPU checker."""
    from moe_bounds import down_term_magnitudes, expert_activation
    from q4_bounds import check as check_class_t
    lib = pkg.lib.load()
    trunk = Trunk([(704, 2816)], 21)
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 17, trunk.base, trunk.blob.nbytes) == 0
    assert eng.salt_gpu_weight_resource_activate(TRUNK, 17, 2) == 0, err(pkg)
    R, Cc, _, vals, scales, biases = trunk.views[0]
    v0, s0, b0 = trunk.pointers(0)
    x = synth.activations(Cc, 1, 22)[0]
    want = q4_want(oracle, vals, scales, biases, R, Cc, x)
    E, H, F = 8, 2816, 704
    pool = synth.expert_pool(E, H, F, 23)
    assert eng.salt_gpu_expert_resource_bind(19, pool.ctypes.data, pool.nbytes) == 0, err(pkg)
    experts = [1, 4, 6]
    recs = (abi.MoeExpert * 3)(*[expert_record(pool, e, H, F, 1) for e in experts])
    xin = np.tile(synth.activations(H, 1, 24)[0], (3, 1)); outputs = np.zeros((3, H), np.float32)
    scratch = np.zeros((2, 3 * F), np.float32)
    chain = chain_want(oracle, pool, H, F, experts, [1, 1, 1], xin)

    assert lib.salt_mi355_set_tolerance_class(1) == 0
    y = np.zeros(R, np.float32)
    assert eng.salt_gpu_q4_matvec(v0, s0, b0, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
    assert lib.salt_mi355_last_kernel().decode().startswith("q4_dot")
    check_class_t(y[None, :], want, vals, scales, biases, R, Cc, x[None, :])
    assert eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(xin), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), 3 * F) == 0, err(pkg)
    assert lib.salt_mi355_last_kernel().decode().startswith("q4_dot")
    for i, e in enumerate(experts):
        terms = down_term_magnitudes(pool, e, expert_activation(pool, e, xin[i:i + 1], H, F), H, F)[0]
        assert (np.abs(outputs[i].astype(np.float64) - chain[i]) <= 2.0 ** -18 * terms + 1e-6).all()

    assert lib.salt_mi355_set_tolerance_class(0) == 1
    assert eng.salt_gpu_q4_matvec(v0, s0, b0, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
    assert np.array_equal(bits(y), bits(want[0]))
    assert eng.salt_gpu_q4_moe_chain(recs, 3, H, F, ptr(xin), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]), 3 * F) == 0, err(pkg)
    assert np.array_equal(bits(outputs), bits(chain))
    assert eng.salt_gpu_expert_resource_unbind(19) == 0
    assert eng.salt_gpu_weight_resource_deactivate(TRUNK, 17) == 0 and eng.salt_gpu_weight_resource_unbind(TRUNK, 17) == 0


def test_moe_chain_from_a_pool_file_image(eng, oracle, pkg):
    """The engine's expert pool file: three 64-bit header words {slot bytes, layers, experts}, then the slots
    (reference gemma4_text.c:73-79, 1618-1623).  The whole image is one resource; every tensor in it sits 8 bytes past a
    multiple of 16 and must still be served by the tiled kernels, bit for bit."""
    import time
    E, H, F = 8, 2816, 704
    slots = synth.expert_pool(E, H, F, 43)
    slot_bytes = synth.expert_slot_bytes(H, F)
    image = np.zeros(24 + slots.nbytes, np.uint8)
    image[:24] = np.array([slot_bytes, 1, E], np.uint64).view(np.uint8)
    image[24:] = slots
    pool = image[24:]                                   # expert 0; a view, so the addresses lie inside the image
    assert pool.ctypes.data % 16 == 8 or image.ctypes.data % 16 != 0
    assert eng.salt_gpu_expert_resource_bind(10, image.ctypes.data, image.nbytes) == 0, err(pkg)
    experts, groups = [0, 2, 5, 7], [1, 1, 1, 1]
    recs = (abi.MoeExpert * 4)(*[expert_record(pool, e, H, F, n) for e, n in zip(experts, groups)])
    rows = sum(groups)
    inputs = synth.activations(H, rows, 44); outputs = np.zeros((rows, H), np.float32)
    scratch = np.zeros((2, rows * F), np.float32)
    eng.salt_gpu_set_mapped_only(1)
    call = lambda: eng.salt_gpu_q4_moe_chain(recs, 4, H, F, ptr(inputs), ptr(outputs), ptr(scratch[0]), ptr(scratch[1]),
                                             rows * F)
    assert call() == 0, err(pkg)
    assert np.array_equal(bits(outputs), bits(chain_want(oracle, slots, H, F, experts, groups, inputs)))
    t0 = time.perf_counter()
    for _ in range(20):
        assert call() == 0
    per_call_us = (time.perf_counter() - t0) / 20 * 1e6
    print(f"moe chain from a pool-file image: {per_call_us:.0f} us per call", flush=True)
    assert per_call_us < 2000                           # the per-row kernel for unaligned tensors needs several ms here
    eng.salt_gpu_set_mapped_only(0)
    assert eng.salt_gpu_expert_resource_unbind(10) == 0


def shared_array(eng, nfloats):
    buf = abi.SharedBuffer()
    assert eng.salt_gpu_shared_buffer_alloc(C.byref(buf), nfloats * 4) == 0
    assert buf.contents and buf.backend and buf.nbytes == nfloats * 4
    arr = np.ctypeslib.as_array(C.cast(buf.contents, C.POINTER(C.c_float)), shape=(nfloats,))
    return buf, arr


def test_expert_seats_through_residency_and_selected_chain(eng, oracle, pkg):
    E, H, F, K = 8, 256, 128, 3
    pool = synth.expert_pool(E, H, F, 51)
    slot_bytes = synth.expert_slot_bytes(H, F)
    ops = eng.salt_gpu_residency_backend_ops().contents
    seats, staging_count = 4, 2
    plan = abi.ResidencyPlan(4096 + seats * slot_bytes, 0, 4096, slot_bytes, slot_bytes, seats, staging_count, 256, 0)
    assert ops.create(None, C.byref(plan)) == 0, err(pkg)
    assert ops.create(None, C.byref(plan)) == -1                      # one arena at a time
    assert eng.salt_gpu_free() == -1                                  # refused while residency is live
    layout = abi.PermanentLayout()
    assert ops.permanent_layout(None, C.byref(layout), C.sizeof(layout)) == -1     # no pool-bound resource: no spans
    assert eng.salt_gpu_selected_resources_prepare(seats, 30 * 128) == 0
    assert eng.salt_gpu_selected_resources_prepare(seats, 30 * 128) == 0
    assert eng.salt_gpu_selected_resources_prepare(seats + 1, 30 * 128) == -1

    chosen = [5, 0, 6]                       # experts placed in seats 0, 1, 2
    layer = 2
    addresses = []
    for seat, e in enumerate(chosen):
        staging, cap = C.c_void_p(), C.c_size_t()
        st_slot = seat % staging_count
        assert ops.staging(None, st_slot, C.byref(staging), C.byref(cap)) == 0 and cap.value >= slot_bytes
        C.memmove(staging.value, pool.ctypes.data + e * slot_bytes, slot_bytes)   # the engine's read callback
        offset = plan.slot_base_offset + seat * slot_bytes
        ticket = 100 + seat
        assert ops.populate(None, seat, offset + 1, st_slot, slot_bytes, ticket) == -1      # wrong offset
        assert ops.populate(None, seat, offset, st_slot, slot_bytes, 0) == -1               # ticket 0
        assert ops.populate(None, seat, offset, st_slot, slot_bytes, ticket) == 0, err(pkg)
        assert ops.populate(None, seat, offset, st_slot, slot_bytes, ticket + 50) == -1     # seat busy
        done = C.c_int(0)
        assert ops.poll(None, seat, ticket + 1, C.byref(done)) == -1                        # stale ticket
        for _ in range(100000):
            assert ops.poll(None, seat, ticket, C.byref(done)) == 0
            if done.value:
                break
        assert done.value == 1
        assert ops.poll(None, seat, ticket, C.byref(done)) == -1                            # already published
        addr = C.c_size_t()
        assert ops.resolve(None, offset, slot_bytes, C.byref(addr)) == 0 and addr.value
        assert ops.resolve(None, plan.device_budget_bytes, 1, C.byref(addr)) == -1
        assert ops.resolve(None, offset, slot_bytes, C.byref(addr)) == 0
        addresses.append(addr.value)
        logical = layer * 128 + e
        payload = pool.ctypes.data + e * slot_bytes
        assert eng.salt_gpu_selected_resource_bind_resident(seat, logical, payload, slot_bytes, 12345, 1) == -1
        assert eng.salt_gpu_selected_resource_bind_resident(seat, logical, payload, slot_bytes, addr.value, 1) == 0, err(pkg)
        assert eng.salt_gpu_selected_resource_bind_resident(seat, logical, payload, slot_bytes, addr.value, 1) == 0
        assert eng.salt_gpu_selected_resource_bind_resident(seat, logical + 1, payload, slot_bytes, addr.value, 1) == -1

    # decode-shaped selected chain: one row per expert, ascending expert order, all four buffers shared
    order = sorted(range(K), key=lambda i: chosen[i])
    recs = (abi.MoeExpert * K)(*[expert_record(pool, chosen[i], H, F, 1, slot=i, logical=layer * 128 + chosen[i])
                                 for i in order])
    bin_, ain = shared_array(eng, K * H); bout, aout = shared_array(eng, K * H)
    bg, _ = shared_array(eng, K * F); bu, _ = shared_array(eng, K * F)
    x = synth.activations(H, 1, 52)[0]
    ain[:] = np.tile(x, K)
    eng.salt_gpu_set_mapped_only(1)
    rc = eng.salt_gpu_q4_moe_chain_selected(recs, K, H, F, bin_.contents, bout.contents, bg.contents, bu.contents, K * F)
    assert rc == 0, err(pkg)
    want = chain_want(oracle, pool, H, F, [chosen[i] for i in order], [1] * K, np.tile(x, (K, 1)))
    assert np.array_equal(bits(aout.reshape(K, H)), bits(want))
    # deferred mode: the device reads the shared inputs where they lie and the outputs are published by sync, so the
    # caller leaves the inputs alone until then
    x2 = synth.activations(H, 1, 54)[0]
    ain[:] = np.tile(x2, K)
    aout[:] = -1.0
    assert eng.salt_gpu_set_defer(1) == 0
    assert eng.salt_gpu_q4_moe_chain_selected(recs, K, H, F, bin_.contents, bout.contents, bg.contents, bu.contents, K * F) == 0, err(pkg)
    assert eng.salt_gpu_sync() == 0
    assert np.array_equal(bits(aout.reshape(K, H)),
                          bits(chain_want(oracle, pool, H, F, [chosen[i] for i in order], [1] * K, np.tile(x2, (K, 1)))))
    assert eng.salt_gpu_set_defer(0) == 0
    ain[:] = np.tile(x, K)
    # plain host memory instead of shared buffers is refused
    plain = np.zeros(K * H, np.float32)
    assert eng.salt_gpu_q4_moe_chain_selected(recs, K, H, F, ptr(plain), bout.contents, bg.contents, bu.contents, K * F) == -1
    # a seat that holds another expert is refused
    recs[0].logical_resource_id += 1
    assert eng.salt_gpu_q4_moe_chain_selected(recs, K, H, F, bin_.contents, bout.contents, bg.contents, bu.contents, K * F) == -1
    recs[0].logical_resource_id -= 1

    # heterogeneous projections inside one shared arena (reference gpu.h:311-316)
    arena, aa = shared_array(eng, 4 * H + 4 * F)
    aa[:H] = x; aa[H:2 * H] = x * 2
    jobs = (abi.SelectedJob * 2)()
    for j, i in enumerate(order[:2]):
        r = recs[j]
        jobs[j] = abi.SelectedJob(r.gate_vals, r.gate_scales, r.gate_biases, r.gate_id, arena.contents + j * H * 4,
                                  arena.contents + (2 * H + j * F) * 4, F, H, 1, r.resource_slot, r.logical_resource_id)
    assert eng.salt_gpu_q4_selected_shared(jobs, 2, C.byref(arena)) == 0, err(pkg)
    for j, i in enumerate(order[:2]):
        gv = synth.expert_views(pool, chosen[i], 0, H, F)
        assert np.array_equal(bits(aa[2 * H + j * F:2 * H + (j + 1) * F]),
                              bits(q4_want(oracle, gv[0], gv[1], gv[2], F, H, aa[j * H:(j + 1) * H].copy())[0]))
    jobs[1].outputs = jobs[0].outputs                                  # overlapping outputs
    assert eng.salt_gpu_q4_selected_shared(jobs, 2, C.byref(arena)) == -1

    # asynchronous indexed projection straight into a shared buffer, published by sync
    gv = synth.expert_views(pool, chosen[0], 0, H, F)
    r0 = expert_record(pool, chosen[0], H, F, 1)
    xb = synth.activations(H, 5, 53)
    dest, adest = shared_array(eng, 16 + 5 * F)
    adest[:] = -1.0
    assert eng.salt_gpu_proj_batch_indexed(r0.gate_vals, r0.gate_scales, r0.gate_biases, F, H, 5, 1, 3, ptr(xb),
                                           C.byref(dest), 16, r0.gate_id) == 0, err(pkg)
    assert eng.salt_gpu_sync() == 0
    want = q4_want(oracle, gv[0], gv[1], gv[2], F, H, xb)
    got = adest[16:].reshape(5, F)
    assert np.array_equal(bits(got[1:4]), bits(want[1:4])) and (got[0] == -1).all() and (got[4] == -1).all()
    assert eng.salt_gpu_proj_batch_indexed(r0.gate_vals, r0.gate_scales, r0.gate_biases, F, H, 5, 4, 3, ptr(xb),
                                           C.byref(dest), 16, r0.gate_id) == -1
    stats = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(stats))
    assert stats.direct_output_batches >= 1 and stats.direct_output_jobs >= 3
    eng.salt_gpu_set_mapped_only(0)

    # eviction: fence, unbind, retire, then the seat can be populated again
    assert eng.salt_gpu_selected_resources_fence() == 0
    for seat, e in enumerate(chosen):
        assert eng.salt_gpu_selected_resource_unbind(seat, layer * 128 + e + 1) == -1
        assert eng.salt_gpu_selected_resource_unbind(seat, layer * 128 + e) == 0
        assert eng.salt_gpu_selected_resource_unbind(seat, layer * 128 + e) == 0      # inactive seat: fine
        assert ops.retire(None, seat, 1) == 0
    # plain (non-resident) bind copies the payload itself
    payload = pool.ctypes.data + 2 * slot_bytes
    assert eng.salt_gpu_selected_resource_bind(3, 77, pool.ctypes.data, pool.nbytes, payload) == 0, err(pkg)
    assert eng.salt_gpu_selected_resource_bind(3, 77, pool.ctypes.data, pool.nbytes, payload) == 0
    assert eng.salt_gpu_selected_resource_bind(3, 78, pool.ctypes.data, pool.nbytes, payload) == -1
    rec = (abi.MoeExpert * 1)(expert_record(pool, 2, H, F, 1, slot=3, logical=77))
    ain[:H] = x
    assert eng.salt_gpu_q4_moe_chain_selected(rec, 1, H, F, bin_.contents, bout.contents, bg.contents, bu.contents, F) == 0, err(pkg)
    assert np.array_equal(bits(aout[:H]), bits(chain_want(oracle, pool, H, F, [2], [1], x[None, :])[0]))
    assert eng.salt_gpu_selected_resource_unbind(3, 77) == 0
    for b in (bin_, bout, bg, bu, arena, dest):
        assert eng.salt_gpu_shared_buffer_free(C.byref(b)) == 0 and not b.contents
    assert ops.destroy(None) == 0
    assert ops.destroy(None) == -1


def test_component_pool_without_and_with_permanent_spans(eng, oracle, pkg):
    """A pool-bound resource (reference gpu_hip.cpp:4208-4217): only the bytes its tensors occupy become resident,
    at the first sync when no residency arena runs, as permanent spans of the arena when one does
    (reference gpu_hip.cpp:3429-3571, gpu_residency.c:334-406)."""
    shapes = [(128, 256), (64, 256), (96, 512)]
    trunk = Trunk(shapes, 61)
    gap = 3 * 4096 + 40                                   # unrelated bytes ahead of the tensors and between two of them
    first = trunk.views[2][2][0]                          # offset of the third tensor: the gap goes in front of it
    image = np.concatenate([np.full(gap, 0xA5, np.uint8), trunk.blob[:first], np.full(5 * 4096, 0x5A, np.uint8),
                            trunk.blob[first:]])
    def pointers(k):
        offs = trunk.views[k][2]
        return [image.ctypes.data + gap + o + (5 * 4096 if k == 2 else 0) for o in offs]
    TR = 7
    assert eng.salt_gpu_weight_resource_describe(TRUNK, TR, image.ctypes.data, image.nbytes) == 0
    assert eng.salt_gpu_weight_resource_pool_bind(TRUNK, TR) == -1                  # not active
    assert eng.salt_gpu_weight_resource_activate(TRUNK, TR, 1) == 0
    assert eng.salt_gpu_weight_resource_pool_bind(TRUNK, TR) == 0, err(pkg)
    assert eng.salt_gpu_weight_resource_pool_bind(TRUNK, TR) == -1                  # once
    assert eng.salt_gpu_weight_window_bind(TRUNK, TR, 0, 4096) == -1                # no windows into a pool
    for k, (R, Cc) in enumerate(shapes):
        v, s, b = pointers(k)
        assert eng.salt_gpu_weight_resource_slot(TRUNK, TR, v, v, s, b, 4, R, Cc) == 0, err(pkg)
    eng.salt_gpu_set_mapped_only(1)

    def check_all():
        for k, (R, Cc) in enumerate(shapes):
            v, s, b = pointers(k)
            x = synth.activations(Cc, 1, 70 + k)[0]; y = np.zeros(R, np.float32)
            assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
            assert np.array_equal(bits(y), bits(q4_want(oracle, *trunk.views[k][3:], R, Cc, x)[0]))

    # 1. no arena: resident from the first sync on
    v, s, b = pointers(0)
    x = synth.activations(256, 1, 1)[0]; y = np.zeros(128, np.float32)
    assert eng.salt_gpu_q4_matvec(v, s, b, 128, 256, ptr(x), ptr(y)) == -1          # nothing resident before the sync
    assert eng.salt_gpu_sync() == 0, err(pkg)
    check_all()
    usage = abi.ResourceUsage()
    assert eng.salt_gpu_weight_resource_usage(C.byref(usage), C.sizeof(usage)) == 0
    tensor_bytes = sum(a.nbytes for view in trunk.views for a in view[3:])
    assert usage.active_windows >= 1 and tensor_bytes <= usage.active_window_bytes < image.nbytes - 4 * 4096
    # a tensor registered after the pool became resident must lie inside it
    assert eng.salt_gpu_weight_resource_slot(TRUNK, TR, image.ctypes.data + gap + first + 4096,
                                             image.ctypes.data + gap + first + 4096, image.ctypes.data + gap + first + 8192,
                                             image.ctypes.data + gap + first + 8192 + 64, 4, 8, 64) == -1
    assert eng.salt_gpu_weight_resource_deactivate(TRUNK, TR) == 0
    assert eng.salt_gpu_q4_matvec(v, s, b, 128, 256, ptr(x), ptr(y)) == -1

    # 2. with an arena: the same regions as permanent spans, copied through staging in chunks
    assert eng.salt_gpu_weight_resource_activate(TRUNK, TR, 1) == 0
    assert eng.salt_gpu_weight_resource_pool_bind(TRUNK, TR) == 0, err(pkg)
    ops = eng.salt_gpu_residency_backend_ops().contents
    layout = abi.PermanentLayout()
    assert ops.permanent_layout(None, C.byref(layout), C.sizeof(layout)) == 0, err(pkg)
    assert layout.span_count == 2 and layout.alignment == 256
    assert layout.maximum_span_bytes <= layout.permanent_bytes < image.nbytes - 4 * 4096
    assert eng.salt_gpu_weight_resource_pool_bind(TRUNK, TR) == -1
    staging_bytes, seat_bytes = 16384, 8192
    base = (layout.permanent_bytes + 255) // 256 * 256
    plan = abi.ResidencyPlan(base + 2 * seat_bytes, layout.permanent_bytes, base, seat_bytes, staging_bytes, 2, 2, 256, 0)
    assert ops.create(None, C.byref(plan)) == 0, err(pkg)
    assert eng.salt_gpu_sync() == 0                                                 # does not make the pool resident by itself
    assert eng.salt_gpu_q4_matvec(v, s, b, 128, 256, ptr(x), ptr(y)) == -1
    assert ops.permanent_publish(None) == -1                                        # nothing populated yet
    ticket = 0
    previous_end = 0
    for index in range(layout.span_count):
        span = abi.PermanentSpan()
        assert ops.permanent_span(None, index, C.byref(span), C.sizeof(span)) == 0
        assert span.kind == TRUNK and span.resource_id == TR and span.device_offset % 256 == 0
        assert span.device_offset >= previous_end and span.source_offset % 4096 == 0
        previous_end = span.device_offset + span.nbytes
        done = 0
        while done < span.nbytes:
            st = ticket % 2
            address, capacity = C.c_void_p(), C.c_size_t()
            assert ops.staging(None, st, C.byref(address), C.byref(capacity)) == 0 and capacity.value == staging_bytes
            chunk = min(capacity.value, span.nbytes - done)
            assert span.read(span.read_context, span.source_offset + done, address, chunk) == 0
            assert span.read(span.read_context, span.source_offset + span.nbytes, address, 1) == -1
            ticket += 1
            if done == 0:
                assert ops.permanent_copy(None, index, span.device_offset + 256, st, chunk, ticket) == -1   # out of order
                assert ops.permanent_copy(None, index, span.device_offset, st, chunk, 0) == -1             # ticket 0
            assert ops.permanent_copy(None, index, span.device_offset + done, st, chunk, ticket) == 0, err(pkg)
            done += chunk
            if index == 0 and done >= span.nbytes:
                assert ops.permanent_publish(None) == -1                            # the second span is still empty
    span = abi.PermanentSpan()
    assert ops.permanent_span(None, layout.span_count, C.byref(span), C.sizeof(span)) == -1
    assert ops.permanent_publish(None) == 0, err(pkg)
    assert ops.permanent_publish(None) == -1
    assert ops.permanent_layout(None, C.byref(layout), C.sizeof(layout)) == -1      # resident: the layout is closed
    check_all()
    assert eng.salt_gpu_weight_resource_usage(C.byref(usage), C.sizeof(usage)) == 0
    assert usage.device_copied_weight_bytes >= tensor_bytes and usage.active_window_bytes == 0
    assert ops.destroy(None) == 0
    assert eng.salt_gpu_q4_matvec(v, s, b, 128, 256, ptr(x), ptr(y)) == -1          # the spans left with the arena
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, TR) == 0
    eng.salt_gpu_set_mapped_only(0)


def test_nvfp4_engine_entry_points(eng, oracle, pkg):
    R, Cc = 96, 2816
    packed, scales = synth.nvfp4_tensor(R, Cc, 61)
    globals_ = np.array([2688.0, 64.0], np.float32)          # stored divisor, input global scale
    blob = np.concatenate([packed, scales, globals_.view(np.uint8)])
    base = blob.ctypes.data
    assert eng.salt_gpu_weight_resource_bind(TRUNK, 12, base, blob.nbytes) == 0, err(pkg)
    key = 0x7777
    wg, ig = base + packed.nbytes + scales.nbytes, base + packed.nbytes + scales.nbytes + 4
    assert eng.salt_gpu_nvfp4_resource_slot(TRUNK, 12, key, base, base + packed.nbytes, wg, ig, R, Cc) == 0, err(pkg)
    assert eng.salt_gpu_nvfp4_resource_slot(TRUNK, 12, key, base, base + packed.nbytes, wg, ig, R, Cc + 32) == -1

    def want(xs):
        out = np.zeros((xs.shape[0], R), np.float32)
        for t in range(xs.shape[0]):
            s = (np.zeros(Cc // 2, np.uint8), np.zeros(Cc // 16, np.uint8), np.zeros(Cc, np.float32))
            assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), 2688.0, 64.0, R, Cc, ptr(xs[t]), ptr(out[t]),
                                           ptr(s[0]), ptr(s[1]), ptr(s[2])) == 0
        return out

    xs = synth.activations(Cc, 5, 62)
    bad_row = xs[0:1].copy(); bad_row[0, 5] = np.nan
    y = np.zeros(R, np.float32)
    assert eng.salt_gpu_nvfp4_matvec(key, R, Cc, ptr(xs[0]), ptr(y)) == 0, err(pkg)
    assert np.array_equal(bits(y), bits(want(xs[:1])[0]))
    yb = np.zeros((5, R), np.float32)
    assert eng.salt_gpu_nvfp4_matvec_batch(key, R, Cc, 5, ptr(xs), ptr(yb)) == 0, err(pkg)
    assert np.array_equal(bits(yb), bits(want(xs)))
    y1 = np.zeros((2, R), np.float32); y2 = np.zeros((1, R), np.float32)
    rc = eng.salt_gpu_nvfp4_batch(abi.ptr_array([key, key]), abi.ptr_array([xs[0:2], xs[4:5]]),
                                  abi.ptr_array([y1, y2]), (C.c_int * 2)(2, 1), R, Cc, 2)
    assert rc == 0, err(pkg)
    assert np.array_equal(bits(y1), bits(want(xs[0:2]))) and np.array_equal(bits(y2), bits(want(xs[4:5])))
    # three single-token jobs: one multi-matrix launch behind the same entry point
    ys3 = [np.zeros((1, R), np.float32) for _ in range(3)]
    rc = eng.salt_gpu_nvfp4_batch(abi.ptr_array([key, key, key]), abi.ptr_array([xs[1:2], xs[3:4], xs[2:3]]),
                                  abi.ptr_array(ys3), (C.c_int * 3)(1, 1, 1), R, Cc, 3)
    assert rc == 0, err(pkg)
    for got, t in zip(ys3, (1, 3, 2)):
        assert np.array_equal(bits(got), bits(want(xs[t:t + 1])))
    ys3[1][:] = 5.0
    rc = eng.salt_gpu_nvfp4_batch(abi.ptr_array([key, key, key]), abi.ptr_array([xs[1:2], bad_row, xs[2:3]]),
                                  abi.ptr_array(ys3), (C.c_int * 3)(1, 1, 1), R, Cc, 3)
    assert rc == -1 and (ys3[1] == 5.0).all()                                            # nothing published
    assert eng.salt_gpu_nvfp4_matvec(0x9999, R, Cc, ptr(xs[0]), ptr(y)) == -1            # unknown key
    assert eng.salt_gpu_nvfp4_matvec(key, R + 1, Cc, ptr(xs[0]), ptr(y)) == -1           # geometry mismatch
    bad = xs[0].copy(); bad[17] = np.inf
    y[:] = 3.0
    assert eng.salt_gpu_nvfp4_matvec(key, R, Cc, ptr(bad), ptr(y)) == -1 and (y == 3.0).all()
    stats = abi.BatchStatsV2()
    assert eng.salt_gpu_batch_stats_get_v2(C.byref(stats), C.sizeof(stats)) == 0
    assert stats.nvfp4_logical_packed_weight_bytes >= 3 * R * Cc // 2 and stats.nvfp4_completion_fences >= 3
    # stand-alone activation Q/DQ
    p = np.zeros(Cc // 2, np.uint8); s = np.zeros(Cc // 16, np.uint8); d = np.zeros(Cc, np.float32)
    assert eng.salt_gpu_nvfp4_qdq(ptr(xs[1]), Cc, 64.0, ptr(p), ptr(s), ptr(d)) == 0, err(pkg)
    op = np.zeros_like(p); os_ = np.zeros_like(s); od = np.zeros_like(d)
    assert oracle.orc_nvfp4_qdq(ptr(xs[1]), Cc, 64.0, ptr(op), ptr(os_), ptr(od)) == 0
    assert np.array_equal(p, op) and np.array_equal(s, os_) and np.array_equal(bits(d), bits(od))
    assert eng.salt_gpu_nvfp4_qdq(ptr(bad), Cc, 64.0, ptr(p), ptr(s), ptr(d)) == -1
    assert eng.salt_gpu_nvfp4_qdq(ptr(xs[1]), Cc, -1.0, ptr(p), ptr(s), ptr(d)) == -1
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, 12) == 0
    assert eng.salt_gpu_nvfp4_matvec(key, R, Cc, ptr(xs[0]), ptr(y)) == -1


def test_nvfp4_mixed_batch_of_two_tensors(eng, oracle, pkg):
    """salt_gpu_nvfp4_mixed_batch (reference gpu.h:56-59): jobs on tensors of different heights that share the column
    count, several tokens per job, one call."""
    Cc = 1024
    shapes = [96, 200]
    tensors = [synth.nvfp4_tensor(R, Cc, 300 + R) for R in shapes]
    globals_ = [np.array([2688.0, 64.0], np.float32), np.array([0.37, 64.0], np.float32)]
    parts, at, offs = [], 0, []
    for (packed, scales), g in zip(tensors, globals_):
        o = []
        for a in (packed, scales, g.view(np.uint8)):
            o.append(at); parts.append(a.view(np.uint8)); at += a.nbytes
            pad = (-at) % 16; parts.append(np.zeros(pad, np.uint8)); at += pad
        offs.append(o)
    blob = np.concatenate(parts); base = blob.ctypes.data
    assert eng.salt_gpu_weight_resource_bind(TRUNK, 13, base, blob.nbytes) == 0, err(pkg)
    keys = [0x8801, 0x8802]
    for k, (R, o) in enumerate(zip(shapes, offs)):
        assert eng.salt_gpu_nvfp4_resource_slot(TRUNK, 13, keys[k], base + o[0], base + o[1], base + o[2], base + o[2] + 4,
                                                R, Cc) == 0, err(pkg)

    def want(k, xs):
        packed, scales = tensors[k]
        out = np.zeros((xs.shape[0], shapes[k]), np.float32)
        for t in range(xs.shape[0]):
            s = (np.zeros(Cc // 2, np.uint8), np.zeros(Cc // 16, np.uint8), np.zeros(Cc, np.float32))
            assert oracle.orc_nvfp4_matvec(ptr(packed), ptr(scales), float(globals_[k][0]), 64.0, shapes[k], Cc,
                                           ptr(np.ascontiguousarray(xs[t])), ptr(out[t]), ptr(s[0]), ptr(s[1]), ptr(s[2])) == 0
        return out

    plan = [(0, 2), (1, 1), (0, 1), (1, 3)]                       # (tensor, tokens)
    xs = [synth.activations(Cc, n, 400 + j) for j, (_, n) in enumerate(plan)]
    ys = [np.full((n, shapes[k]), 7.0, np.float32) for k, n in plan]
    rc = eng.salt_gpu_nvfp4_mixed_batch(abi.ptr_array([keys[k] for k, _ in plan]), abi.ptr_array(xs), abi.ptr_array(ys),
                                        (C.c_int * 4)(*[n for _, n in plan]), (C.c_int * 4)(*[shapes[k] for k, _ in plan]),
                                        Cc, 4)
    assert rc == 0, err(pkg)
    for (k, n), x, y in zip(plan, xs, ys):
        assert np.array_equal(bits(y), bits(want(k, x))), (k, n)
    # a height that is not the key's
    assert eng.salt_gpu_nvfp4_mixed_batch(abi.ptr_array([keys[0]]), abi.ptr_array(xs[:1]), abi.ptr_array(ys[:1]),
                                          (C.c_int * 1)(2), (C.c_int * 1)(shapes[1]), Cc, 1) == -1
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, 13) == 0


def test_router_gate_and_head_through_the_engine(eng, oracle, pkg):
    """An 8-bit router gate (one job per token of the same matrix, the way the engine batches it) and the bf16 head,
    both inside one described trunk resource."""
    g = synth.rng(77)
    GR, Cc, HR = 128, 2816, 4100
    gate_vals = g.integers(0, 256, size=GR * Cc, dtype=np.uint8)
    gate_scales = (g.uniform(0.001, 0.01, GR * Cc // 64).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    gate_biases = (g.uniform(-1.0, 0.0, GR * Cc // 64).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    head = (g.standard_normal(HR * Cc).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    parts, offs, at = [], [], 0
    for a in (gate_vals, gate_scales, gate_biases, head):
        offs.append(at); parts.append(a.view(np.uint8)); at += a.nbytes
        pad = (-at) % 16; parts.append(np.zeros(pad, np.uint8)); at += pad
    blob = np.concatenate(parts); base = blob.ctypes.data
    gv, gs, gb, hw = (base + o for o in offs)
    assert eng.salt_gpu_weight_resource_describe(TRUNK, 21, base, blob.nbytes) == 0
    assert eng.salt_gpu_weight_resource_activate(TRUNK, 21, 2) == 0, err(pkg)
    assert eng.salt_gpu_weight_resource_slot(TRUNK, 21, gv, gv, gs, gb, 8, GR, Cc) == 0, err(pkg)
    assert eng.salt_gpu_bf16_resource_slot(TRUNK, 21, hw, hw, HR, Cc) == 0, err(pkg)
    assert eng.salt_gpu_bf16_resource_slot(TRUNK, 21, hw, hw, HR, Cc) == 0                 # identical re-registration
    assert eng.salt_gpu_bf16_resource_slot(TRUNK, 21, hw, hw + 16, HR - 1, Cc) == -1       # key bound to another tensor
    assert eng.salt_gpu_bf16_resource_slot(TRUNK, 21, 0x5000, hw, HR, Cc + 4) == -1        # columns not a multiple of 8
    assert eng.salt_gpu_bf16_resource_slot(TRUNK, 21, 0x5000, hw, HR * 4, Cc) == -1        # outside the resource
    eng.salt_gpu_set_mapped_only(1)
    before = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(before))

    T = 5
    xs = synth.activations(Cc, T, 31); ys = np.full((T, GR), np.nan, np.float32)
    rc = eng.salt_gpu_q8_batch(abi.ptr_array([gv] * T), abi.ptr_array([gs] * T), abi.ptr_array([gb] * T),
                               abi.ptr_array([xs[t] for t in range(T)]), abi.ptr_array([ys[t] for t in range(T)]),
                               abi.ptr_array([gv] * T), (C.c_int * T)(*([GR] * T)), Cc, T)
    assert rc == 0, err(pkg)
    want = np.zeros(GR, np.float32)
    for t in range(T):
        oracle.orc_q8_matvec(ptr(gate_vals), ptr(gate_scales), ptr(gate_biases), GR, Cc, ptr(xs[t]), ptr(want))
        assert np.array_equal(bits(ys[t]), bits(want)), t
    y1 = np.full(GR, np.nan, np.float32)
    assert eng.salt_gpu_q8_matvec(gv, gs, gb, GR, Cc, ptr(xs[2]), ptr(y1)) == 0, err(pkg)
    assert np.array_equal(bits(y1), bits(ys[2]))
    # a key registered for another geometry is refused; so are weights outside every resource in mapped-only mode
    assert eng.salt_gpu_q8_matvec(gv, gs, gb, GR - 1, Cc, ptr(xs[2]), ptr(y1)) == -1
    loose = gate_vals.copy()
    assert eng.salt_gpu_q8_matvec(ptr(loose), gs, gb, GR, Cc, ptr(xs[2]), ptr(y1)) == -1

    logits = np.full(HR, np.nan, np.float32)
    assert eng.salt_gpu_bf16_matvec(hw, HR, Cc, ptr(xs[0]), ptr(logits)) == 0, err(pkg)
    want = np.zeros(HR, np.float32)
    oracle.orc_bf16_matvec(ptr(head), HR, Cc, ptr(xs[0]), None, ptr(want))
    assert np.array_equal(bits(logits), bits(want))
    assert eng.salt_gpu_bf16_matvec(hw, HR - 1, Cc, ptr(xs[0]), ptr(logits)) == -1         # geometry differs from the slot
    assert eng.salt_gpu_bf16_matvec(0x5000, HR, Cc, ptr(xs[0]), ptr(logits)) == -1         # unknown key
    assert eng.salt_gpu_bf16_matvec(gv, GR, Cc, ptr(xs[0]), ptr(logits)) == -1             # an 8-bit tensor's key
    assert eng.salt_gpu_bf16_matvec_batch(hw, HR, Cc, 2, ptr(xs), ptr(logits)) == -1       # left to the CPU, like the ROCm reference
    after = abi.BatchStats(); eng.salt_gpu_batch_stats_get(C.byref(after))
    assert after.trunk_batches - before.trunk_batches == 3
    eng.salt_gpu_set_mapped_only(0)
    # deferred publication: outputs appear at salt_gpu_sync
    assert eng.salt_gpu_set_defer(1) == 0
    logits[:] = np.nan
    assert eng.salt_gpu_bf16_matvec(hw, HR, Cc, ptr(xs[0]), ptr(logits)) == 0
    assert eng.salt_gpu_sync() == 0 and np.array_equal(bits(logits), bits(want))
    assert eng.salt_gpu_set_defer(0) == 0
    assert eng.salt_gpu_weight_resource_unbind(TRUNK, 21) == 0
    assert eng.salt_gpu_bf16_matvec(hw, HR, Cc, ptr(xs[0]), ptr(logits)) == -1


def test_exact_cells_over_a_shared_buffer(eng, oracle, pkg):
    """The block's fp32 cells the way the engine submits them: views into one startup-owned shared buffer, element
    offsets, one completion for the sequence (reference gemma4_text.c:6704-6822)."""
    n, E, K = 2816, 128, 8
    f32 = np.float32
    buf = abi.SharedBuffer()
    total = 16 * n
    assert eng.salt_gpu_shared_buffer_alloc(C.byref(buf), total * 4) == 0
    arr = np.ctypeslib.as_array(C.cast(buf.contents, C.POINTER(C.c_float)), shape=(total,))
    g = synth.rng(91)
    names = ["x", "w", "w2", "w3", "res", "dense", "routed", "out", "out2", "out3", "scratch", "scratch_hi", "logits",
             "scale", "sel", "wt"]
    off = {name: k * n for k, name in enumerate(names)}
    view = lambda name, count=n: arr[off[name]:off[name] + count]
    for name, spread in [("x", 3), ("w", 1), ("w2", 1), ("w3", 1), ("res", 2), ("dense", 5), ("routed", 0.01)]:
        view(name)[:] = (g.standard_normal(n) * spread).astype(f32)
    view("logits", E)[:] = synth.router_logits(E, 5)
    view("scale", E)[:] = g.uniform(0.5, 2.0, E).astype(f32)
    eps = f32(1e-6)

    def cell(kind, views, count, aux=0, scalar=0.0):
        c = abi.ExactCell()
        c.kind, c.n, c.aux, c.eps, c.scalar = kind, count, aux, eps, scalar
        for k, name in enumerate(views):
            c.views[k] = C.pointer(buf)
            c.offsets[k] = off[name]
        return c

    root = float(f32(1.0) / f32(oracle.orc_sqrtf(f32(n))))
    cells = (abi.ExactCell * 5)(
        cell(1, ["x", "w", "out"], n, aux=1),
        cell(6, ["x", "w2", "out2"], n, scalar=root),
        cell(2, ["logits", "scale", "sel", "wt"], E, aux=K),
        cell(4, ["res", "dense", "routed", "w", "w2", "w3", "scratch", "out3"], n, scalar=0.37),
        cell(5, ["logits"], E, scalar=30.0))
    logits = view("logits", E).copy()
    assert eng.salt_gpu_exact_cells(cells, 5) == 0, err(pkg)
    want = np.zeros(n, f32)
    assert oracle.orc_rmsnorm(ptr(want), ptr(view("x").copy()), ptr(view("w").copy()), n, eps, 1) == 0
    assert np.array_equal(bits(view("out")), bits(want))
    assert oracle.orc_router_input(ptr(want), ptr(view("x").copy()), ptr(view("w2").copy()), n, eps) == 0
    assert np.array_equal(bits(view("out2")), bits(want))
    sel = np.zeros(K, np.int32); wt = np.zeros(K, f32)
    assert oracle.orc_router_topk(ptr(logits), ptr(view("scale", E).copy()), E, K, ptr(sel), ptr(wt)) == 0
    oracle.orc_sort_selection(ptr(sel), ptr(wt), K)
    assert np.array_equal(view("sel", K).view(np.int32), sel) and np.array_equal(bits(view("wt", K)), bits(wt))
    assert oracle.orc_parallel_ffn_combine(ptr(want), ptr(view("res").copy()), ptr(view("dense").copy()),
                                           ptr(view("routed").copy()), ptr(view("w").copy()), ptr(view("w2").copy()),
                                           ptr(view("w3").copy()), f32(0.37), n, eps) == 0
    assert np.array_equal(bits(view("out3")), bits(want))
    capped = logits.copy()
    assert oracle.orc_softcap(ptr(capped), E, f32(30.0)) == 0 and np.array_equal(bits(view("logits", E)), bits(capped))
    # a non-finite element fails the call; a view past the buffer, an unknown kind and a foreign buffer are refused
    view("dense")[17] = np.inf
    before = view("out3").copy()
    assert eng.salt_gpu_exact_cells(cells, 4) == -1 and np.array_equal(bits(view("out3")), bits(before))
    view("dense")[17] = 1.0
    bad = cell(1, ["x", "w", "out"], n, aux=1); bad.offsets[2] = total - n + 1
    assert eng.salt_gpu_exact_cells(C.byref(bad), 1) == -1
    bad = cell(9, ["x", "w", "out"], n)
    assert eng.salt_gpu_exact_cells(C.byref(bad), 1) == -1
    host = np.zeros(n, f32)
    foreign = abi.SharedBuffer(host.ctypes.data, host.nbytes, host.ctypes.data)
    bad = cell(1, ["x", "w", "out"], n, aux=1); bad.views[0] = C.pointer(foreign); bad.offsets[0] = 0
    assert eng.salt_gpu_exact_cells(C.byref(bad), 1) == -1
    assert eng.salt_gpu_exact_cells(cells, 0) == -1
    assert eng.salt_gpu_shared_buffer_free(C.byref(buf)) == 0


def test_off_path_entry_points_answer_like_the_null_backend(eng):
    z = np.zeros(64, np.float32)
    assert eng.salt_dispatch_get() is None and eng.salt_gpu_tensor_program_ops() is None


def test_whole_mapping_conveniences(eng, oracle, pkg):
    """salt_gpu_resident_trunk_map / _unmap / _pool_map: one trunk range at a time, weights served from it."""
    R, Cc = 130, 2816
    vals, scales, biases = synth.q4_tensor(R, Cc, 61)
    blob = np.concatenate([np.zeros(100, np.uint8), vals.view(np.uint8), scales.view(np.uint8), biases.view(np.uint8)])
    base = blob.ctypes.data
    v, s, b = base + 100, base + 100 + vals.nbytes, base + 100 + vals.nbytes + scales.nbytes
    assert eng.salt_gpu_resident_trunk_map(base, blob.nbytes) == 0, err(pkg)
    assert eng.salt_gpu_resident_trunk_map(base, blob.nbytes) == -1                 # one mapping at a time
    eng.salt_gpu_set_mapped_only(1)
    x = synth.activations(Cc, 1, 62)[0]; y = np.zeros(R, np.float32)
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == 0, err(pkg)
    assert np.array_equal(bits(y), bits(q4_want(oracle, vals, scales, biases, R, Cc, x)[0]))
    assert eng.salt_gpu_resident_trunk_unmap() == 0
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == -1             # gone, and copying is forbidden
    assert eng.salt_gpu_resident_pool_map(base, blob.nbytes) == 0, err(pkg)         # expert-layer resource 0
    assert eng.salt_gpu_q4_matvec(v, s, b, R, Cc, ptr(x), ptr(y)) == 0
    assert eng.salt_gpu_expert_resource_unbind(0) == 0
    eng.salt_gpu_set_mapped_only(0)


def test_zz_free_and_reinit(eng, pkg):
    assert eng.salt_gpu_free() == 0
    z = np.zeros(64, np.float32)
    assert eng.salt_gpu_q4_matvec(ptr(z), ptr(z), None, 1, 64, ptr(z), ptr(z)) == -1     # fails loudly when not initialised
    assert eng.salt_gpu_init() == 0
