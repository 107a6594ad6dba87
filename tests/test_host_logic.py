"""Host-side logic that needs no GPU: pool policy, plan argument checks, table building and
expression lowering."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from fortis_amd import stencil as S
from fortis_amd._lib import Ins, Stencil

# ---- pool: the reference's policy (runtime/fortis_rt.c:14-40) on a host allocator ---------------
ALLOC = C.CFUNCTYPE(C.c_int, C.POINTER(C.c_void_p), C.c_size_t)
FREE = C.CFUNCTYPE(None, C.c_void_p)


class FakeDevice:
    def __init__(self, capacity):
        self.capacity, self.live, self.next = capacity, {}, 0x1000
        self.allocs = self.frees = 0

        def a(pp, n):
            if sum(self.live.values()) + n > self.capacity:
                return -1
            self.next += 0x100000
            self.live[self.next] = n
            pp[0] = self.next
            self.allocs += 1
            return 0

        def f(p):
            del self.live[p]
            self.frees += 1

        self.a, self.f = ALLOC(a), FREE(f)


@pytest.fixture
def pool(L):
    dev = FakeDevice(1000)
    L.fortis_pool_set_allocator(C.cast(dev.a, C.c_void_p), C.cast(dev.f, C.c_void_p))
    yield L, dev
    L.fortis_pool_set_allocator(None, None)


def stats(L):
    h, u = C.c_int(), C.c_int()
    L.fortis_pool_stats(C.byref(h), C.byref(u))
    return h.value, u.value


def test_pool_best_fit_reuse(pool):
    L, dev = pool
    a, b, c = L.fortis_alloc(100), L.fortis_alloc(300), L.fortis_alloc(200)
    assert dev.allocs == 3 and stats(L) == (3, 3)
    for p in (a, b, c):
        L.fortis_free(p)
    assert stats(L) == (3, 0) and dev.frees == 0          # released buffers stay allocated
    assert L.fortis_alloc(150) == c                        # smallest released buffer that fits
    assert L.fortis_alloc(150) == b
    assert L.fortis_alloc(50) == a
    assert dev.allocs == 3


def test_pool_release_all_and_retry_on_oom(pool):
    L, dev = pool
    a, b = L.fortis_alloc(400), L.fortis_alloc(400)
    L.fortis_free(a)
    L.fortis_free(b)
    c = L.fortis_alloc(900)                                # does not fit beside 800 held bytes
    assert c and dev.frees == 2 and stats(L) == (1, 1)
    assert not L.fortis_alloc(200)                         # genuinely out of memory: NULL, no crash
    L.fortis_free(c)
    assert L.fortis_alloc(900) == c


def test_pool_trim_frees_what_is_held_unused(pool):
    L, dev = pool
    a, b, c = L.fortis_alloc(100), L.fortis_alloc(300), L.fortis_alloc(200)
    L.fortis_free(a)
    L.fortis_free(c)
    assert L.fortis_pool_trim() == 2 and dev.frees == 2 and stats(L) == (1, 1)      # b is in use and stays
    assert sorted(dev.live.values()) == [300]
    assert L.fortis_pool_trim() == 0
    L.fortis_free(b)
    assert L.fortis_alloc(250) == b                        # the pool goes on as before


def test_pool_unknown_pointer_is_really_freed(pool):
    L, dev = pool
    p = C.c_void_p()
    assert dev.a(C.byref(p), 10) == 0
    L.fortis_free(p.value)
    assert dev.frees == 1


# ---- allocations the library makes for itself fail cleanly ---------------------------------------------
def test_finalize_fails_when_the_weights_find_no_device_memory(pool, capfd):
    """Weights, vectors and packed blobs go through the same switchable allocator as the pool: when one of them
    finds no memory, finalize returns -1 (the reference prints and returns NULL, runtime/fortis_rt.c:35), the
    plan never launches, and destroying it hands everything back."""
    L, dev = pool                                              # 1000 bytes of "device" memory
    p = L.fortis_plan_create()
    t0, t1 = L.fortis_plan_tensor(p, 2 * 4 * 4), L.fortis_plan_tensor(p, 2 * 300 * 4)
    W = np.zeros((300, 4), np.float32)                         # 4800 bytes: does not fit
    assert L.fortis_plan_linear(p, t0, t1, W.ctypes.data_as(C.c_void_p), None, 2, 4, 300, 0, 0.0) == 0
    assert L.fortis_plan_finalize(p, t0, t1) == -1
    err = capfd.readouterr().err
    assert "device allocation of 4800 bytes failed (plan weights)" in err and "out of device memory" in err
    assert L.fortis_plan_num_kernels(p) == -1                  # not finalized
    L.fortis_plan_run(p)
    assert "not finalized" in capfd.readouterr().err
    L.fortis_plan_destroy(p)
    assert not dev.live and stats(L)[1] == 0


def test_stencil_config_fails_when_the_cell_list_finds_no_device_memory(pool, capfd, golden):
    L, dev = pool
    g, lp, kd = [json.load(open(os.path.join(golden, f"zb_{n}.json"))) for n in ("gather", "loop", "kdist")]
    cells = (np.arange(300, dtype=np.int32) % 60) + 1 + 68 * (1 + np.arange(300, dtype=np.int32) // 60)   # 1200 bytes
    t = S.build_table(g, lp, kd, "gather", cells=cells)
    assert L.fortis_stencil_check(C.byref(t)) == 0
    assert L.fortis_gather_config(C.byref(t)) == -1
    assert "stencil cell list" in capfd.readouterr().err
    L.fortis_gather_v(None, None)                              # nothing configured: prints, touches nothing
    assert "no gather table configured" in capfd.readouterr().err
    assert not dev.live


def test_stencil_table_must_hold_the_planes_it_names(L, golden, capfd):
    """nk planes from iteration klo on must fit the array: the host-array entries copy exactly those."""
    g, lp, kd = [json.load(open(os.path.join(golden, f"zb_{n}.json"))) for n in ("gather", "loop", "kdist")]
    t = S.build_table(g, lp, kd, "gather")
    assert L.fortis_stencil_check(C.byref(t)) == 0
    t.nk = 16                                                  # the arrays hold 15 planes
    assert L.fortis_stencil_check(C.byref(t)) == -1
    t.nk, t.klo = 15, 2
    assert L.fortis_stencil_check(C.byref(t)) == -1
    t.nk, t.klo = 14, 2
    assert L.fortis_stencil_check(C.byref(t)) == 0
    assert "fewer than the" in capfd.readouterr().err


# ---- plan argument checks (no device work before finalize) ------------------------------------------
def test_plan_rejects_bad_arguments(L):
    p = L.fortis_plan_create()
    t0, t1 = L.fortis_plan_tensor(p, 64 * 27 * 4), L.fortis_plan_tensor(p, 64 * 3 * 4)
    W = np.zeros((3, 27), np.float32)
    vp = W.ctypes.data_as(C.c_void_p)
    assert L.fortis_plan_tensor(p, 0) == -1
    assert L.fortis_plan_linear(p, t0, t1, vp, None, 64, 27, 3, 0, 0.0) == 0
    assert L.fortis_plan_linear(p, t0, t1, vp, None, 65, 27, 3, 0, 0.0) == -1      # tensor too small
    assert L.fortis_plan_linear(p, t0, t0, vp, None, 64, 27, 27, 0, 0.0) == -1     # aliased
    assert L.fortis_plan_linear(p, t0, 7, vp, None, 64, 27, 3, 0, 0.0) == -1       # unknown tensor
    assert L.fortis_plan_linear(p, t0, t1, vp, None, 64, 27, 3, 9, 0.0) == -1      # unknown activation
    assert L.fortis_plan_linear(p, t0, t1, None, None, 64, 27, 3, 0, 0.0) == -1
    assert L.fortis_plan_mask_relu(p, t1, t1, 64, 3, 4) == -1                       # tail > n
    assert L.fortis_plan_conv2d(p, t0, t1, vp, None, vp, None, None, None, 1e-5, 1, 8, 8, 1, 3, 3, 1, 1, 0, 0.0, 0, 0) == -1  # partial BN
    assert L.fortis_plan_num_kernels(p) == -1                                       # not finalized
    L.fortis_plan_destroy(p)


def test_entries_without_a_bound_step_do_not_crash(L, capfd):
    L.fortis_step_reset()
    L.mlp_forward_dev()
    assert "no step bound" in capfd.readouterr().err


# ---- tables ---------------------------------------------------------------------------------------------
def test_zb_tables_from_the_reference_descriptors(golden, L):
    g, s, gd, sd, lp, kd = S.load_tables(*[os.path.join(golden, f"zb_{n}.json") for n in ("gather", "scatter", "loop", "kdist")])
    assert (g.count, g.nk, g.klo, g.ilo, g.jlo, g.ni, g.nj, g.nargs) == (4736, 15, 1, 3, 3, 64, 74, 0)
    assert (s.count, s.nk, s.nrefs, s.nscal, s.nargs) == (4736, 15, 3, 2, 1)
    # slot q = f*9 + (dj+1)*3 + (di+1) reads A_f[(i+di-1) + (j+dj-1)*68] (mom6_zb/gather.cu:21-48)
    for q in range(27):
        f, dj, di = q // 9, (q % 9) // 3 - 1, q % 3 - 1
        r = g.refs[q]
        assert (r.array, r.planar, r.base, r.si, r.sj) == (f, 1, (di - 1) + (dj - 1) * 68, 1, 68)
    assert [g.plane[a] for a in range(4)] == [5304] * 4 and [g.total[a] for a in range(4)] == [79560] * 4
    assert [s.plane[a] for a in range(5)] == [5304] * 5 and [s.total[a] for a in range(5)] == [79560, 5304, 5304, 79560, 79560]
    assert [(s.refs[q].array, s.refs[q].planar) for q in range(3)] == [(2, 0), (3, 1), (4, 1)]
    assert L.fortis_stencil_check(C.byref(g)) == 0 and L.fortis_stencil_check(C.byref(s)) == 0


def test_batch_already_multiplied_by_nk_is_accepted(golden):
    paths = [os.path.join(golden, f"zb_{n}.json") for n in ("gather", "scatter", "loop", "kdist")]
    gd, lp, kd = json.load(open(paths[0])), json.load(open(paths[2])), json.load(open(paths[3]))
    lp["batch"] *= kd["nk"]                                 # what driver/fortisc.sh:44 does before emitting
    assert S.build_table(gd, lp, kd, "gather").count == 4736


def test_expression_compiler():
    assert S.compile_exprs(["(((tv * S0) * S0) * S1)"])[0] == [(2, 0, 1), (2, 32, 1), (2, 33, 2)]
    ins, consts = S.compile_exprs(["(tv / (S0 + 1.000000e-30f))"])
    assert ins == [(0, 1, 16), (3, 0, 32)] and consts == [(float(np.float32(1e-30)), False)]
    ins, _ = S.compile_exprs(["(tv * S0)", "(tv - 2.0f)"])   # two expressions in order, each replacing tv
    assert ins == [(2, 0, 1), (1, 32, 16)]
    with pytest.raises(ValueError):
        S.compile_exprs(["cbrtf(tv)"])


def _table_with(ins, nscal=2, nconst=1):
    t = Stencil()
    t.narrays, t.nrefs, t.nscal, t.count, t.nk, t.ni, t.sx = 1, 1, nscal, 4, 1, 2, 4
    t.total[0] = t.plane[0] = 16
    t.nins, t.nconst = len(ins), nconst
    for n, i3 in enumerate(ins):
        t.ins[n] = Ins(*i3)
    return t


def test_table_routing_chains_general_forms_and_invalid_tables(L, capfd):
    """One chain of + - * / on the slot value runs in the fused-form kernels (route 0); other valid
    programs take the general kernels (route 1); malformed tables are refused (route -1)."""
    chains = [[(0, 1, 16), (3, 0, 32)], [(2, 0, 1), (2, 32, 1), (2, 33, 2)], [(1, 16, 0)], []]
    for ins in chains:
        assert L.fortis_stencil_route(C.byref(_table_with(ins))) == 0
        assert L.fortis_stencil_check(C.byref(_table_with(ins))) == 0
    general = [[(2, 0, 0)],                  # tv * tv
               [(2, 0, 1), (0, 32, 0)],      # re-reads tv after transforming it
               [(2, 0, 1), (0, 1, 2)],       # last instruction does not involve the slot value
               [(0, 1, 2)],                  # never uses tv
               [(7, 0, 0)],                  # sqrtf
               [(2 | 0x100, 0, 1), (11, 32, 32)]]   # double product, converted back
    for ins in general:
        assert L.fortis_stencil_route(C.byref(_table_with(ins))) == 1
        assert L.fortis_stencil_check(C.byref(_table_with(ins))) == 0
    bad = [[(12, 0, 1)],                     # unknown op
           [(2 | 0x200, 0, 1)],              # unknown flag
           [(0, 0, 5)],                      # scalar out of range
           [(0, 0, 17)],                     # constant out of range
           [(0, 0, 32)]]                     # result not yet computed
    for ins in bad:
        assert L.fortis_stencil_route(C.byref(_table_with(ins))) == -1
        assert L.fortis_stencil_check(C.byref(_table_with(ins))) == -1
    capfd.readouterr()


# ---- persistent GEMM work list --------------------------------------------------------------------
@pytest.mark.parametrize("B,N,slots", [(24576, 768, 512), (24576, 368, 512), (24576, 768, 768), (8300, 1100, 512),
                                       (12000, 1100, 512), (1, 1, 512), (128, 128, 8), (100000, 4000, 512), (257, 385, 512)])
def test_gemm_schedule_covers_every_tile_once(L, B, N, slots):
    """Whole rounds of 128 x 128 tiles, then halves, then quarters: every 64 x 64 quarter of every tile
    is produced exactly once, no phase but the first exceeds one round, and full tiles come in whole rounds."""
    tri = (C.c_long * 12)()
    n = L.fortis_gemm_schedule(B, N, slots, tri)
    assert 1 <= n <= 4
    tiles = -(-B // 128) * -(-N // 128)
    cover = np.zeros((tiles, 4), np.int32)
    for p in range(n):
        level, base, count = tri[3 * p], tri[3 * p + 1], tri[3 * p + 2]
        if level == 0:
            assert p == 0 and base == 0 and count % slots == 0
            cover[:count] += 1
        elif level == 1:
            assert count <= slots and count % 2 == 0
            cover[base:base + count // 2] += 1
        else:
            assert level == 2 and count <= slots and count % 4 == 0
            cover[base:base + count // 4] += 1
    assert (cover == 1).all()
    # balance: the items of the tail phases are at most one round each, so no workgroup gets more than
    # (whole rounds) + 1/2 + 1/4 + 1/4 of a tile beyond the ideal share
    work = sum({0: 1.0, 1: 0.5, 2: 0.25}[tri[3 * p]] * -(-tri[3 * p + 2] // slots) for p in range(n))
    assert work <= tiles / slots + 1.0


def test_gemm_schedule_rejects_bad_arguments(L):
    tri = (C.c_long * 12)()
    assert L.fortis_gemm_schedule(0, 5, 512, tri) == -1
    assert L.fortis_gemm_schedule(5, 5, 7, tri) == -1


# ---- exact division by a launch constant (cell decode of the stencil kernels) ---------------------------
def test_magic_divmod_is_exact():
    """q = (n * ceil(2^64 / d)) >> 64 must equal n // d for every 32-bit n: checked on the edges of the
    range, around multiples of d, and on random pairs, against Python integers."""
    import fortis_amd
    L = fortis_amd.load()
    rng = np.random.default_rng(0)
    ds = [1, 2, 3, 5, 7, 64, 65, 4736, 2376, 1048576, 65535, 65537, 2**31 - 1, 2**31, 2**31 + 1, 2**32 - 1] + \
        [int(v) for v in rng.integers(1, 2**32, 40)]
    q, r = C.c_uint(), C.c_uint()
    for d in ds:
        ns = {0, 1, d - 1, d, d + 1, 2**32 - 1, 2**32 - 2, 2**31, (2**32 - 1) // d * d, max((2**32 - 1) // d * d - 1, 0)}
        ns |= {int(v) for v in rng.integers(0, 2**32, 200)}
        ns |= {min(int(k) * d + off, 2**32 - 1) for k in rng.integers(0, max(2**32 // d, 1), 50) for off in (-1, 0, 1) if int(k) * d + off >= 0}
        for n_ in (v for v in ns if 0 <= v < 2**32):
            L.fortis_magic_divmod(n_, d, C.byref(q), C.byref(r))
            assert (q.value, r.value) == (n_ // d, n_ % d), (n_, d)


def test_bench_contract_without_a_gpu():
    """bench.py refuses more than one GPU with a message (the path has no exchange step to measure), and its
    measured-traffic table has an entry for every workload that reports a roofline against measured HBM bytes."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "ONE GPU" in (r.stderr + r.stdout)
    sys.path.insert(0, root)
    import bench
    for key in ("climsim", "zb", "zb_ref", "zb_1028x1028x15", "zb_unfused_1028x1028x15", "zb_unfused_1028x1028x15_f64", "unet", "tsrgan"):
        assert bench.MEASURED_TRAFFIC[key] > 0
    assert bench.PEAK_HBM_GBS == 8000.0 and bench.PEAK_F32_MFMA_TFLOPS == 157.3


def _mask_relu_stack(L, sizes):
    """A plan of weightless row-wise ops t0 -> t1 -> ... (one tensor per entry of sizes, in floats)."""
    p = L.fortis_plan_create()
    ts = [L.fortis_plan_tensor(p, 4 * n) for n in sizes]
    for a, b, n in zip(ts[:-1], ts[1:], sizes[1:]):
        assert L.fortis_plan_mask_relu(p, a, b, 1, min(n, sizes[ts.index(a)]), 0) == 0
    return p, ts


def test_buffer_walk_survives_a_raw_allocation_that_fails_once(pool):
    """The walk that gives tensors their buffers hands a temporary back behind its last reader.  When a later raw
    allocation fails, the pool frees every buffer it holds unused and retries (runtime/fortis_rt.c:24-35): none of
    those may be a buffer an earlier tensor of the same walk still points to.  One raw allocation is made to fail
    once in the middle of the walk; afterwards every tensor's buffer is a live allocation, tensors alive at the same
    time have different buffers, and destroying the plan hands everything back."""
    L, dev = pool
    dev.capacity = 1 << 20
    fail_at, real = [4], dev.a                       # the walk's 4th raw allocation fails once (t3: larger than released t1)

    def flaky(pp, n):
        fail_at[0] -= 1
        return -1 if fail_at[0] == 0 else real(pp, n)

    fa = ALLOC(flaky)
    L.fortis_pool_set_allocator(C.cast(fa, C.c_void_p), C.cast(dev.f, C.c_void_p))
    sizes = [8, 16, 16, 32, 8]                       # t0 in, t1, t2, t3 (needs a new, larger buffer), t4 out
    p, ts = _mask_relu_stack(L, sizes)
    assert L.fortis_plan_finalize(p, ts[0], ts[-1]) == 0
    ptr = [L.fortis_plan_tensor_ptr(p, t) for t in ts]
    assert all(q in dev.live for q in ptr), "a tensor points at a buffer the raw allocator has taken back"
    for a, b in zip(ptr[:-1], ptr[1:]):
        assert a != b                                # a kernel's source and destination never share
    assert ptr[0] not in ptr[1:]                     # the model's input is never shared
    held, used = stats(L)
    assert used == len(set(ptr)) and held == used    # every buffer of the plan stays in use in the pool; nothing else is held
    L.fortis_plan_destroy(p)
    assert stats(L)[1] == 0


def test_buffer_walk_that_runs_out_of_memory_fails_cleanly(pool, capfd):
    """A walk whose later tensor finds no memory even after the pool has released what it can: finalize returns -1,
    no tensor pointer is handed out, and destroy returns every buffer exactly once."""
    L, dev = pool                                    # 1000 bytes
    p, ts = _mask_relu_stack(L, [50, 50, 50, 200, 50])      # 200 + 200 + 200 + 800 bytes > 1000
    assert L.fortis_plan_finalize(p, ts[0], ts[-1]) == -1
    assert "out of device memory for the activations" in capfd.readouterr().err
    assert L.fortis_plan_tensor_ptr(p, ts[1]) is None
    frees0 = dev.frees
    L.fortis_plan_destroy(p)
    assert stats(L)[1] == 0 and dev.frees == frees0  # handed back to the pool (still held there), none freed twice


def test_conv_partial_sum_buffer_fails_cleanly_without_memory(pool, capfd):
    """The convolution path's own buffers come from the same switchable allocator: a request the device cannot
    meet prints what was asked and returns -1 (the launchers then launch nothing), a smaller one succeeds and is
    kept, and a later request that fits the kept buffer allocates nothing."""
    L, dev = pool                                              # 1000 bytes
    assert L.fortis_conv_scratch_reserve(5000) == -1
    assert "device allocation of 5000 bytes failed (conv partial sums)" in capfd.readouterr().err
    assert L.fortis_conv_scratch_reserve(600) == 0 and dev.allocs == 1
    assert L.fortis_conv_scratch_reserve(400) == 0 and dev.allocs == 1
    assert L.fortis_conv_scratch_reserve(-1) == -1
