"""Device arena and stream pool: the behaviours the upstream tests pin for
NumaArena / ThreadPool (test_linux_threading.mojo:56-102, :164-215, :304-398),
restated for device memory and streams."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx(mi):
    h = C.c_void_p()
    mi.check(mi.lib.mi_ctx_create(0, C.byref(h)))
    yield h
    mi.lib.mi_ctx_destroy(h)


def test_context_reports_gfx950(mi, ctx):
    buf = C.create_string_buffer(64)
    mi.check(mi.lib.mi_ctx_arch_name(ctx, buf, 64))
    assert buf.value.startswith(b"gfx950")
    assert mi.lib.mi_ctx_compute_units(ctx) >= 64
    assert mi.lib.mi_ctx_memory_bytes(ctx) > (64 << 30)
    bad = C.c_void_p()
    assert mi.lib.mi_ctx_create(99, C.byref(bad)) == mi.ENODEV


def test_arena_bump_marks_and_exhaustion(mi, ctx):
    lib = mi.lib
    a = C.c_void_p()
    mi.check(lib.mi_arena_create(ctx, 1 << 20, 256, C.byref(a)))
    assert lib.mi_arena_used(a) == 0 and lib.mi_arena_remaining(a) == 1 << 20
    assert lib.mi_arena_verify_placement(a) == 1          # nothing allocated: true
    p1 = lib.mi_arena_alloc(a, 100)
    p2 = lib.mi_arena_alloc(a, 100)
    assert p1 and p2 and p2 - p1 == 256 and p1 % 256 == 0  # aligned bump
    assert lib.mi_arena_used(a) == 256 + 100
    mark = lib.mi_arena_mark(a)
    p3 = lib.mi_arena_alloc(a, 4096)
    assert lib.mi_arena_reset_to(a, mark + 1 << 30) == mi.EINVAL   # beyond used: ignored
    assert lib.mi_arena_reset_to(a, -1) == mi.EINVAL
    assert lib.mi_arena_reset_to(a, mark) == mi.OK
    assert lib.mi_arena_alloc(a, 4096) == p3                       # watermark restored
    assert lib.mi_arena_alloc(a, 2 << 20) is None                  # exhausted: null, no error
    assert lib.mi_arena_verify_placement(a) == 1
    # fresh arena memory reads as zero
    host = np.ones(64, np.uint32)
    mi.check(lib.mi_memcpy_d2h(host.ctypes.data, p1, host.nbytes, None))
    mi.check(lib.mi_stream_synchronize(None))
    assert not host.any()
    lib.mi_arena_reset(a)
    assert lib.mi_arena_used(a) == 0
    bad = C.c_void_p()
    assert lib.mi_arena_create(ctx, 1 << 20, 48, C.byref(bad)) == mi.EINVAL   # alignment not a power of two
    mi.check(lib.mi_arena_destroy(a))


def test_stream_pool_launch_wait_all_and_reuse(mi, ctx):
    """32 launches on a pool of 4 in batches, as test_thread_pool / test_pool_reuse."""
    lib = mi.lib
    pool, a = C.c_void_p(), C.c_void_p()
    mi.check(lib.mi_stream_pool_create(ctx, 4, C.byref(pool)))
    mi.check(lib.mi_arena_create(ctx, 1 << 20, 256, C.byref(a)))
    assert lib.mi_stream_pool_capacity(pool) == 4
    buf = lib.mi_arena_alloc(a, 32 * 4096)
    for batch in range(8):
        for i in range(4):
            slot = lib.mi_stream_pool_begin(pool)
            assert slot >= 0
            k = batch * 4 + i
            mi.check(lib.mi_fill_u32(buf + k * 4096, 2 * k * k, 1024, lib.mi_stream_pool_stream(pool, slot)))
            mi.check(lib.mi_stream_pool_end(pool, slot))
        mi.check(lib.mi_stream_pool_wait_all(pool))
    host = np.empty(32 * 1024, np.uint32)
    mi.check(lib.mi_memcpy_d2h(host.ctypes.data, buf, host.nbytes, None))
    mi.check(lib.mi_stream_synchronize(None))
    assert np.array_equal(host.reshape(32, 1024)[:, 0], 2 * np.arange(32, dtype=np.uint32) ** 2)
    assert lib.mi_stream_pool_wait_any(pool) == -1       # nothing in flight
    mi.check(lib.mi_stream_pool_destroy(pool))
    mi.check(lib.mi_arena_destroy(a))


def test_stream_pool_full_wait_any_and_busy_destroy(mi, ctx):
    lib = mi.lib
    pool, a, gate = C.c_void_p(), C.c_void_p(), C.c_void_p()
    mi.check(lib.mi_stream_pool_create(ctx, 2, C.byref(pool)))
    mi.check(lib.mi_arena_create(ctx, 64 << 20, 256, C.byref(a)))
    mi.check(lib.mi_gate_create(ctx, C.byref(gate)))
    assert lib.mi_gate_wait(gate, None) == mi.EINVAL      # never released
    big = lib.mi_arena_alloc(a, 48 << 20)
    done = []
    launched = 0
    for it in range(50):                                  # launch-all / wait-any / wait-all, as test_wait_any_reuse
        while True:
            slot = lib.mi_stream_pool_begin(pool)
            if slot < 0:
                assert slot == mi.EBUSY
                break
            s = lib.mi_stream_pool_stream(pool, slot)
            mi.check(lib.mi_fill_u32(big, it, (48 << 20) // 4, s))
            mi.check(lib.mi_stream_pool_end(pool, slot))
            launched += 1
            if launched % 2 == 0:
                break
        got = lib.mi_stream_pool_wait_any(pool)
        assert got in (0, 1)
        done.append(got)
        mi.check(lib.mi_stream_pool_wait_all(pool))
    assert launched == 100
    # destroy while busy is refused, not fatal
    slot = lib.mi_stream_pool_begin(pool)
    s = lib.mi_stream_pool_stream(pool, slot)
    for _ in range(20):
        mi.check(lib.mi_fill_u32(big, 7, (48 << 20) // 4, s))
    mi.check(lib.mi_gate_release(gate, s))
    mi.check(lib.mi_stream_pool_end(pool, slot))
    rc = lib.mi_stream_pool_destroy(pool)
    assert rc in (mi.EBUSY, mi.OK)
    if rc == mi.EBUSY:
        mi.check(lib.mi_gate_wait_host(gate))
        mi.check(lib.mi_stream_pool_wait_all(pool))
        mi.check(lib.mi_stream_pool_destroy(pool))
    mi.check(lib.mi_gate_reset(gate))
    assert lib.mi_gate_wait_host(gate) == mi.EINVAL
    mi.check(lib.mi_gate_destroy(gate))
    mi.check(lib.mi_arena_destroy(a))


def test_gate_orders_two_streams(mi, ctx):
    """Chain reduce across streams: each stage waits on the previous stage's
    gate, as the NUMA ring reduce waits on futex gates (test_linux_threading.mojo:400-476)."""
    lib = mi.lib
    n = 4
    pool, a = C.c_void_p(), C.c_void_p()
    mi.check(lib.mi_stream_pool_create(ctx, n, C.byref(pool)))
    mi.check(lib.mi_arena_create(ctx, 1 << 20, 256, C.byref(a)))
    gates = []
    buf = lib.mi_arena_alloc(a, 4096)
    stage = lib.mi_arena_alloc(a, 4096)
    for i in range(n):
        g = C.c_void_p()
        mi.check(lib.mi_gate_create(ctx, C.byref(g)))
        gates.append(g)
    for i in range(n):
        slot = lib.mi_stream_pool_begin(pool)
        s = lib.mi_stream_pool_stream(pool, slot)
        if i:
            mi.check(lib.mi_gate_wait(gates[i - 1], s))
        mi.check(lib.mi_fill_u32(stage, i + 1, 1024, s))        # each stage overwrites: order matters
        mi.check(lib.mi_memcpy_d2d(buf, stage, 4096, s))
        mi.check(lib.mi_gate_release(gates[i], s))
        mi.check(lib.mi_stream_pool_end(pool, slot))
    mi.check(lib.mi_stream_pool_wait_all(pool))
    host = np.empty(1024, np.uint32)
    mi.check(lib.mi_memcpy_d2h(host.ctypes.data, buf, 4096, None))
    mi.check(lib.mi_stream_synchronize(None))
    assert np.all(host == n)
    for g in gates:
        lib.mi_gate_destroy(g)
    mi.check(lib.mi_stream_pool_destroy(pool))
    mi.check(lib.mi_arena_destroy(a))


def test_wait_any_returns_slots_in_completion_order(mi, ctx):
    """test_wait_any (test_linux_threading.mojo:304-357): workers with inverse amounts of work finish in
    reverse order.  A worker's work is a chain of one-workgroup kernels (1500, 1000, 500 of them) recorded as a graph
    beforehand, so that the launches leave the host within microseconds of each other and the chains run side by
    side.  Three workers, not four: a process has four hardware queues here and streams beyond that share one, which
    serializes them behind each other whatever their length."""
    lib = mi.lib
    pool, a = C.c_void_p(), C.c_void_p()
    mi.check(lib.mi_stream_pool_create(ctx, 3, C.byref(pool)))
    mi.check(lib.mi_arena_create(ctx, 1 << 20, 256, C.byref(a)))
    bufs = [lib.mi_arena_alloc(a, 4096) for _ in range(3)]
    one = lib.mi_arena_alloc(a, 4096)
    ones = np.ones(1024, np.float32)
    mi.check(lib.mi_memcpy_h2d(one, ones.ctypes.data, ones.nbytes, None))
    mi.check(lib.mi_add_f32(one, one, bufs[0], 1024, None))      # first-launch costs paid before the race
    mi.check(lib.mi_stream_synchronize(None))
    graphs = []
    for i in range(3):
        s = lib.mi_stream_pool_stream(pool, i)
        mi.check(lib.mi_fill_u32(bufs[i], 0, 1024, s))
        mi.check(lib.mi_stream_synchronize(s))
        mi.check(lib.mi_graph_capture_begin(s))
        for _ in range(500 * (3 - i)):
            mi.check(lib.mi_add_f32(bufs[i], one, bufs[i], 1024, s))
        g = C.c_void_p()
        mi.check(lib.mi_graph_capture_end(s, C.byref(g)))
        graphs.append(g)
    for i in range(3):
        slot = lib.mi_stream_pool_begin(pool)
        assert slot == i
        mi.check(lib.mi_graph_launch(graphs[i], lib.mi_stream_pool_stream(pool, slot)))
        mi.check(lib.mi_stream_pool_end(pool, slot))
    order = [lib.mi_stream_pool_wait_any(pool) for _ in range(3)]
    assert order == [2, 1, 0]
    assert lib.mi_stream_pool_wait_any(pool) == -1
    out = np.empty(1024, np.float32)
    for i in range(3):
        mi.check(lib.mi_memcpy_d2h(out.ctypes.data, bufs[i], out.nbytes, None))
        mi.check(lib.mi_stream_synchronize(None))
        assert np.all(out == 500 * (3 - i))                      # every link of the chain ran, in order
    for g in graphs:
        mi.check(lib.mi_graph_destroy(g))
    mi.check(lib.mi_stream_pool_destroy(pool))
    mi.check(lib.mi_arena_destroy(a))


def test_butterfly_all_reduce_over_eight_pools(mi, ctx):
    """test_all_reduce (test_linux_threading.mojo:478-553) with a stream pool per "node": log2(N) rounds, in round r
    node i reads the value of node i ^ (1 << r) into its scratch (phase 1), every pool is waited for, then adds the
    scratch to its own value (phase 2), every pool is waited for.  Afterwards every node holds 1 + 2 + ... + N."""
    lib = mi.lib
    N, L = 8, 4096
    a = C.c_void_p()
    mi.check(lib.mi_arena_create(ctx, 1 << 20, 256, C.byref(a)))
    values = [lib.mi_arena_alloc(a, L * 4) for _ in range(N)]
    scratch = [lib.mi_arena_alloc(a, L * 4) for _ in range(N)]
    for i in range(N):
        host = np.full(L, i + 1, np.float32)
        mi.check(lib.mi_memcpy_h2d(values[i], host.ctypes.data, host.nbytes, None))
    mi.check(lib.mi_stream_synchronize(None))
    pools = []
    for _ in range(N):
        p = C.c_void_p()
        mi.check(lib.mi_stream_pool_create(ctx, 1, C.byref(p)))
        pools.append(p)

    def launch(node, op):
        slot = lib.mi_stream_pool_begin(pools[node])
        assert slot == 0
        mi.check(op(lib.mi_stream_pool_stream(pools[node], slot)))
        mi.check(lib.mi_stream_pool_end(pools[node], slot))

    r = 0
    while (1 << r) < N:
        for node in range(N):
            partner = node ^ (1 << r)
            launch(node, lambda s, n=node, q=partner: lib.mi_memcpy_d2d(scratch[n], values[q], L * 4, s))
        for p in pools:
            mi.check(lib.mi_stream_pool_wait_all(p))
        for node in range(N):
            launch(node, lambda s, n=node: lib.mi_add_f32(values[n], scratch[n], values[n], L, s))
        for p in pools:
            mi.check(lib.mi_stream_pool_wait_all(p))
        r += 1
    assert r == 3
    out = np.empty(L, np.float32)
    for i in range(N):
        mi.check(lib.mi_memcpy_d2h(out.ctypes.data, values[i], out.nbytes, None))
        mi.check(lib.mi_stream_synchronize(None))
        assert np.all(out == N * (N + 1) // 2)
    for p in pools:
        mi.check(lib.mi_stream_pool_destroy(p))
    mi.check(lib.mi_arena_destroy(a))


def test_pinned_host_staging_and_events(mi, ctx):
    lib = mi.lib
    p = lib.mi_host_alloc(1 << 20)
    assert p
    a = C.c_void_p()
    mi.check(lib.mi_arena_create(ctx, 2 << 20, 256, C.byref(a)))
    d = lib.mi_arena_alloc(a, 1 << 20)
    src = (C.c_uint8 * (1 << 20)).from_address(p)
    C.memset(p, 0x5a, 1 << 20)
    e0, e1 = mi.Event(), mi.Event()
    e0.record()
    mi.check(lib.mi_memcpy_h2d(d, p, 1 << 20, None))
    C.memset(p, 0, 0)
    e1.record()
    e1.synchronize()
    assert e0.elapsed_ms(e1) >= 0.0
    back = np.zeros(1 << 20, np.uint8)
    mi.check(lib.mi_memcpy_d2h(back.ctypes.data, d, 1 << 20, None))
    mi.check(lib.mi_stream_synchronize(None))
    assert np.all(back == 0x5a) and src[0] == 0x5a
    e0.destroy(); e1.destroy()
    mi.check(lib.mi_host_free(p))
    mi.check(lib.mi_arena_destroy(a))


def test_host_arena_is_the_same_allocator_on_pinned_memory(mi, ctx):
    """The pinned staging slab answers every arena call like the device slab (numa_arena.mojo:40-87), reads as
    zero when fresh, sits on the node it was bound to, and feeds asynchronous copies."""
    lib = mi.lib
    h = C.c_void_p()
    mi.check(lib.mi_host_arena_create(ctx, 4 << 20, 256, 0, C.byref(h)))       # bound to NUMA node 0
    assert lib.mi_arena_used(h) == 0 and lib.mi_arena_remaining(h) == 4 << 20
    assert lib.mi_arena_verify_placement(h) == 1                               # nothing allocated: true
    p1 = lib.mi_arena_alloc(h, 1000)
    p2 = lib.mi_arena_alloc(h, 1 << 20)
    assert p1 and p2 and p1 % 256 == 0 and p2 - p1 == 1024
    assert lib.mi_arena_verify_placement(h) == 1                               # pinned, and on node 0 where the kernel can tell
    fresh = np.frombuffer((C.c_uint8 * (1 << 20)).from_address(p2), np.uint8)
    assert not fresh.any()
    mark = lib.mi_arena_mark(h)
    p3 = lib.mi_arena_alloc(h, 4096)
    assert lib.mi_arena_reset_to(h, mark + (1 << 30)) == mi.EINVAL
    assert lib.mi_arena_reset_to(h, mark) == mi.OK
    assert lib.mi_arena_alloc(h, 4096) == p3
    assert lib.mi_arena_alloc(h, 8 << 20) is None                              # exhausted: null, no error
    # host slab -> device -> host slab, all asynchronous on one stream
    rng = np.random.default_rng(5)
    fresh[:] = rng.integers(0, 256, 1 << 20, dtype=np.uint8)
    want = fresh.copy()
    a = C.c_void_p()
    mi.check(lib.mi_arena_create(ctx, 2 << 20, 256, C.byref(a)))
    d = lib.mi_arena_alloc(a, 1 << 20)
    lib.mi_arena_reset_to(h, mark)
    back_p = lib.mi_arena_alloc(h, 1 << 20)
    mi.check(lib.mi_memcpy_h2d(d, p2, 1 << 20, None))
    mi.check(lib.mi_memcpy_d2h(back_p, d, 1 << 20, None))
    mi.check(lib.mi_stream_synchronize(None))
    back = np.frombuffer((C.c_uint8 * (1 << 20)).from_address(back_p), np.uint8)
    assert np.array_equal(back, want)
    unbound = C.c_void_p()
    mi.check(lib.mi_host_arena_create(ctx, 1 << 20, 64, -1, C.byref(unbound)))  # no binding
    assert lib.mi_arena_alloc(unbound, 64) and lib.mi_arena_verify_placement(unbound) == 1
    bad = C.c_void_p()
    assert lib.mi_host_arena_create(ctx, 1 << 20, 48, 0, C.byref(bad)) == mi.EINVAL
    assert lib.mi_host_arena_create(ctx, 1 << 20, 64, 99, C.byref(bad)) == mi.EINVAL
    del fresh, back
    mi.check(lib.mi_arena_destroy(unbound))
    mi.check(lib.mi_arena_destroy(a))
    mi.check(lib.mi_arena_destroy(h))


def test_graph_replays_match_eager(mi, dev, orc):
    """A captured rotate+quant -> GEMM -> dequant chain replayed four times with
    new inputs between replays; every replay must equal the eager result."""
    import workload
    M, K, N = 16, 1024, 256
    mark = dev.mark()
    pool = mi.StreamPool(dev, 1)
    s = pool.stream(0)
    w = workload.weights(71, N, K)
    dqw, dsw = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
    mi.fwht_quant(dev.upload(w), dqw, dsw, 128)
    dev.sync()                       # pool streams do not order against the null stream
    dx = dev.upload(workload.activations(72, M, K))
    ws = dev.empty(mi.lib.mi_w8a8_linear_workspace_bytes(M, N, K), np.uint8)
    dy, dy_eager = dev.empty((M, N), np.float32), dev.empty((M, N), np.float32)
    mi.linear(dx, dqw, dsw, dy_eager, 128, ws, stream=s)      # eager warm-up sets kernel attributes
    dev.sync(s)
    with mi.Graph.capture(s) as g:
        mi.linear(dx, dqw, dsw, dy, 128, ws, stream=s)
    for rep in range(4):
        x = workload.activations(100 + rep, M, K)
        mi.check(mi.lib.mi_memcpy_h2d(dx.ptr, x.ctypes.data, x.nbytes, s))
        dev.sync(s)
        mi.linear(dx, dqw, dsw, dy_eager, 128, ws, stream=s)
        dev.sync(s)
        want = dev.download(dy_eager, s)
        mi.check(mi.lib.mi_fill_u32(dy.ptr, 0x7fc00000, M * N, s))     # poison the output
        g.launch()
        dev.sync(s)
        got = dev.download(dy, s)
        assert np.array_equal(got, want), rep
    g.destroy()
    pool.destroy()
    assert mi.lib.mi_graph_capture_begin(None) == mi.EINVAL
    dev.reset_to(mark)
