"""The reference-named operator surface: send / recv / sync, argument checks,
asynchronous launch, benchmark configuration 2 (256 MiB sendrecv) and the
allgather sweep of configuration 5."""
import numpy as np
import pytest
import torch

from oracle import ring
from tests.helpers import as_bytes, normal, rank_rows, uniform

pytestmark = pytest.mark.gpu


def make_comm(world, **kw):
    from mintccl_amd.common import VirtualComm
    kw.setdefault("spin_budget", 400000)
    return VirtualComm(world_size=world, **kw)


@pytest.mark.parametrize("nbytes", [2, 4096, (1 << 20) + 6])
def test_direct_send_recv(dev, nbytes):
    from mintccl_amd import sendrecv_direct as m
    comm = make_comm(2)
    src = normal(nbytes // 2, 1).to(dev)
    dst = torch.zeros_like(src)
    with comm.rank(0):
        m.send(src, 1, comm)
    with comm.rank(1):
        m.recv(dst, 0, comm=comm)
    assert torch.equal(dst.view(torch.int16), src.view(torch.int16))


@pytest.mark.parametrize("module", ["sendrecv_buffer", "sendrecv_indirect"])
@pytest.mark.parametrize("route", [None, [0, 2, 1], [0, 3, 2, 1]])
@pytest.mark.parametrize("n", [1, 123457])
def test_deferred_send_recv_sync(dev, module, route, n):
    import importlib
    m = importlib.import_module(f"mintccl_amd.{module}")
    comm = make_comm(4)
    src = torch.randn(n, generator=torch.Generator().manual_seed(n)).to(dev)   # fp32 like the reference test
    dst = torch.zeros_like(src)
    with comm.rank(0):
        m.send(src, 1, comm)
    with comm.rank(1):
        m.recv(dst, 0, comm)
    for r in range(4):                      # everyone calls sync (3_sendrecv_buffer.py:98)
        with comm.rank(r):
            m.sync(comm, route=route)
    comm.check()
    assert torch.equal(dst.view(torch.int32), src.view(torch.int32))


def test_sync_rejects_mismatched_pairs(dev):
    from mintccl_amd import sendrecv_buffer as m
    comm = make_comm(2)
    a = torch.zeros(16, device=dev)
    b = torch.zeros(32, device=dev)
    with comm.rank(0):
        m.send(a, 1, comm)
    with comm.rank(1):
        m.recv(b, 0, comm)
    with pytest.raises(ValueError):
        m.sync(comm)


def test_config2_sendrecv_256mib_ll128_and_simple(dev):
    # 134,217,728 fp16 normal(0,1) seed 1, rank 0 -> rank 1, 512 KiB slots
    from mintccl_amd import sendrecv_buffer as m, sendrecv_direct as direct
    src = normal(134217728, 1).to(dev)
    for proto in (0, 1):
        comm = make_comm(2, buff_size_=8 * 512 * 1024, nslots=8, protocol=proto)
        dst = torch.zeros_like(src)
        with comm.rank(0):
            m.send(src, 1, comm)
        with comm.rank(1):
            m.recv(dst, 0, comm)
        m.sync(comm)
        comm.check()
        assert torch.equal(dst.view(torch.int16), src.view(torch.int16))
    comm = make_comm(2)
    dst = torch.zeros_like(src)
    with comm.rank(0):
        direct.send(src, 1, comm)
    with comm.rank(1):
        direct.recv(dst, 0, comm=comm)
    assert torch.equal(dst.view(torch.int16), src.view(torch.int16))


@pytest.mark.parametrize("proto", [0, 1])
def test_config5_allgather_sweep(dev, proto):
    """Every power of two from 512 B to 128 MiB per rank shard, LL128 and
    Simple, fixed 8 x 512 KiB staging.  Up to 4 MiB the inputs are drawn on the
    host (uniform[-1, 1], seed 4 + rank) and every row is compared on the
    host; above that they are drawn on the device and compared there:
    row c of every rank must be rank c's row c, every byte of it."""
    from mintccl_amd.allgather import allgather
    world = 8
    comm = make_comm(world, buff_size_=8 * 512 * 1024, nslots=8, protocol=proto)
    for log2 in range(9, 28):
        n = (1 << log2) // 2
        if log2 <= 22:
            host = [uniform(world * n, -1.0, 1.0, 4 + r).reshape(world, n) for r in range(world)]
            bufs = [h.to(dev) for h in host]
            own = [host[c][c].to(dev) for c in range(world)]
        else:
            bufs = []
            for r in range(world):
                g = torch.Generator(device=dev).manual_seed(4 + r)
                bufs.append((torch.rand(world, n, generator=g, device=dev) * 2 - 1).to(torch.float16))
            own = [bufs[c][c].clone() for c in range(world)]
        comm.run(lambda r: allgather(bufs[r], comm))
        comm.check()
        for r in range(world):
            for c in range(world):
                assert torch.equal(bufs[r][c].view(torch.int16), own[c].view(torch.int16)), (log2, r, c)
        del bufs, own


def test_argument_checks(dev):
    from mintccl_amd.reduce import reduce
    from mintccl_amd.reducescatter import reducescatter
    comm = make_comm(2)
    with comm.rank(0):
        with pytest.raises(TypeError):
            reduce(torch.zeros(8, dtype=torch.int32, device=dev), 0, comm)
        with pytest.raises(TypeError):
            reduce(torch.zeros(8, dtype=torch.float16), 0, comm)          # host tensor
        with pytest.raises(ValueError):
            reducescatter(torch.zeros(3, 3, dtype=torch.float16, device=dev), comm)
        with pytest.raises(ValueError):
            reduce(torch.zeros(8, 8, dtype=torch.float16, device=dev).t(), 0, comm)
    with pytest.raises(RuntimeError):
        comm.Get_rank()                                                   # outside a rank context
    a = torch.zeros(8, dtype=torch.float16, device=dev)
    b = torch.zeros(16, dtype=torch.float16, device=dev)
    with comm.rank(0):
        reduce(a, 0, comm)
    with comm.rank(1):
        with pytest.raises(ValueError):
            reduce(b, 0, comm)                                            # ranks disagree on size


def test_world_of_one_is_a_no_op(dev):
    from mintccl_amd.reducescatter import reducescatter
    from mintccl_amd.broadcast import broadcast
    comm = make_comm(1)
    x = normal(4096, 0).to(dev).reshape(1, -1)
    y = x.clone()
    with comm.rank(0):
        reducescatter(x, comm)
        broadcast(x, 0, comm)
    comm.check()
    assert torch.equal(x, y)


def test_launch_is_asynchronous_and_stream_ordered(dev):
    # the operator enqueues on the current stream and returns; a later kernel
    # on the same stream sees the result
    from mintccl_amd.broadcast import broadcast
    world, n = 8, 1 << 22
    comm = make_comm(world)
    s = torch.cuda.Stream(device=dev)
    host = uniform(n, -4.0, 4.0, 9)
    with torch.cuda.stream(s):
        bufs = [host.to(dev, non_blocking=False) if r == 3 else
                torch.zeros(n, dtype=torch.float16, device=dev) for r in range(world)]
        comm.run(lambda r: broadcast(bufs[r], 3, comm))
        total = torch.stack([b.float().sum() for b in bufs])
    s.synchronize()
    comm.check()
    want = host.to(dev).float().sum()
    assert torch.all(total == want)


@pytest.mark.gpu
@pytest.mark.parametrize("world,count", [(8, 1 << 20), (4, (1 << 18) + 24), (2, 65536)])
def test_reference_style_self_tests_pass(monkeypatch, capsys, world, count):
    """MINTCCL_TEST_MODE=1 python -m mintccl_amd.<op>: every collective prints
    `equal: True` against the same collective done with plain torch operations
    (the reference compares with torch.distributed, 4_broadcast.py:111-126)."""
    from mintccl_amd import selftest
    monkeypatch.setenv("MINTCCL_TEST_MODE", "1")
    monkeypatch.setenv("MINTCCL_TEST_COUNT", str(count))
    monkeypatch.setenv("MINTCCL_WORLD_SIZE", str(world))
    monkeypatch.setenv("ROOT_TEMP", str(world - 1))
    monkeypatch.setenv("DST_TEMP", str(world - 1))
    assert selftest.main("all") == 0
    out = capsys.readouterr().out
    assert "equal: False" not in out
    # 3 point-to-point tests, broadcast, allgather, allreduce and alltoall on every
    # rank, reduce at the root, reducescatter on every rank; then the tree's
    # broadcast on every rank and its reduce at the root, the hypercube's
    # reducescatter and allgather on every rank
    assert out.count("equal: True") == 3 + 4 * world + 1 + world + world + 1 + 2 * world


@pytest.mark.gpu
def test_device_epoch_wraps_and_clears(dev):
    """With the epoch in device memory every launch advances it; when it starts
    over the staging is cleared, so results stay right across the wrap."""
    from mintccl_amd.reducescatter import reducescatter
    world, n = 4, 3000
    comm = make_comm(world, device_epoch=True)
    host = rank_rows(world, n, "f16")
    want = ring.reducescatter([as_bytes(h) for h in host], "f16")
    bufs = [h.to(dev) for h in host]
    seen = []
    for i in range(6):
        if i == 2:
            comm.epoch_word[0] = 4094            # two launches before the count starts over
        for b, h in zip(bufs, host):
            b.copy_(h)
        comm.run(lambda r: reducescatter(bufs[r], comm))
        comm.check()
        seen.append(int(comm.epoch_word[0].item()))
        assert all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want)), i
    assert seen == [1, 2, 4095, 1, 2, 3]


@pytest.mark.gpu
@pytest.mark.parametrize("world", [3, 6, 7])
@pytest.mark.parametrize("knobs", [
    {},
    {"MINTCCL_PROTOCOL": "simple"},
    {"MINTCCL_PLACEMENT": "spread", "MINTCCL_CACHE": "agent"},
    {"MINTCCL_TOPOLOGY": "tree", "MINTCCL_ALLGATHER": "temporal"},
    {"MINTCCL_ALLREDUCE": "split", "MINTCCL_NSLOTS": "2", "MINTCCL_BUFFSIZE": "262144"},
    {"MINTCCL_DEVICE_EPOCH": "1", "ROOT_TEMP": "1"},
])
def test_self_tests_over_world_sizes_and_knobs(monkeypatch, capsys, world, knobs):
    """Every operator's self-test under the environment knobs a user can set,
    on world sizes the other tests do not visit."""
    from mintccl_amd import selftest
    monkeypatch.setenv("MINTCCL_TEST_MODE", "1")
    monkeypatch.setenv("MINTCCL_TEST_COUNT", str((1 << 18) + 8 * world))
    monkeypatch.setenv("MINTCCL_WORLD_SIZE", str(world))
    for k, v in knobs.items():
        monkeypatch.setenv(k, v)
    assert selftest.main("all") == 0
    out = capsys.readouterr().out
    assert "equal: False" not in out
    assert out.count("equal: True") == 3 + 4 * world + 1 + world + world + 1


@pytest.mark.gpu
def test_captured_large_collectives_replay(dev):
    """The same for messages large enough for the tuned launches with compute
    units set apart for the origins (allgather in both schedules, broadcast,
    sendrecv over one hop, alltoall): three replays against eager runs."""
    from mintccl_amd import sendrecv_buffer
    from mintccl_amd.allgather import allgather
    from mintccl_amd.alltoall import alltoall
    from mintccl_amd.broadcast import broadcast
    world, n = 8, (1 << 20) + 40
    comm = make_comm(world, device_epoch=True)
    eager = make_comm(world)
    ins = [torch.zeros(world, n, dtype=torch.float16, device=dev) for _ in range(world)]

    def buffers():
        return ([torch.zeros_like(x) for x in ins], [torch.zeros_like(x) for x in ins],
                [torch.zeros(world * n, dtype=torch.float16, device=dev) for _ in range(world)],
                [torch.zeros_like(x) for x in ins], [torch.zeros_like(x) for x in ins])

    def sequence(cm, a, t, c, x, y):
        for r in range(world):
            a[r].copy_(ins[r]); t[r].copy_(ins[r]); c[r].copy_(ins[r].view(-1)); x[r].copy_(ins[r])
        cm.run(lambda r: allgather(a[r], cm))
        cm.run(lambda r: allgather(t[r], cm, schedule="temporal"))
        cm.run(lambda r: broadcast(c[r], 5, cm))
        cm.run(lambda r: alltoall(x[r], y[r], cm))
        with cm.rank(2):
            sendrecv_buffer.send(a[2], 6, cm)     # the gathered rows land in rank 6's alltoall input
        with cm.rank(6):
            sendrecv_buffer.recv(x[6], 2, cm)
        cm.run(lambda r: sendrecv_buffer.sync(cm))

    def fill(seed):
        for r, h in enumerate(rank_rows(world, n, "f16", seed0=seed)):
            ins[r].copy_(h.to(dev))

    fill(300)
    got, want = buffers(), buffers()
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        sequence(comm, *got)                      # warm up outside the capture
    side.synchronize()
    comm.check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sequence(comm, *got)
    for replay in range(3):
        fill(400 + 10 * replay)
        sequence(eager, *want)
        eager.check()
        graph.replay()
        torch.cuda.synchronize()
        comm.check()
        for g, w in zip(got, want):
            for r in range(world):
                assert torch.equal(g[r], w[r]), replay
    # sanity of what was compared: the allgathers gathered, the broadcast spread rank 5's buffer
    assert all(torch.equal(want[0][r][q], ins[q][q]) for r in range(world) for q in range(world))
    assert all(torch.equal(want[1][r], want[0][r]) for r in range(world))
    assert torch.equal(want[3][6], want[0][2]) and torch.equal(want[3][5], ins[5])


def test_captured_collectives_replay(dev):
    """A captured sequence of collectives (epoch in device memory) is replayed
    several times, with eager work and fresh inputs in between; every replay
    must equal the eager result."""
    from mintccl_amd.allgather import allgather
    from mintccl_amd.allreduce import allreduce
    from mintccl_amd.broadcast import broadcast
    world, n = 8, 4096 + 24
    comm = make_comm(world, device_epoch=True)
    eager = make_comm(world)
    ins = [torch.zeros(world, n, dtype=torch.float16, device=dev) for _ in range(world)]
    a = [torch.zeros_like(x) for x in ins]
    b = [torch.zeros(world * n, dtype=torch.float16, device=dev) for _ in range(world)]
    c = [torch.zeros(n, dtype=torch.float16, device=dev) for _ in range(world)]

    def sequence(cm, a, b, c):
        for r in range(world):
            a[r].copy_(ins[r]); b[r].copy_(ins[r].view(-1)); c[r].copy_(ins[r][r])
        cm.run(lambda r: allgather(a[r], cm))
        cm.run(lambda r: allreduce(b[r], cm))
        cm.run(lambda r: broadcast(c[r], 3, cm))

    def fill(seed):
        for r, h in enumerate(rank_rows(world, n, "f16", seed0=seed)):
            ins[r].copy_(h.to(dev))

    fill(100)
    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        sequence(comm, a, b, c)                   # warm up outside the capture
    side.synchronize()
    comm.check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sequence(comm, a, b, c)
    ea, eb, ec = [torch.zeros_like(x) for x in a], [torch.zeros_like(x) for x in b], [torch.zeros_like(x) for x in c]
    for replay in range(5):
        fill(200 + 10 * replay)
        sequence(eager, ea, eb, ec)
        eager.check()
        graph.replay()
        torch.cuda.synchronize()
        comm.check()
        for r in range(world):
            assert torch.equal(a[r], ea[r]) and torch.equal(b[r], eb[r]) and torch.equal(c[r], ec[r]), replay


@pytest.mark.gpu
def test_local_placement_on_a_stream_confined_to_half_of_the_compute_units(dev):
    """Thread blocks claim their seats whatever compute units they land on: on
    a stream with a CU mask every compute unit in use gets twice its share of
    the blocks, and the launches (several rounds over the compute units, with
    and without compute units set apart for origins) still seat every block."""
    import ctypes
    from mintccl_amd import _lib
    from mintccl_amd.allgather import allgather
    from mintccl_amd.common import VirtualComm
    from mintccl_amd.reducescatter import reducescatter
    hip = ctypes.CDLL("libamdhip64.so")
    words = (ctypes.c_uint32 * 8)(*([0x00FF00FF] * 8))
    handle = ctypes.c_void_p()
    assert hip.hipExtStreamCreateWithCUMask(ctypes.byref(handle), 8, words) == 0
    stream = torch.cuda.ExternalStream(handle.value)
    world, n = 8, 100003
    comm = VirtualComm(world_size=world, device=dev, spin_budget=4000000)
    assert comm.placement == _lib.PLACE_LOCAL
    host = rank_rows(world, n, "f16", 8100)
    bufs = [h.to(dev) for h in host]
    torch.cuda.synchronize(dev)
    with torch.cuda.stream(stream):
        for _ in range(2):          # the second launch finds the counters as the first left them
            for b, h in zip(bufs, host):
                b.copy_(h, non_blocking=False)
            comm.run(lambda r: reducescatter(bufs[r], comm))
            assert comm.last_grid >= 8 * 64
        comm.check()
        want = ring.reducescatter([as_bytes(h) for h in host], "f16")
        assert all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want))
        comm.run(lambda r: allgather(bufs[r], comm))
        assert comm.last_grid >= 8 * 64
        comm.check()
        for b, w in zip(bufs, ring.allgather(want)):
            assert np.array_equal(as_bytes(b), w)
    # and the same communicator on an ordinary stream afterwards
    for b, h in zip(bufs, host):
        b.copy_(h)
    comm.run(lambda r: reducescatter(bufs[r], comm))
    comm.check()
    assert all(np.array_equal(as_bytes(b), w) for b, w in zip(bufs, want))
    torch.cuda.synchronize(dev)
    assert hip.hipStreamDestroy(handle) == 0


@pytest.mark.gpu
def test_local_placement_beside_another_streams_kernels(dev):
    """A collective under the local placement while matrix products of another
    stream hold part of the compute units: the thread blocks land on whatever
    units have room, in whatever numbers, and still find their seats."""
    from mintccl_amd import _lib
    from mintccl_amd.allgather import allgather
    from mintccl_amd.common import VirtualComm
    from mintccl_amd.reducescatter import reducescatter
    world, n = 8, 524309
    comm = VirtualComm(world_size=world, device=dev, spin_budget=4000000)
    assert comm.placement == _lib.PLACE_LOCAL
    host = rank_rows(world, n, "f16", 8200)
    want = ring.reducescatter([as_bytes(h) for h in host], "f16")
    gathered = ring.allgather(want)
    bufs = [h.to(dev) for h in host]
    a = torch.randn(8192, 8192, device=dev, dtype=torch.float16)
    other = torch.cuda.Stream(device=dev)
    for _ in range(4):
        for b, h in zip(bufs, host):
            b.copy_(h)
        torch.cuda.synchronize(dev)
        with torch.cuda.stream(other):
            for _ in range(6):
                a @ a
        comm.run(lambda r: reducescatter(bufs[r], comm))
        assert comm.last_grid >= 8 * 64
        comm.run(lambda r: allgather(bufs[r], comm))
        comm.check()
        other.synchronize()
        for b, w in zip(bufs, gathered):
            assert np.array_equal(as_bytes(b), w)


@pytest.mark.gpu
def test_captured_ll128_launch_replayed_after_an_eager_simple_launch(dev):
    """A communicator with its epoch in device memory: an LL128 allgather is
    captured while the launch before it was LL128 too; between the replays an
    eager Simple broadcast on the same communicator leaves payload in the
    slots that would pass for sector tags.  The kernel that advances the epoch
    clears them when the graph runs - the host took no such decision when the
    graph was captured - so every replay equals the eager result."""
    from mintccl_amd import _lib
    from mintccl_amd.allgather import allgather
    world, n = 8, 52000
    comm = make_comm(world, device_epoch=True)
    ins = [torch.zeros(world, n, dtype=torch.float16, device=dev) for _ in range(world)]
    g = [torch.zeros_like(x) for x in ins]

    def sequence():
        for r in range(world):
            g[r].copy_(ins[r])
        comm.run(lambda r: allgather(g[r], comm))

    side = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(side):
        sequence()
    side.synchronize()
    comm.check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sequence()
    n32 = 1 << 18
    src = torch.arange(n32, dtype=torch.int64)
    forged = ((((src // 256) % 4095 + 1) << 20) | 1).to(torch.int32)
    bc = [forged.to(dev) if r == 0 else torch.zeros(n32, dtype=torch.int32, device=dev)
          for r in range(world)]
    ptrs = {r: bc[r].data_ptr() for r in range(world)}
    for replay in range(4):
        host = [uniform(world * n, -1.0, 1.0, 700 + 10 * replay + r).reshape(world, n)
                for r in range(world)]
        for r in range(world):
            ins[r].copy_(host[r].to(dev))
        if replay % 2 == 0:
            d = comm.make_op(_lib.OP_BROADCAST, _lib.BYTES, n32 * 4, {0: ptrs[0]},
                             {r: ptrs[r] for r in range(1, world)}, list(range(world)) + [0],
                             root=0, protocol=_lib.PROTO_SIMPLE)
            comm.launch(d)
            comm.check()
            for t in bc:
                assert torch.equal(t.cpu(), forged)
        graph.replay()
        torch.cuda.synchronize()
        comm.check()
        for r in range(world):
            for c in range(world):
                assert torch.equal(g[r][c].cpu(), host[c][c]), (replay, r, c)
