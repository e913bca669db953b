"""The single-process torch front end (one tensor per emulated rank, worked on in place through
sar_adopt_ranks) against the CPU checker and against torch's own sum."""
import numpy as np
import pytest

from conftest import assert_bits_equal, read_golden, report_placement
from oracle import parse_table

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def rank_tensors(n, numel, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return [(torch.rand(numel, generator=g, dtype=torch.float32) * 2 - 1).to(dtype).cuda() for _ in range(n)]


def to_np_bits(t):
    if t.dtype == torch.float32:
        return t.cpu().numpy()
    return t.cpu().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("dtype,name", [(torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")])
def test_all_reduce_in_place_matches_checker(oracle, dtype, name):
    from stragglar_amd.torch_emulation import EmulatedGroup
    n, numel = 8, 7 * 8 * 4096 + 7 * 8
    tensors = rank_tensors(n, numel, dtype, seed=1)
    inputs = [to_np_bits(t).copy() for t in tensors]
    ptrs = [t.data_ptr() for t in tensors]
    group = EmulatedGroup(n)
    try:
        ms = group.all_reduce(tensors)
        assert ms > 0
        assert [t.data_ptr() for t in tensors] == ptrs                      # in place, nothing reallocated
        want = [x.copy() for x in inputs]
        oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
        for r in range(n):
            assert_bits_equal(to_np_bits(tensors[r]), want[r], "rank %d" % r)
        # a second call on the same tensors reuses the lowered plan and sums the sums
        group.all_reduce(tensors)
        oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
        for r in range(n):
            assert_bits_equal(to_np_bits(tensors[r]), want[r], "second call, rank %d" % r)
    finally:
        group.close()


def test_straggler_relabelling_and_comparators(oracle):
    """STRAGGLER_RANK = 6 in the reference (dummy.cpp:157, dp.py:22): whichever rank is late, every rank ends
    with the same sum; the relabelled order decides the association, which the checker reproduces."""
    from stragglar_amd.torch_emulation import EmulatedGroup
    n, numel = 8, 7 * 8 * 1024
    for alg in ("stragglar", "ring", "rhd", "direct"):
        tensors = rank_tensors(n, numel, torch.float32, seed=2)
        inputs = [t.cpu().numpy().copy() for t in tensors]
        group = EmulatedGroup(n, straggler_rank=6, algorithm=alg)
        try:
            group.all_reduce(tensors)
        finally:
            group.close()
        order = list(range(n))
        order[6], order[7] = order[7], order[6]
        want = [inputs[i].copy() for i in order]
        oracle.run(alg, want, "f32", rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
        for k, i in enumerate(order):
            assert_bits_equal(tensors[i].cpu().numpy(), want[k], "%s rank %d" % (alg, i))
        total = np.sum(np.stack(inputs).astype(np.float64), axis=0)
        assert np.allclose(tensors[0].cpu().numpy(), total, rtol=0, atol=1e-5)


def test_gradient_averaging_like_the_reference_trainer():
    """dp.py:28-65: flatten -> all_reduce(SUM) -> / world_size -> unflatten, for all emulated ranks."""
    from stragglar_amd.torch_emulation import EmulatedGroup
    n = 4
    shapes = [(33, 7), (129,), (5, 5, 5)]
    g = torch.Generator(device="cpu").manual_seed(3)
    group = EmulatedGroup(n)
    try:
        flats = None
        for step in range(3):                      # the flat buffers are the library's and stay from step to step
            grads = [[torch.randn(s, generator=g).cuda() for s in shapes] for _ in range(n)]
            expect = [sum(grads[r][k].double() for r in range(n)) / n for k in range(len(shapes))]
            again = group.allreduce_gradients(grads)
            assert flats is None or [t.data_ptr() for t in again] == [t.data_ptr() for t in flats]
            flats = again
            for r in range(n):
                for k in range(len(shapes)):
                    assert torch.allclose(grads[r][k].double(), expect[k], rtol=0, atol=1e-6)
        # another size, then tensors of the caller's own, then gradients again
        other = [[torch.randn(1000, generator=g).cuda().half()] for _ in range(n)]
        expect = sum(o[0].double() for o in other) / n
        group.allreduce_gradients(other)
        assert torch.allclose(other[2][0].double(), expect, rtol=0, atol=2e-3)
        mine = [torch.full((3 * 1024,), float(r), device="cuda") for r in range(n)]
        group.all_reduce(mine)
        assert all(torch.all(t == 6.0) for t in mine)
        grads = [[torch.randn(s, generator=g).cuda() for s in shapes] for _ in range(n)]
        expect = [sum(grads[r][k].double() for r in range(n)) / n for k in range(len(shapes))]
        group.allreduce_gradients(grads)
        for r in range(n):
            for k in range(len(shapes)):
                assert torch.allclose(grads[r][k].double(), expect[k], rtol=0, atol=1e-6)
    finally:
        group.close()


def test_adopt_rejects_bad_buffers(sarlib):
    import stragglar_amd as sa
    ctx = sarlib.context(0)
    try:
        t = torch.zeros(1024, device="cuda")
        with pytest.raises(sa.SarError):
            ctx.adopt_ranks([t.data_ptr(), t.data_ptr() + 1024], 4096, "f32")        # overlapping
        with pytest.raises(sa.SarError):
            ctx.adopt_ranks([t.data_ptr(), 0], 1024, "f32")                          # null
        host = np.zeros(1024, np.float32)
        with pytest.raises(sa.SarError):
            ctx.adopt_ranks([t.data_ptr(), host.ctypes.data], 1024, "f32")           # host memory
        ctx.adopt_ranks([t.data_ptr(), t.data_ptr() + 2048], 2048, "f32")
        ctx.fill_const(0, 2.0)
        ctx.fill_const(1, 3.0)
        ctx.snapshot()
        ctx.prepare(sarlib.builtin("ring", 2))
        ctx.run(-1.0)
        assert torch.all(t == 5.0)
        ctx.restore()
        assert torch.all(t[:512] == 2.0) and torch.all(t[512:] == 3.0)
    finally:
        ctx.close()


@pytest.mark.parametrize("dtype,name", [(torch.float32, "f32"), (torch.bfloat16, "bf16")])
@pytest.mark.parametrize("shifts", ["same", "mixed"])
def test_rank_tensors_that_start_off_the_vector_boundary(oracle, dtype, name, shifts):
    """Views into a larger allocation, as a caller's flat gradient slices would be: every rank tensor starts a few
    elements past a 16-byte boundary.  With the same distance in all ranks the rows still run as vectors (moved up
    to the boundary, the bytes in front element by element); with different distances they run element by element.
    Either way the bits are the checker's."""
    from stragglar_amd.torch_emulation import EmulatedGroup
    n, numel = 8, 7 * 8 * 515
    for alg in ("stragglar", "ring", "rhd", "direct"):
        g = torch.Generator(device="cpu").manual_seed(11)
        pool = torch.zeros(n * (numel + 64), dtype=dtype, device="cuda")
        tensors = []
        for r in range(n):
            shift = 3 if shifts == "same" else (1, 3, 0, 5, 2, 7, 4, 6)[r]
            v = pool[r * (numel + 64) + shift:r * (numel + 64) + shift + numel]
            v.copy_((torch.rand(numel, generator=g, dtype=torch.float32) * 2 - 1).to(dtype))
            tensors.append(v)
        assert all(t.data_ptr() % 16 for t in tensors if shifts == "same")
        inputs = [to_np_bits(t).copy() for t in tensors]
        group = EmulatedGroup(n, algorithm=alg)
        try:
            group.all_reduce(tensors)
            want = [x.copy() for x in inputs]
            oracle.run(alg, want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")) if alg == "stragglar" else None, delay=0.0)
            for r in range(n):
                assert_bits_equal(to_np_bits(tensors[r]), want[r], "%s %s shifts, rank %d" % (alg, shifts, r))
            # nothing outside the views was touched
            for r in range(n):
                lo, hi = r * (numel + 64), (r + 1) * (numel + 64)
                shift = 3 if shifts == "same" else (1, 3, 0, 5, 2, 7, 4, 6)[r]
                assert torch.all(pool[lo:lo + shift] == 0) and torch.all(pool[lo + shift + numel:hi] == 0)
        finally:
            group.close()


@pytest.fixture()
def c10d_group():
    import torch.distributed as dist
    import stragglar_amd.c10d_backend as sb
    sb.configure(straggler_rank=6)                       # STRAGGLER_RANK of the reference (dummy.cpp:157, dp.py:22)
    dist.init_process_group(sb.BACKEND_NAME, store=dist.HashStore(), rank=0, world_size=1)
    yield sb
    dist.destroy_process_group()


@pytest.mark.parametrize("dtype,name", [(torch.float32, "f32"), (torch.float16, "f16"), (torch.bfloat16, "bf16")])
def test_dist_all_reduce_reaches_the_emulation(c10d_group, oracle, dtype, name):
    """torch.distributed.all_reduce on a backend registered by name, as the reference's callers use theirs
    (example.py:16-30): the rows of one [8, numel] tensor are the emulated ranks, the straggler is rank 6 and
    takes the last place, and every row ends with the checker's bits."""
    import torch.distributed as dist
    n = 8
    numel = c10d_group.padded_numel(100000, n, dtype.itemsize)          # example.py:19
    assert (numel * dtype.itemsize) % (1024 * 7) == 0
    g = torch.Generator(device="cpu").manual_seed(5)
    y = (torch.rand(n, numel, generator=g, dtype=torch.float32) * 2 - 1).to(dtype).cuda()
    inputs = [to_np_bits(y[r]).copy() for r in range(n)]
    work = dist.all_reduce(y, async_op=True)
    assert work.is_completed() and work.wait()
    order = list(range(n))
    order[6], order[7] = order[7], order[6]
    want = [inputs[i].copy() for i in order]
    oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
    for k, i in enumerate(order):
        assert_bits_equal(to_np_bits(y[i]), want[k], "rank %d" % i)
    # a second call on the same tensor sums the sums (dist.all_reduce without async_op returns nothing)
    assert dist.all_reduce(y) is None
    oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
    for k, i in enumerate(order):
        assert_bits_equal(to_np_bits(y[i]), want[k], "second call, rank %d" % i)


def test_dist_all_reduce_leaves_the_tail_as_the_reference_does(c10d_group, oracle):
    """chunkSize = numel / (size - 1) in allreduce_stragglar (dummy.cpp:265): what lies behind the last chunk is
    not reduced.  Other rank counts get groups of their own."""
    import torch.distributed as dist
    for n, numel in ((8, 7 * 300 + 5), (4, 3 * 1000 + 2)):
        y = torch.arange(n * numel, dtype=torch.float32).reshape(n, numel).cuda() % 17
        before = y.clone()
        dist.all_reduce(y)
        body = (numel // (n - 1)) * (n - 1)
        assert torch.equal(y[:, body:], before[:, body:])
        assert torch.equal(y[:, :body], before[:, :body].sum(dim=0, keepdim=True).expand(n, body))     # small integers: exact in any order


def test_rank_tensors_are_placed_by_the_library(oracle):
    """EmulatedGroup.rank_tensors: torch tensors over memory that sar_alloc_ranks allocated and placed (half the
    ranks in another region of HBM from 128 MiB over all ranks), worked on without adoption."""
    from stragglar_amd.torch_emulation import EmulatedGroup
    n, numel = 8, 7 * 8 * 160000                     # 9 M elements per rank: 143 MB over all ranks in bf16, 287 MB in fp32
    group = EmulatedGroup(n, straggler_rank=6)
    try:
        for dtype, name in ((torch.float32, "f32"), (torch.bfloat16, "bf16")):
            tensors = group.rank_tensors(numel, dtype)
            assert len(tensors) == n and all(t.dtype == dtype and t.numel() == numel and t.is_cuda for t in tensors)
            g = torch.Generator(device="cpu").manual_seed(9)
            for t in tensors:
                t.copy_((torch.rand(numel, generator=g, dtype=torch.float32) * 2 - 1).to(dtype))
            inputs = [to_np_bits(t).copy() for t in tensors]
            group.all_reduce(tensors)
            st = group._ctx.stats()
            why = "reason %d, %d candidates, probe %.1f us within a region, %.1f us for the pair, %.1f GiB held" % (
                st.spread_reason, st.spread_candidates, st.spread_same_ms * 1e3, st.spread_pair_ms * 1e3, st.spread_search_bytes / 2.0 ** 30)
            assert st.arena_spread == (1 if st.spread_reason == 0 else 0), why
            report_placement("rank_tensors %s" % name, st, why)
            order = list(range(n))
            order[6], order[7] = order[7], order[6]
            want = [inputs[i].copy() for i in order]
            oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
            for k, i in enumerate(order):
                assert_bits_equal(to_np_bits(tensors[i]), want[k], "%s rank %d" % (name, i))
    finally:
        group.close()


def test_data_parallel_step_through_dist_all_reduce(c10d_group):
    """The reference trainer's gradient exchange (dp.py:28-65: flatten the gradients, dist.all_reduce(SUM), divide by
    the world size, copy back) with eight replicas of a small model emulated on one GPU: the flat gradient buffers are the
    rows of one tensor, padded as example.py:19 pads, and after the step every replica holds the mean gradient."""
    import torch.distributed as dist
    n = 8
    torch.manual_seed(0)
    proto = torch.nn.Sequential(torch.nn.Linear(37, 64), torch.nn.Tanh(), torch.nn.Linear(64, 11)).cuda()
    replicas = []
    for r in range(n):
        m = torch.nn.Sequential(torch.nn.Linear(37, 64), torch.nn.Tanh(), torch.nn.Linear(64, 11)).cuda()
        m.load_state_dict(proto.state_dict())
        x = torch.randn(16, 37, device="cuda", generator=torch.Generator(device="cuda").manual_seed(100 + r))
        m(x).square().mean().backward()
        replicas.append(m)
    grads = [[p.grad for p in m.parameters()] for m in replicas]
    numel = sum(g.numel() for g in grads[0])
    padded = c10d_group.padded_numel(numel, n, 4)
    flat = torch.zeros(n, padded, device="cuda")                       # flatten_tensors (dp.py:28-39), one row per replica
    for r in range(n):
        flat[r, :numel] = torch.cat([g.reshape(-1) for g in grads[r]])
    want = flat[:, :numel].double().sum(dim=0) / n
    dist.all_reduce(flat, op=dist.ReduceOp.SUM)                        # dp.py:59
    flat /= n                                                          # dp.py:60
    for r in range(n):                                                 # unflatten_tensors + copy back (dp.py:41-65)
        off = 0
        for g in grads[r]:
            g.copy_(flat[r, off:off + g.numel()].view_as(g))
            off += g.numel()
    for r in range(n):
        got = torch.cat([p.grad.reshape(-1) for p in replicas[r].parameters()]).double()
        assert torch.allclose(got, want, rtol=1e-6, atol=1e-9), "replica %d" % r
        assert torch.equal(flat[r], flat[0])                           # every replica holds the same bits


def test_rank_block_is_one_tensor_in_two_regions(oracle):
    """EmulatedGroup.rank_block: the emulated ranks as the rows of ONE contiguous tensor in memory the library maps
    (sar_alloc_rows: two physical allocations in different regions of HBM side by side in one virtual range), worked
    on in place, bit for bit the checker's result; a small block is a plain allocation."""
    from stragglar_amd.capi import SPREAD_REASONS
    from stragglar_amd.torch_emulation import EmulatedGroup
    n = 8
    group = EmulatedGroup(n, straggler_rank=6)
    try:
        for numel, dtype, name in ((7 * 8 * 160000, torch.float32, "f32"), (7 * 512, torch.float32, "f32"), (7 * 8 * 160000, torch.bfloat16, "bf16")):
            y = group.rank_block(numel, dtype)
            assert y.shape == (n, numel) and y.dtype == dtype and y.is_cuda and y.is_contiguous()
            assert y[1].data_ptr() - y[0].data_ptr() == numel * dtype.itemsize
            _, placed, reason = group._ctx.alloc_rows(n, numel * dtype.itemsize)        # the same request again: same verdict
            y = group.rank_block(numel, dtype)
            big = n * numel * dtype.itemsize >= 128 << 20
            # (that a block of this size IS placed on a 288 GiB device is asserted where the entry point is tested by
            # itself, tests/test_gpu_parity.py::test_rows_in_one_virtual_range; here other contexts hold memory around it)
            assert placed == (reason == 0) and group.block_placed == placed and (big or not placed), SPREAD_REASONS.get(reason, "?")
            g = torch.Generator(device="cpu").manual_seed(11)
            y.copy_((torch.rand(n, numel, generator=g, dtype=torch.float32) * 2 - 1).to(dtype))
            inputs = [to_np_bits(y[r]).copy() for r in range(n)]
            group.all_reduce([y[r] for r in range(n)])
            group.all_reduce([y[r] for r in range(n)])        # the second call finds the rows adopted and sums the sums
            order = list(range(n))
            order[6], order[7] = order[7], order[6]
            want = [inputs[i].copy() for i in order]
            for _ in range(2):
                oracle.run("stragglar", want, name, rounds=parse_table(read_golden("synth_pow2_n8.txt")), delay=0.0)
            for k, i in enumerate(order):
                assert_bits_equal(to_np_bits(y[i]), want[k], "%s %d rank %d" % (name, numel, i))
        # tensors of the library's own arena, in another order than they were handed out, are refused rather than
        # adopted (adoption gives the arena back)
        import stragglar_amd as sa
        ts = group.rank_tensors(7 * 1024, torch.float32)
        with pytest.raises(sa.SarError, match="own rank arena"):
            group.all_reduce(ts[::-1])
    finally:
        group.close()


def test_dist_all_reduce_on_rows_the_library_placed(c10d_group):
    """empty_ranks: the [n, numel] tensor for dist.all_reduce in memory of the library's (two regions of HBM from
    128 MiB in all); the result as for any other tensor."""
    import torch.distributed as dist
    n = 8
    numel = c10d_group.padded_numel(5_000_000, n, 4)                  # 160 MB in all
    y = c10d_group.empty_ranks(n, numel)
    assert y.shape == (n, numel) and y.is_contiguous()
    y.copy_((torch.arange(n * numel, device="cuda") % 13).reshape(n, numel).float())
    want = y.sum(dim=0, keepdim=True).expand(n, numel).clone()        # small integers: exact in any order
    dist.all_reduce(y)
    assert torch.equal(y, want)
    z = c10d_group.empty_ranks(4, 3 * 256, torch.float16)             # another rank count has a block of its own
    z.fill_(1.0)
    dist.all_reduce(z)
    assert torch.all(z == 4.0) and torch.equal(y, want)
