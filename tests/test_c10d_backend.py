"""The c10d backend name (host side, no GPU): registration as the reference registers "dummy"
(implementation/custom_backend/include/dummy.hpp:106-111), the one-process rule, "not supported" for
everything but allreduce (src/dummy.cpp:731-811), and the padding rule of example.py:19."""
import math

import pytest

torch = pytest.importorskip("torch")
dist = pytest.importorskip("torch.distributed")


@pytest.fixture()
def group():
    import stragglar_amd.c10d_backend as sb
    sb.configure()
    dist.init_process_group(sb.BACKEND_NAME, store=dist.HashStore(), rank=0, world_size=1)
    yield sb
    dist.destroy_process_group()


def test_backend_is_registered_by_import():
    import stragglar_amd.c10d_backend as sb
    assert sb.BACKEND_NAME == "stragglar"
    assert hasattr(dist.Backend, sb.BACKEND_NAME.upper())
    sb.register()                                            # a second call is harmless


def test_one_process_carries_all_ranks():
    import stragglar_amd.c10d_backend as sb
    with pytest.raises(RuntimeError, match="ONE process"):
        sb.create_backend(None, 1, 8, None)


def test_only_allreduce_is_supported(group):
    t = torch.zeros(8, 14)
    for call in (lambda: dist.broadcast(t, 0), lambda: dist.barrier(), lambda: dist.reduce(t, 0),
                 lambda: dist.all_gather_into_tensor(torch.zeros(8, 14), t),
                 lambda: dist.reduce_scatter_tensor(torch.zeros(14), t), lambda: dist.all_to_all_single(torch.zeros(8, 14), t)):
        with pytest.raises(RuntimeError, match="not supported|Invalid"):
            call()
    # the zero-filling allgather of the reference (dummy.cpp:233-247)
    outs = [torch.ones(8, 14)]
    dist.all_gather(outs, t)
    assert float(outs[0].abs().sum()) == 0.0
    # allreduce itself: there is no CPU path, and the shape rule is spelled out
    with pytest.raises(RuntimeError, match="CUDA"):
        dist.all_reduce(t)
    with pytest.raises(RuntimeError, match="emulated ranks, elements per rank"):
        dist.all_reduce(torch.zeros(14))
    with pytest.raises(RuntimeError, match="not supported"):
        dist.all_reduce(t, op=dist.ReduceOp.MAX)
    work = None
    with pytest.raises(RuntimeError):
        work = dist.all_reduce(t, async_op=True)
    assert work is None


def test_padding_rule_of_the_reference_example():
    from stragglar_amd.torch_emulation import padded_numel
    for size in (1024 ** 3 // 4, 1, 7 * 256, 7 * 256 + 1, 12345678):
        want = math.ceil(size * 4 / (1024 * 7)) * 1024 * 7 // 4          # example.py:19
        assert padded_numel(size, 8, 4) == want
    assert padded_numel(1000, 8, 2) % (7 * 512) == 0                     # 16-bit elements: chunks of whole KiB as well
    assert padded_numel(1000, 8, 4, parts=8) % (8 * 256) == 0            # ring / rhd cut the buffer in n


def test_completed_work():
    import stragglar_amd.c10d_backend as sb
    w = sb.CompletedWork([torch.zeros(2)])
    assert w.is_completed() and w.is_success() and w.wait()
    assert w.get_future().wait()[0].shape == (2,)
