"""The concurrent sub-batch runner: graphs of the sub-batch forwards replayed side by side on separate streams must
reproduce the eager forwards on every replay (the trap it guards against: graph nodes whose result depends on what else
runs on the GPU -- the library's multi-workgroup mean was one, 5-9 % off on some replays), and match the whole-batch
forward to bf16 accuracy.  The bound is the bf16 parity tolerance, 2e-2 on logits of order one, not bit equality: at
these small batches the library picks convolution kernels that accumulate with atomics and differ in the last place
from run to run, eager or not."""
import pytest
import torch

from vmamba_amd.runner import ConcurrentGraphRunner
from vmamba_amd.vssm import vmamba_tiny_s1l8

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-2


@pytest.fixture(scope="module")
def model():
    torch.manual_seed(0)
    return vmamba_tiny_s1l8(channel_first=False).to(DEV).bfloat16().eval().to(memory_format=torch.channels_last)


# (320 x 320 images: the stage-1 map of 80 x 80 takes more than the default 64 KB of LDS per workgroup)
@pytest.mark.parametrize("batch,size,sub_batches", [(8, 224, 4), (8, 224, 2), (6, 64, 3), (4, 224, 1), (4, 320, 2)])
def test_concurrent_replays_equal_the_eager_forwards(model, batch, size, sub_batches):
    print("CASE runner", batch, size, sub_batches, flush=True)
    x = torch.randn(batch, 3, size, size, device=DEV, generator=torch.Generator(DEV).manual_seed(batch + size)).bfloat16()
    runner = ConcurrentGraphRunner(model, x, sub_batches)
    assert runner.validate(replays=6, atol=TOL)
    with torch.no_grad():
        eager = torch.cat([model(c) for c in x.chunk(sub_batches)])
        whole = model(x)
    for _ in range(3):
        runner.replay()
        torch.cuda.synchronize()
        assert torch.allclose(runner.output().float(), eager.float(), rtol=0, atol=TOL)
    assert torch.allclose(runner.output().float(), whole.float(), rtol=2e-2, atol=2e-2)
    # new inputs go into the captured tensor in place
    x.copy_(torch.randn_like(x))
    runner.replay()
    torch.cuda.synchronize()
    with torch.no_grad():
        assert torch.allclose(runner.output().float(), torch.cat([model(c) for c in x.chunk(sub_batches)]).float(), rtol=0, atol=TOL)


def test_graphs_of_padded_maps_survive_other_map_sizes(model):
    """300 x 300 images give stage maps of 75 x 75 and 19 x 19, which run on padded maps whose added positions are marked by
    a cached 0/1 row; a captured forward holds that row's address.  Forwards on ten other odd sizes push it out of the
    cache of recent sizes; the replays must still reproduce the eager forwards."""
    print("CASE runner padded maps", flush=True)
    x = torch.randn(4, 3, 300, 300, device=DEV, generator=torch.Generator(DEV).manual_seed(300)).bfloat16()
    runner = ConcurrentGraphRunner(model, x, 2)
    assert runner.validate(replays=3, atol=TOL)
    with torch.no_grad():
        for size in (68, 76, 84, 92, 100, 108, 116, 132, 140, 148):          # stage maps 17 / 19 / 21 / 23 / 25 ... : all padded
            model(torch.randn(1, 3, size, size, device=DEV).bfloat16())
        garbage = [torch.full((1 << 20,), float("nan"), device=DEV) for _ in range(8)]   # reuse whatever was freed
        eager = torch.cat([model(c) for c in x.chunk(2)])
    for _ in range(2):
        runner.replay()
        torch.cuda.synchronize()
        assert torch.allclose(runner.output().float(), eager.float(), rtol=0, atol=TOL)
    del garbage


@pytest.mark.parametrize("sub_batches", [2, 4])
def test_benchmark_batch_replays_are_bit_identical(model, sub_batches):
    """The benchmark's own configuration (128 images at 224^2 as 2 or 4 sub-batch graphs side by side): every concurrent
    replay must equal the eager sub-batch forwards bit for bit.  Bit equality presupposes that the eager forward itself
    is reproducible at this sub-batch size (the library may pick kernels that accumulate with atomics); where two eager
    forwards already differ, the replays are held to the bf16 tolerance instead and the test says so."""
    print("CASE runner bench-shape", sub_batches, flush=True)
    x = torch.randn(128, 3, 224, 224, device=DEV, generator=torch.Generator(DEV).manual_seed(sub_batches)).bfloat16()
    with torch.no_grad():
        first = [model(c) for c in x.chunk(sub_batches)]
        second = [model(c) for c in x.chunk(sub_batches)]
        torch.cuda.synchronize()
    reproducible = all(torch.equal(a, b) for a, b in zip(first, second))
    runner = ConcurrentGraphRunner(model, x, sub_batches)
    err = runner.max_replay_error(replays=5)
    print(f"eager forward reproducible: {reproducible}; max replay error {err:g}", flush=True)
    if reproducible:
        assert err == 0.0
    else:
        assert err <= TOL


def test_graph_survives_cache_eviction_and_refuses_stale_weights():
    """A captured forward records the addresses of the per-block constants (A, D, dt bias, repeated projection weights).
    Forwards at five other batch sizes evict them from the blocks' caches; the graphs must still replay correctly.
    After an in-place parameter update the runner must refuse to replay (its graphs hold copies of the old values)."""
    print("CASE runner eviction", flush=True)
    torch.manual_seed(1)
    m = vmamba_tiny_s1l8(channel_first=False).to(DEV).bfloat16().eval().to(memory_format=torch.channels_last)
    x = torch.randn(4, 3, 64, 64, device=DEV, generator=torch.Generator(DEV).manual_seed(9)).bfloat16()
    runner = ConcurrentGraphRunner(m, x, 2)
    with torch.no_grad():
        for b in (1, 3, 5, 6, 7):                   # more batch sizes than a block's cache holds
            m(torch.randn(b, 3, 64, 64, device=DEV).bfloat16())
        garbage = [torch.full((1 << 20,), float("nan"), device=DEV) for _ in range(8)]   # reuse whatever was freed
        torch.cuda.synchronize()
        eager = torch.cat([m(c) for c in x.chunk(2)])
    for _ in range(3):
        runner.replay()
        torch.cuda.synchronize()
        assert torch.allclose(runner.output().float(), eager.float(), rtol=0, atol=TOL)
    del garbage
    block = m.layers[0].blocks[0].op
    with torch.no_grad():
        block.Ds.mul_(2.0)
    assert not runner.parameters_unchanged()
    with pytest.raises(RuntimeError):
        runner.replay()
    # a re-capture after the update pins fresh constants and drops the stale ones instead of piling them up
    runner2 = ConcurrentGraphRunner(m, x, 2)
    pinned = block.__dict__["_pinned_consts"]
    assert len({k[2] for k in pinned}) == 1
    runner2.replay()
    torch.cuda.synchronize()
    # storage replaced without touching the version counter (what .half() / .to() / `param.data = ...` do)
    with torch.no_grad():
        block.Ds.data = block.Ds.data.clone()
    assert not runner2.parameters_unchanged()
    with pytest.raises(RuntimeError):
        runner2.replay()


def test_runner_rejects_uneven_sub_batches(model):
    x = torch.zeros(6, 3, 64, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ConcurrentGraphRunner(model, x, 4)
    with pytest.raises(NotImplementedError):
        ConcurrentGraphRunner(model, x.cpu(), 2)
