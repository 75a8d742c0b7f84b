"""A compiled program's tensors live in ONE device allocation, intermediates sharing bytes by lifetime
(csrc/hlir/memory_plan.h; the reference allocates per tensor, cinn/hlir/framework/memory.cc:43-53, tensor.h:64-82).
The results must not depend on it: the same program with one allocation per tensor gives the same bits."""
import numpy as np
import pytest

import oracle
from cinn_amd.common import Float
from cinn_amd.frontend import NetBuilder

from helpers import run

pytestmark = pytest.mark.gpu


def residual_chain(b, x_shape, widths):
    X = b.create_input(Float(32), x_shape, "x")
    y = X
    mids = []
    for i, w in enumerate(widths):
        W = b.create_input(Float(32), [y.shape()[1], w], "w%d" % i)
        W.set_const()
        z = b.relu(b.matmul(y, W))
        mids.append(z)
        # a value that stays alive across the next layer (the residual), so lifetimes overlap in more than a chain
        y = b.add(z, b.reduce_sum(z, [1], keep_dim=True)) if i % 2 else z
    return X, mids, y


def test_arena_with_shared_intermediates_gives_the_same_bits_as_one_allocation_per_tensor(gpu):
    rng = np.random.default_rng(5)
    widths = [192, 64, 320, 64, 128, 256, 32]
    x = rng.standard_normal((96, 80)).astype(np.float32)
    results = {}
    for mode, opts in (("shared", {}), ("arena", dict(reuse_intermediates=0)), ("plain", dict(memory_arena=0))):
        b = NetBuilder("arena")
        X, mids, y = residual_chain(b, list(x.shape), widths)
        feeds = {X: x}
        cin = x.shape[1]
        wr = np.random.default_rng(6)
        for i, w in enumerate(widths):
            feeds["w%d" % i] = (wr.standard_normal((cin, w)) / np.sqrt(cin)).astype(np.float32)
            cin = w
        (out,), comp = run(b, feeds, [y], **opts)
        arena, unshared = comp.memory_info()
        results[mode] = (out, arena, unshared, comp, mids)
        for _ in range(2):  # a second and third execution, eager and replayed, see the same bytes
            comp.execute()
        assert np.array_equal(comp.get_tensor(y.id).numpy(), out)
    shared, arena, plain = results["shared"], results["arena"], results["plain"]
    assert np.array_equal(shared[0], plain[0]) and np.array_equal(arena[0], plain[0])
    assert plain[1] == 0 and arena[1] == arena[2] and shared[2] == arena[2]
    assert shared[1] < shared[2], "intermediates of a %d-layer chain must share bytes" % len(widths)
    # an intermediate that shares bytes cannot be read or written by name; with its own slice it can
    with pytest.raises(Exception, match="reuse_intermediates"):
        shared[3].get_tensor(shared[4][2].id).numpy()
    with pytest.raises(Exception, match="reuse_intermediates"):
        shared[3].get_tensor(shared[4][2].id).from_numpy(np.zeros((96, 320), np.float32))
    assert arena[3].get_tensor(arena[4][2].id).numpy().shape == (96, 320)
    # fed inputs, const weights and the fetched output keep slices of their own
    assert np.array_equal(shared[3].get_tensor("x").numpy(), x)
    assert shared[3].get_tensor("w3").numpy().shape == (320, 64)


def test_graph_replay_on_shared_intermediates(gpu):
    """the captured graph holds the arena's addresses; replays with new inputs match eager runs"""
    from cinn_amd import runtime
    rng = np.random.default_rng(8)
    widths = [64, 64, 128, 64]
    x = rng.standard_normal((64, 48)).astype(np.float32)
    b = NetBuilder("arena_graph")
    X, mids, y = residual_chain(b, list(x.shape), widths)
    feeds = {X: x}
    cin = x.shape[1]
    for i, w in enumerate(widths):
        feeds["w%d" % i] = (rng.standard_normal((cin, w)) / np.sqrt(cin)).astype(np.float32)
        cin = w
    stream = runtime.Stream()
    (eager,), comp = run(b, feeds, [y], stream=stream)
    stream.synchronize()
    eager = comp.get_tensor(y.id).numpy()
    for replay in range(3):
        x2 = rng.standard_normal(x.shape).astype(np.float32)
        comp.get_tensor("x").from_numpy(x2)
        comp.execute()
        stream.synchronize()
        want = comp.get_tensor(y.id).numpy()
        comp.get_tensor(y.id).from_numpy(np.zeros_like(want))
        comp.execute_graph()
        stream.synchronize()
        assert np.array_equal(comp.get_tensor(y.id).numpy(), want), "replay %d" % replay
    assert not np.array_equal(want, eager)
