"""GraphedStep: a layer's forward + backward recorded once in a HIP graph.  Every replay, with
eager work, parameter updates and synchronisation between the replays, must reproduce what the
eager calls give for the operands then in place (bit for bit: the kernels' summation order does
not depend on how they are launched)."""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def layers():
    import butterfly_amd
    from butterfly_amd import legacy
    from butterfly_amd.diagonal import Diagonal
    from butterfly_amd.permutation import FusedSequential
    yield "butterfly with bias", butterfly_amd.Butterfly(1024, 1024, bias=True, nblocks=2), (256, 1024), torch.float32
    yield "three stacks, padded", butterfly_amd.Butterfly(100, 300, bias=True, increasing_stride=False), (64, 100), torch.float32
    yield "folded diagonals", FusedSequential(Diagonal(1024), butterfly_amd.Butterfly(1024, 1024, bias=False, nblocks=2,
                                                                                    increasing_stride=False),
                                              Diagonal(1024)), (512, 1024), torch.float32
    yield "complex", butterfly_amd.Butterfly(256, 256, bias=False, complex=True), (128, 256), torch.complex64
    yield "legacy layer", legacy.Butterfly(512, 512, bias=False, tied_weight=False), (2048, 512), torch.float32


@pytest.mark.parametrize("case", range(5))
def test_replays_match_eager_steps(case):
    import butterfly_amd
    name, layer, shape, dtype = list(layers())[case]
    say("graphed step:", name, shape, dtype)
    torch.manual_seed(50 + case)
    layer = layer.cuda()
    params = [t for t in layer.parameters() if t.requires_grad]
    x = torch.randn(shape, dtype=dtype).cuda()
    g = torch.randn_like(layer(x).detach())
    step = butterfly_amd.GraphedStep(layer, x, g, params)
    for rep in range(3):
        x = torch.randn(shape, dtype=dtype).cuda()
        g = torch.randn_like(g)
        with torch.no_grad():
            for t in params:      # an optimiser step in place: the replay must see the new values
                t.mul_(1.0 + 0.01 * (rep + 1))
        y, grads = step(x, g)
        torch.cuda.synchronize()
        xe = x.clone().requires_grad_()
        ye = layer(xe)
        want = torch.autograd.grad(ye, [xe] + params, g)
        torch.cuda.synchronize()
        assert torch.equal(y, ye.detach()), (name, rep)
        assert len(grads) == len(want)
        for i, (a, b) in enumerate(zip(grads, want)):
            assert torch.equal(a, b), (name, rep, i)


def test_forward_only_and_argument_checks():
    import butterfly_amd
    torch.manual_seed(60)
    layer = butterfly_amd.Butterfly(1024, 1024, bias=False).cuda()
    x = torch.randn(2048, 1024).cuda()
    say("graphed forward only")
    step = butterfly_amd.GraphedStep(layer, x)
    for rep in range(2):
        x = torch.randn(2048, 1024).cuda()
        y, grads = step(x)
        torch.cuda.synchronize()
        assert grads == () and torch.equal(y, layer(x).detach())
    # written in place, replayed without the copies
    step.input.detach().copy_(x * 2)
    y, _ = step.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, layer(x * 2).detach())
    with pytest.raises(ValueError, match="recorded for input"):
        step(x[:100])
    with pytest.raises(ValueError, match="without a backward"):
        step(x, x)
    with pytest.raises(ValueError, match="device tensor"):
        butterfly_amd.GraphedStep(layer, x.cpu())


def test_random_zoo_layers_replay_bit_identically():
    """Forty seeded random layers (every `special` constructor, the legacy layer, KOP2d; the
    generator of test_gpu_zoo_random.py) recorded as one graph each: three replays with fresh
    inputs and output gradients, each bit-identical to the eager forward + autograd backward."""
    import butterfly_amd as bfa
    from test_gpu_zoo_random import draw_layer
    for seed in range(8100, 8140):
        rng = np.random.default_rng(seed)
        torch.manual_seed(seed)
        kind, layer, x = draw_layer(rng)
        print("graphed zoo case", seed, kind, tuple(x.shape), flush=True)
        layer, x = layer.cuda(), x.cuda()
        params = [p for p in layer.parameters() if p.requires_grad]
        with torch.no_grad():
            g = torch.randn_like(layer(x))
        step = bfa.GraphedStep(layer, x, g, params)
        for _ in range(3):
            x2, g2 = torch.randn_like(x), torch.randn_like(g)
            y, grads = step(x2, g2)
            y, grads = y.clone(), [t.clone() for t in grads]
            torch.cuda.synchronize()
            xe = x2.clone().requires_grad_()
            ye = layer(xe)
            want = torch.autograd.grad(ye, [xe] + params, g2)
            assert torch.equal(y, ye.detach())
            for a, b in zip(grads, want):
                assert torch.equal(a, b)
