"""GraphedForward: a stack of quantized layers recorded once as a HIP graph and replayed; every replay against the
eager result, with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

from tests import cases

pytestmark = pytest.mark.gpu


def _stack(dev, dims, seed, asym_last=False):
    from duqlinear4bitcuda_amd.nn import Linear4bitASQ, Linear4bitSQ, SymQuantizer
    layers = []
    torch.manual_seed(seed)
    for i, (k, n) in enumerate(zip(dims[:-1], dims[1:])):
        lin = torch.nn.Linear(k, n, bias=(i % 2 == 0)).half().to(dev)
        with torch.no_grad():
            lin.weight.mul_(8.0)   # keep the activations of the later layers away from zero
        if asym_last and i == len(dims) - 2:
            layers.append(Linear4bitASQ.from_linear(lin).to(dev))
        else:
            sw = (lin.weight.abs().amax(dim=1, keepdim=True) / 7).half()
            layers += [SymQuantizer(1.0), Linear4bitSQ.from_float(lin, sw).to(dev)]
    return torch.nn.Sequential(*layers)


@pytest.mark.parametrize("M", [1, 4, 16, 100])
def test_graphed_stack_equals_eager_on_every_replay(dev, M):
    from duqlinear4bitcuda_amd.tools.graphs import GraphedForward
    print("graphed stack", M, flush=True)
    model = _stack(dev, (512, 768, 512, 256), seed=M, asym_last=True)
    xs = [cases.t(cases.acts_normal(M, 512, seed=100 + i), dev) for i in range(4)]
    want = [model(x).clone() for x in xs]
    g = GraphedForward(model, xs[0])
    for rep in range(3):
        for x, w in zip(xs, want):
            y = g(x)
            assert y is g.output and torch.equal(y.view(torch.int16), w.view(torch.int16)), (rep, M)
            # eager work of the same layers and a synchronisation between two replays
            assert torch.equal(model(x).view(torch.int16), w.view(torch.int16))
            torch.cuda.synchronize()
    # the static tensors can be driven by hand
    g.input.copy_(xs[2])
    g.replay()
    assert torch.equal(g.output.view(torch.int16), want[2].view(torch.int16))
    with pytest.raises(RuntimeError, match="recorded for"):
        g(xs[0][:, :256])
    # weights changed in place are seen by the recording
    with torch.no_grad():
        model[1].weight.copy_(torch.randint(0, 256, model[1].weight.shape, dtype=torch.uint8, device=dev))
    assert torch.equal(g(xs[1]).view(torch.int16), model(xs[1]).view(torch.int16))
