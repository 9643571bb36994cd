"""HIP-graph capture of the launches a decode step issues: every replay must equal the eager result.

The library only enqueues kernels (no allocation, no memset, no synchronisation), so its
entry points can be captured; inputs are updated in place between replays, with the program's
own eager work and synchronisations in between.
"""
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import to_device

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def test_graph_replays_match_eager(ops_mod):
    G = 128
    shapes = [(1, 2048, 2048), (1, 2048, 512), (1, 5632, 256)]
    sets = []
    for i, (M, K, N) in enumerate(shapes):
        ops = o.make_operands(9900 + i, M, K, N, G)
        d = to_device(ops, DEV)
        sets.append((d, ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)))
    xs = [d["x"].clone() for d, _ in sets]
    direct = ops_mod.DirectGemv([(xs[0], sets[0][1], False), (xs[1], sets[1][1], False)])
    single = ops_mod.DirectGemv([(xs[2], sets[2][1], False)])
    plan = ops_mod.GroupedGemv([(x, pw, False) for x, (_, pw) in zip(xs, sets)])
    y_canon = torch.empty((1, shapes[0][2]), dtype=torch.bfloat16, device=DEV)

    def step():
        direct.launch()
        single.launch()
        plan.launch()
        d0 = sets[0][0]
        ops_mod.int4_gemv_into(y_canon, xs[0], d0["qweight"], d0["scales"], d0["qzeros"], G)

    def snapshot():
        torch.cuda.synchronize()
        return [t.clone() for t in (*direct.outputs, *single.outputs, *plan.outputs, y_canon)]

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    gen = torch.Generator(device=DEV).manual_seed(5)
    for rep in range(4):
        for x in xs:  # new activations in place, as a decode loop would write them
            x.copy_(torch.randn(x.shape, generator=gen, device=DEV).to(torch.bfloat16))
        step()
        want = snapshot()
        for t in (*direct.outputs, *single.outputs, *plan.outputs, y_canon):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        assert all(torch.equal(a, b) for a, b in zip(want, got)), f"replay {rep} differs from eager"
        assert any(bool(t.abs().sum() > 0) for t in got)
