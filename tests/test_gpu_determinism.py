"""Run-to-run determinism of the resident layer: the same layer on the same inputs gives bit-identical outputs on repeated eager
launches and on replays of a HIP graph that recorded the same launches (the kernels use no atomics on outputs and no
order-dependent reductions, so any difference would be a race)."""
import numpy as np
import pytest

from dwarfstar_red_lite_amd import synth

pytestmark = pytest.mark.gpu
torch = pytest.importorskip("torch")


@pytest.mark.parametrize("layout", ["iq2", "f2"])
def test_eager_and_graph_replays_bit_identical(layout):
    from dwarfstar_red_lite_amd.moe import ResidentMoe
    cfg = synth.layer_config(layout=layout)
    NL, max_tok = 2, 64
    m = ResidentMoe(cfg, n_layer=NL, max_tokens=max_tok)
    for l in range(NL):
        m.load_layer(l, synth.make_layer(600 + l, cfg))
    rng = np.random.default_rng(12)
    stream = torch.cuda.Stream()
    for ntok in (1, 2, 8, max_tok):
        xs = torch.from_numpy(synth.normed_x(rng, 3 * ntok, cfg["hidden"]).reshape(3, ntok, -1)).cuda()
        outs = torch.zeros_like(xs)

        def steps():
            for i in range(6):                               # both layers, three activation sets, back to back
                m.forward(i % NL, xs[i % 3], outs[i % 3]) if i < 3 else m.forward((i + 1) % NL, xs[i % 3], outs[i % 3])

        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            steps()
            stream.synchronize()
            first = outs.clone()
            outs.zero_()
            steps()
            stream.synchronize()
            assert torch.equal(outs, first), (layout, ntok, "second eager run")
            assert bool(torch.isfinite(first).all())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                steps()
        for replay in range(3):
            outs.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(outs, first), (layout, ntok, "graph replay", replay)
            # eager work of the program's own between the replays
            with torch.cuda.stream(stream):
                m.forward(0, xs[1], outs[1])
                stream.synchronize()
        del graph
    m.close()
