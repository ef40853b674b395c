"""GPU test: the decode call of a model's layers captured into a HIP graph through the entry point
that allocates nothing, replayed several times with eager work in between; every replay must equal
the eager result bit for bit (same kernels, same split plan)."""
import numpy as np
import pytest

import oracle as O
from gpu_util import check_attention_out, ctx, dev, host, normal

pytestmark = pytest.mark.gpu


def test_layer_loop_captured_in_a_graph_replays_like_eager():
    import torch
    layers, hq, hkv, d, L = 6, 32, 8, 128, 2048
    rng = np.random.default_rng(3)
    k = [dev(O.f32_to_f16_bits(rng.standard_normal((hkv, L, d)).astype(np.float32)).view(np.float16)) for _ in range(layers)]
    v = [dev(O.f32_to_f16_bits(rng.standard_normal((hkv, L, d)).astype(np.float32)).view(np.float16)) for _ in range(layers)]
    q = dev(normal((layers, hq, d), 5))
    out = torch.zeros((layers, hq, d), device="cuda")
    sc = torch.zeros((layers, hq, L), device="cuda")

    def token(noalloc):
        for i in range(layers):
            # odd layers emit scores (the H2O layers of a model), even ones do not
            ctx().attention_gen(q[i], k[i], v[i], out[i], hkv, L, L, scores=sc[i] if i % 2 else None,
                                score_stride=L if i % 2 else 0, noalloc=noalloc)

    token(False)
    torch.cuda.synchronize()
    eager, eager_sc = out.clone(), sc.clone()
    for i in (0, 3):
        ref = O.attention_gen(normal((layers, hq, d), 5)[i], host(k[i]), host(v[i]), hkv, L, L)
        check_attention_out(host(eager[i]), ref, "layer %d" % i)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        token(True)  # first launch of every kernel happens outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        token(True)
    for r in range(4):
        out.fill_(float(r))
        sc.fill_(-1.0)
        token(False) if r == 2 else None  # the program's own eager work between replays
        out.fill_(float(r))
        sc.fill_(-1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), "replay %d" % r
        assert torch.equal(sc[1::2], eager_sc[1::2]), "replay %d scores" % r
        assert (sc[0::2] == -1.0).all()
