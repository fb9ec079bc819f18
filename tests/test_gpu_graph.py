"""The entry points are safe to record into a HIP graph: they launch on the given stream only, never
synchronise, and allocate nothing themselves.  A training step (forward + backward on the chunk cache) and
a decode step are captured once and replayed several times with the inputs changed in place and eager work
in between; every replay must equal the eager result on the same inputs bit for bit."""
import pytest
import torch

from helpers import gen

pytestmark = pytest.mark.gpu


def _step_inputs(seed, dtype=torch.bfloat16):
    N, C, Hq, Hkv, S, d, K = 2, 9, 4, 2, 64, 64, 3
    q = gen((N * (C - 1), Hq, S, d), seed, 0.5, dtype).cuda()
    ck = gen((N, C, S, Hkv * d), seed + 1, 0.5, dtype).cuda()
    cv = gen((N, C, S, Hkv * d), seed + 2, 0.5, dtype).cuda()
    g = torch.Generator().manual_seed(seed + 3)
    idx = torch.stack([torch.stack([torch.randperm(C, generator=g)[:K] for _ in range(C - 1)]) for _ in range(N)])
    w = torch.softmax(torch.rand(N * (C - 1), K, generator=g), -1).cuda()
    do = gen(tuple(q.shape), seed + 4, 1.0, dtype).cuda()
    return q, ck, cv, idx.reshape(N * (C - 1), K).cuda(), w, do


def test_training_step_replays_in_a_graph():
    import gca_hip

    def step(q, ck, cv, idx, w, do):
        q, ck, cv, w = [t.detach().requires_grad_() for t in (q, ck, cv, w)]
        o = gca_hip.attention_indexed(q, ck, cv, idx, w, 0.125, 1.0)
        return (o,) + torch.autograd.grad(o, (q, ck, cv, w), do)

    static = list(_step_inputs(200))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(*static)                                     # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(*static)
    for seed in (210, 220, 230):
        fresh = _step_inputs(seed)
        for s, f in zip(static, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        ref = step(*fresh)                                    # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, ref):
            assert torch.equal(a, b)


def test_decode_step_replays_in_a_graph():
    import gca_hip
    N, C, Hq, Hkv, S, d, K = 4, 12, 4, 2, 64, 64, 3
    dt = torch.bfloat16
    m = gca_hip.ChunkKVManager(capacity=32)
    with torch.no_grad():
        m.append(gen((N, C, S, Hkv * d), 1, 0.5, dt).cuda(), gen((N, C, S, Hkv * d), 2, 0.5, dt).cuda(),
                 gen((N, C, 64), 3, 1.0, dt).cuda())
        m.batch_retrieval(gen((N, C, 64), 4, 1.0, dt).cuda(), K, 0, use_cache=True)
        q = gen((N, Hq, 1, d), 5, 0.5, dt).cuda()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            m.decode_attention(q, 0, 1.0)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = m.decode_attention(q, 0, 1.0)
        for seed in (6, 7, 8):
            fresh = gen((N, Hq, 1, d), seed, 0.5, dt).cuda()
            q.copy_(fresh)
            graph.replay()
            torch.cuda.synchronize()
            got = out.clone()
            ref = m.decode_attention(fresh, 0, 1.0)
            assert torch.equal(got, ref)
