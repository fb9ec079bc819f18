"""GPU parity of the chunk cache (append kernel, strided landmark scoring) and of chunk-by-chunk
generation on it, against the CPU oracle, through the C ABI.

Copies and selections are compared bit for bit.  Landmarks in the flow tests hold small integers and
hidden sizes are powers of four, so every score is an exactly representable number whatever the
summation order: the selected chunk ids must then equal the oracle's exactly (ties included), and the
attention outputs agree within the kernels' tolerance (1e-5 relative fp32, 2e-2 bf16)."""
import pytest
import torch

from helpers import gen, rel_err
from oracle import cache_oracle as co
from oracle import gca_oracle as orc

pytestmark = pytest.mark.gpu


def _ints(shape, seed, lo=-3, hi=4, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g).to(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["keep", "zero", "drop"])
@pytest.mark.parametrize("N,S,Dm,Dl", [(2, 64, 768, 768), (3, 8, 20, 7), (1, 64, 1024, 256), (2, 5, 3, 1)])
def test_append_kernel_bit_exact(N, S, Dm, Dl, mode, dtype):
    """Appends of 3, 1, 1 and 4 chunks into stores with spare capacity == torch.cat of the oracle;
    slots beyond the count stay untouched.  Widths cover the 16-byte vector path and the element path."""
    import gca_hip
    cap = 12
    ks = torch.full((N, cap, S, Dm), 7, dtype=dtype, device="cuda")
    vs = torch.full((N, cap, S, Dm), 7, dtype=dtype, device="cuda")
    ls = torch.full((N, cap, Dl), 7, dtype=dtype, device="cuda")
    ref = co.ChunkCacheOracle()
    count = 0
    for i, n_new in enumerate((3, 1, 1, 4)):
        rows = S + 1 if mode == "drop" else S
        k = gen((N, n_new, rows, Dm), 10 * i + 1, 1.0, dtype)
        v = gen((N, n_new, rows, Dm), 10 * i + 2, 1.0, dtype)
        l = gen((N, n_new, Dl), 10 * i + 3, 1.0, dtype)
        ref.append(co.landmark_row(k, mode), co.landmark_row(v, mode), l)
        gca_hip.chunk_cache_append(k.cuda(), v.cuda(), l.cuda(), ks, vs, ls, count, mode)
        count += n_new
        assert torch.equal(ks[:, :count].cpu(), ref.chunk_k)
        assert torch.equal(vs[:, :count].cpu(), ref.chunk_v)
        assert torch.equal(ls[:, :count].cpu(), ref.lmk_embs)
        assert (ks[:, count:] == 7).all() and (vs[:, count:] == 7).all() and (ls[:, count:] == 7).all()


def test_append_rejects_overflow_and_bad_rows():
    import gca_hip
    ks = torch.zeros((1, 2, 8, 16), device="cuda")
    ls = torch.zeros((1, 2, 4), device="cuda")
    k = torch.zeros((1, 2, 8, 16), device="cuda")
    l = torch.zeros((1, 2, 4), device="cuda")
    with pytest.raises(RuntimeError):
        gca_hip.chunk_cache_append(k, k, l, ks, ks.clone(), ls, 1, "keep")        # 1 + 2 > capacity 2
    with pytest.raises(AssertionError):
        gca_hip.chunk_cache_append(k, k, l, ks, ks.clone(), ls, 0, "drop")        # drop needs S + 1 source rows


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,C,E,cap,Dm", [(3, 1, 37, 64, 256), (2, 5, 9, 16, 64), (4, 1, 700, 1024, 768), (2, 40, 130, 200, 128)])
def test_scoring_reads_strided_landmark_store(N, C, E, cap, Dm, dtype):
    """Scoring the first E landmarks of a store with spare capacity, in place, == scoring a dense copy."""
    import gca_hip
    store = gen((N, cap, Dm), 5, 1.0, dtype).cuda()
    lq = gen((N, C, Dm), 6, 1.0, dtype).cuda()
    view = store[:, :E]
    assert not view.is_contiguous() or N == 1
    got = gca_hip.landmark_scores(lq, view, Dm, causal=True)
    dense = gca_hip.landmark_scores(lq, view.contiguous(), Dm, causal=True)
    assert torch.equal(got, dense)
    ref = orc.mask_scores(orc.landmark_scores(lq.cpu().double(), view.cpu().double(), Dm))
    fin = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(got.cpu()), fin)
    assert rel_err(got.cpu()[fin], ref[fin]) < (1e-5 if dtype == torch.float32 else 2e-2)


def _flow_inputs(N, C, Hq, Hkv, S, d, Dl, dtype, seed):
    q_all = gen((N, C, Hq, S, d), seed, 0.5, dtype)
    ck = gen((N, C, S, Hkv * d), seed + 1, 0.5, dtype)
    cv = gen((N, C, S, Hkv * d), seed + 2, 0.5, dtype)
    lq, lk = _ints((N, C, Dl), seed + 3, dtype=dtype), _ints((N, C, Dl), seed + 4, dtype=dtype)
    return q_all, ck, cv, lq, lk


def _generate_hip(q_all, ck, cv, lq, lk, topk, prompt, sm_n, steps, offloading=False, capacity=0, mode="keep"):
    """The oracle's ``generate`` on gca_hip.ChunkKVManager: prompt -> batch retrieval with use_cache ->
    per chunk: decode steps, append, end-of-chunk retrieval."""
    import gca_hip
    N, C, Hq, S, d = q_all.shape
    m = gca_hip.ChunkKVManager(offloading=offloading, group_size=1, capacity=capacity)
    dev = lambda t: t.cuda()
    with torch.no_grad():
        m.append(dev(ck[:, :prompt]), dev(cv[:, :prompt]), dev(lk[:, :prompt]), landmark_row=mode)
        m.batch_retrieval(dev(lq[:, :prompt]), topk, 0, use_cache=True)
        out = torch.zeros_like(q_all)
        picked = []
        for c in range(prompt, C):
            picked.append(m.current_retrieved_indices(0)[0].cpu().clone())
            s, i = 0, 0
            while s < S:
                n = min(steps[i % len(steps)], S - s)
                out[:, c, :, s:s + n] = m.decode_attention(dev(q_all[:, c, :, s:s + n]), 0, sm_n).cpu()
                s += n
                i += 1
            m.append(dev(ck[:, c:c + 1]), dev(cv[:, c:c + 1]), dev(lk[:, c:c + 1]), landmark_row=mode)
            m.step_retrieval(dev(lq[:, c:c + 1]), topk, 0)
    return out, picked, m


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("steps,prompt,offloading,capacity", [
    ((1,), 1, False, 0), ((2,), 3, False, 0), ((1, 2, 61), 2, False, 64), ((64,), 4, False, 0), ((2,), 2, True, 0)])
def test_generation_matches_oracle_and_batch_form(steps, prompt, offloading, capacity, dtype):
    """Chunk-by-chunk generation on the HIP cache == the oracle's generation (ids bit-exact, outputs within
    tolerance) == the batch layer of the whole sequence (the reference's generation_unittest property)."""
    import gca_hip
    N, C, Hq, Hkv, S, d, Dl, topk = 2, 9, 4, 2, 64, 64, 64, 3
    q_all, ck, cv, lq, lk = _flow_inputs(N, C, Hq, Hkv, S, d, Dl, dtype, seed=70)
    f64 = lambda t: t.double()
    ref, picked_ref = co.generate(f64(q_all), f64(ck), f64(cv), f64(lq), f64(lk), topk, Hkv, prompt, 1.0, None, steps)
    out, picked, m = _generate_hip(q_all, ck, cv, lq, lk, topk, prompt, 1.0, steps, offloading, capacity)
    assert m.count == C and m.capacity >= C
    assert torch.equal(m.chunk_k.cpu(), ck) and torch.equal(m.chunk_v.cpu(), cv) and torch.equal(m.lmk_embs.cpu(), lk)
    for a, b in zip(picked, picked_ref):
        assert torch.equal(a, b)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert rel_err(out, ref) < tol
    full, _, _ = gca_hip.gca_layer(q_all.cuda(), ck.cuda(), cv.cuda(), lq.cuda(), lk.cuda(), topk, sm_n=1.0, training=False)
    assert rel_err(out[:, prompt:], full[:, prompt:].cpu()) < tol


def test_generation_with_landmark_row_zeroed():
    """``landmark_row="zero"`` at append == the oracle fed chunks whose last row was zeroed beforehand."""
    N, C, Hq, Hkv, S, d, Dl, topk = 1, 6, 2, 2, 64, 64, 16, 2
    q_all, ck, cv, lq, lk = _flow_inputs(N, C, Hq, Hkv, S, d, Dl, torch.float32, seed=90)
    f64 = lambda t: t.double()
    ref, picked_ref = co.generate(f64(q_all), f64(co.landmark_row(ck, "zero")), f64(co.landmark_row(cv, "zero")),
                                  f64(lq), f64(lk), topk, Hkv, 2, 0.0, None, (2,))
    out, picked, m = _generate_hip(q_all, ck, cv, lq, lk, topk, 2, 0.0, (2,), mode="zero")
    assert torch.equal(m.chunk_k.cpu(), co.landmark_row(ck, "zero"))
    for a, b in zip(picked, picked_ref):
        assert torch.equal(a, b)
    assert rel_err(out, ref) < 1e-5


def test_training_append_keeps_autograd():
    """A first append of tensors with gradients adopts them: the cache gradients of the indexed kernels
    reach the tensors that were appended (what the reference gets from storing the tensor itself)."""
    import gca_hip
    N, C, Hq, Hkv, S, d, Dl, topk = 2, 5, 4, 2, 64, 64, 32, 2
    q_all, ck, cv, lq, lk = _flow_inputs(N, C, Hq, Hkv, S, d, Dl, torch.float32, seed=110)
    ckg, cvg = ck.cuda().requires_grad_(), cv.cuda().requires_grad_()
    m = gca_hip.ChunkKVManager()
    m.append(ckg, cvg, lk.cuda())
    idx, w = m.batch_retrieval(lq.cuda(), topk)
    kk = idx.shape[-1]
    q = q_all[:, 1:].reshape(N * (C - 1), Hq, S, d).cuda()
    o = gca_hip.attention_indexed(q, m.k_store, m.v_store, idx[:, :-1].reshape(-1, kk).contiguous(),
                                  w[:, :-1].reshape(-1, kk).contiguous(), 0.125, 0.0)
    do = gen(tuple(o.shape), 111).cuda()
    o.backward(do)
    k, v, wg = orc.gather_chunks(ck.double(), cv.double(), idx.cpu(), w.cpu().double(), Hkv)
    k.requires_grad_(); v.requires_grad_()
    # oracle gradient of the gathered copies, scattered back by index_put(accumulate)
    oo = orc.gca_forward(q.cpu().double(), k, v, wg, 0.125, 0.0)
    oo.backward(do.cpu().double())
    dk_ref = torch.zeros_like(ck, dtype=torch.float64)
    flat = idx[:, :-1].reshape(N, (C - 1) * kk).cpu()
    gk = k.grad.reshape(N, C - 1, Hkv, kk, S, d).permute(0, 1, 3, 4, 2, 5).reshape(N, (C - 1) * kk, S, Hkv * d)
    dk_ref.index_put_((torch.arange(N).unsqueeze(1), flat), gk, accumulate=True)
    assert rel_err(ckg.grad, dk_ref) < 1e-5
