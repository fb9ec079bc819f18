"""The window of the score mask (``max_chunk_win`` of ``_enc_dec_score_mask``, model/DRT.py:590-607) on the GPU path.

A row with id r = E - C + c sees chunk e iff r > e and r <= e + w.  Checked against the oracle's mask (which is pinned
by a brute-force loop in test_oracle.py): the -inf pattern of the scores bit for bit, the selection exactly on given
scores (masked chunks on both sides of the window tie at -inf and fill short rows lowest index first), and the three
forms -- two launches, selection while scoring, the chunk cache's retrieval -- against one another.
"""
import pytest
import torch

from helpers import gen
from oracle import gca_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _topk_ref(scores, k, win, noise=None):
    s = orc.mask_scores(scores.float(), win)
    sel = s if noise is None else orc.mask_scores((scores + noise).float(), win)
    kk = min(s.shape[-1], k)
    _, idx = orc.topk_canonical(sel, kk)
    return idx, orc.retrieval_weights(s, idx)


# (N, C, E, Dm): square; E > C (the rows are the last C ids); shapes of the 64 x 128 and (the last one) 128 x 128 block
# kernels, of the 32 x 32 tile kernel (width 100, and every fp32 case with C > 32) and of the decode scans (C <= 32)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("win", [1, 3, 64, 200, 100000])
@pytest.mark.parametrize("N,C,E,Dm", [(2, 16, 16, 256), (1, 300, 300, 64), (1, 70, 500, 100), (1, 8, 3000, 64),
                                      (2, 1100, 1100, 64), (1, 4224, 4224, 64)])
def test_window_mask_of_the_scores(N, C, E, Dm, win, dtype):
    import gca_hip
    lq, lk = gen((N, C, Dm), 1, 1.0, dtype).to(DEV), gen((N, E, Dm), 2, 1.0, dtype).to(DEV)
    plain = gca_hip.landmark_scores(lq, lk, None, True)
    got = gca_hip.landmark_scores(lq, lk, None, True, max_chunk_win=win)
    vis = orc.causal_visible(C, E, win, device=DEV)
    assert vis.any() and (win >= E or not torch.equal(vis, orc.causal_visible(C, E, -1, device=DEV)))
    assert torch.equal(torch.isneginf(got), (~vis).expand(N, C, E))
    bits = torch.int32 if dtype == torch.float32 else torch.int16
    assert torch.equal(got[:, vis].view(bits), plain[:, vis].view(bits))     # visible scores are untouched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,C,E,k,win", [(2, 64, 64, 8, 3), (1, 300, 300, 8, 8), (1, 300, 300, 8, 20), (1, 40, 5000, 16, 7),
                                         (1, 12, 9001, 8, 4000), (1, 50, 50, 33, 5), (1, 64, 64, 4, 1)])
def test_window_topk_exact_on_given_scores(N, C, E, k, win, dtype):
    import gca_hip
    scores = gen((N, C, E), 300 + C + win, 1.0, dtype)
    idx_ref, w_ref = _topk_ref(scores, k, win)
    idx, w = gca_hip.landmark_topk(scores.to(DEV), k, True, None, max_chunk_win=win)
    assert torch.equal(idx.cpu(), idx_ref)
    assert (w.cpu() - w_ref).abs().max() <= 1e-6
    masked_slots = orc.mask_scores(scores.float(), win).gather(2, idx_ref) == float("-inf")
    assert (w.cpu()[masked_slots] == 0).all()
    if win < k:                                               # a window shorter than k: every row has -inf slots
        assert masked_slots.any(-1).all()
    # rows far enough in see exactly `win` chunks, the most recent ones
    r = E - 1                                                 # id of the last row
    if win < min(k, r):
        assert sorted(idx[0, -1, :win].tolist()) == list(range(r - win, r))


def test_window_topk_with_noise():
    import gca_hip
    N, C, k, win = 2, 200, 8, 30
    scores = gen((N, C, C), 41, 1.0, torch.bfloat16)
    u = torch.rand(N, C, C, generator=torch.Generator().manual_seed(42)).clamp_min(1e-6)
    noise = (-(-u.log()).log()).bfloat16()
    idx_ref, w_ref = _topk_ref(scores, k, win, noise)
    idx, w = gca_hip.landmark_topk(scores.to(DEV), k, True, noise.to(DEV), max_chunk_win=win)
    assert torch.equal(idx.cpu(), idx_ref)
    assert (w.cpu() - w_ref).abs().max() <= 1e-6


@pytest.mark.parametrize("noisy", [False, True])
@pytest.mark.parametrize("N,C,E,Dm,k,win", [(2, 256, 256, 128, 8, 5), (1, 96, 3000, 64, 8, 700), (2, 1024, 1024, 64, 5, 130),
                                            (1, 64, 70000, 64, 8, 66000), (1, 2048, 2048, 192, 32, 12)])
def test_window_selecting_while_scoring(N, C, E, Dm, k, win, noisy):
    """The fused kernel against the two launches on the kernel's own scores: same bits."""
    import gca_hip
    g = torch.Generator(device=DEV).manual_seed(70 + C)
    lq = torch.randn(N, C, Dm, device=DEV, generator=g).bfloat16()
    lk = torch.randn(N, E, Dm, device=DEV, generator=g).bfloat16()
    noise = None
    if noisy:
        noise = (-torch.empty(N, C, E, device=DEV).exponential_(generator=g).log()).bfloat16()
    scores = gca_hip.landmark_scores(lq, lk, None, True, max_chunk_win=win)
    ref_idx, ref_w = gca_hip.landmark_topk(scores, k, True, noise, max_chunk_win=win)
    none, idx, w = gca_hip.landmark_score_topk(lq, lk, k, None, True, noise, return_scores=False, fused=True,
                                               max_chunk_win=win)
    assert none is None
    assert torch.equal(idx, ref_idx) and torch.equal(w, ref_w)
    # and the two-launch form on these scores is the canonical rule
    o_idx, o_w = _topk_ref(scores.cpu(), k, win, None if noise is None else noise.cpu())
    assert torch.equal(ref_idx.cpu(), o_idx)
    assert (ref_w.cpu() - o_w).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_window_retrieval_against_the_oracle_with_gradients(dtype, tol):
    """landmark_retrieve with a window: scores within tolerance, selection equal wherever the oracle's gaps exceed it,
    and the weights' gradient reaches both landmark sets as autograd gives it through the oracle."""
    import gca_hip
    N, C, Dm, k, win = 2, 48, 128, 4, 9
    lq = gen((N, C, Dm), 5, 1.0, dtype)
    lk = gen((N, C, Dm), 6, 1.0, dtype)
    lq_o, lk_o = lq.float().clone().requires_grad_(), lk.float().clone().requires_grad_()
    s_o, idx_o, w_o = orc.retrieve(lq_o, lk_o, k, None, None, win)
    lq_g, lk_g = lq.to(DEV).requires_grad_(), lk.to(DEV).requires_grad_()
    s, idx, w = gca_hip.landmark_retrieve(lq_g, lk_g, k, None, True, None, True, max_chunk_win=win)
    assert torch.equal(torch.isneginf(s.cpu()), torch.isneginf(s_o))
    fin = torch.isfinite(s_o)
    assert (s.cpu().float()[fin] - s_o.detach()[fin]).abs().max() <= tol * s_o.detach()[fin].abs().max()
    # the selection on the kernel's own scores is the canonical one
    idx_own, w_own = _topk_ref(s.detach().cpu(), k, win)
    assert torch.equal(idx.cpu(), idx_own)
    assert (w.detach().cpu() - w_own).abs().max() <= 1e-6
    if dtype == torch.float32:
        assert torch.equal(idx.cpu(), idx_o)
        dw = gen((N, C, k), 8, 1.0, torch.float32)
        w_o.backward(dw)
        w.backward(dw.to(DEV))
        for got, ref in ((lq_g.grad, lq_o.grad), (lk_g.grad, lk_o.grad)):
            assert (got.cpu() - ref).abs().max() <= 1e-5 * max(1.0, ref.abs().max().item())


def test_window_zero_and_the_cache_call():
    import gca_hip
    from gca_hip.chunk_cache import ChunkKVManager
    N, C, S, Dm, k = 2, 40, 64, 64, 4
    lq = gen((N, C, Dm), 11, 1.0, torch.bfloat16).to(DEV)
    lk = gen((N, C, Dm), 12, 1.0, torch.bfloat16).to(DEV)
    # max_chunk_win = 0: dec > enc and dec <= enc cannot both hold, nothing is visible (model/DRT.py:599-603)
    s, idx, w = gca_hip.landmark_retrieve(lq, lk, k, None, True, None, True, max_chunk_win=0)
    s_o, idx_o, w_o = orc.retrieve(lq.cpu().float(), lk.cpu().float(), k, None, None, 0)
    assert torch.isneginf(s).all() and torch.isneginf(s_o).all()
    assert torch.equal(idx.cpu(), idx_o) and torch.equal(w.cpu(), w_o) and (w == 0).all()
    # the cache's batch retrieval passes the window through
    cache = ChunkKVManager()
    kv = gen((N, C, S, Dm), 13, 0.5, torch.bfloat16).to(DEV)
    cache.append(kv, kv, lk)
    idx_c, w_c = cache.batch_retrieval(lq, k, max_chunk_win=6)
    _, idx_r, w_r = gca_hip.landmark_retrieve(lq, lk, k, None, True, None, True, max_chunk_win=6)
    assert torch.equal(idx_c, idx_r) and torch.equal(w_c, w_r)
    _, idx_plain, _ = gca_hip.landmark_retrieve(lq, lk, k)
    assert not torch.equal(idx_plain, idx_r)


def test_negative_window_is_refused():
    import ctypes
    from gca_hip import _lib
    from gca_hip.retrieval import _lmk_desc
    from gca_hip.gca import _ptr, _stream
    lq = torch.randn(1, 64, 64, device=DEV)
    sc = torch.empty(1, 64, 64, device=DEV)
    desc = _lmk_desc(torch.float32, 8, 1, 64, 64, 64, True, 64.0)
    desc.chunk_win = -1
    rc = _lib.lib().lmk_score(ctypes.byref(desc), _ptr(lq), _ptr(lq), _ptr(sc), _stream(lq.device))
    assert rc == _lib.GCA_ERR_SHAPE
