"""Selection while scoring (``lmk_score_topk`` with ``scores == NULL``) against the two-launch form.

The fused kernel scores with the same block routine as ``lmk_score`` and orders candidates by the same rule as
``lmk_topk`` (higher value first, then lower index), so indices AND weights must be the same bits as
``landmark_scores`` + ``landmark_topk`` give on the kernel's own scores -- for one and for several column segments,
ragged last blocks, rows that see fewer than k chunks, noise, heavy ties, k that is not a power of two.  The
two-launch form itself is checked against the oracle in test_gpu_retrieval.py.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _landmarks(N, C, E, Dm, seed, ties=False):
    g = torch.Generator(device=DEV).manual_seed(seed)
    lq = torch.randn(N, C, Dm, device=DEV, generator=g)
    lk = torch.randn(N, E, Dm, device=DEV, generator=g)
    if ties:   # few distinct values per coordinate: thousands of exactly equal scores per row
        lq, lk = (lq * 1.5).round() / 2, (lk * 1.5).round() / 2
    return lq.bfloat16(), lk.bfloat16()


def _both(lq, lk, k, causal=True, noise=None, hidden=None):
    import gca_hip
    scores = gca_hip.landmark_scores(lq, lk, hidden, causal)
    ref_idx, ref_w = gca_hip.landmark_topk(scores, k, causal, noise)
    none, idx, w = gca_hip.landmark_score_topk(lq, lk, k, hidden, causal, noise, return_scores=False, fused=True)
    assert none is None
    return scores, ref_idx, ref_w, idx, w


# (N, C, E, Dm, k): one segment; several segments with a ragged last block; a partial last row block; E > C (rows that
# see a long past); the 16-bit offset limit of a segment (E > 65536); k = 1, 5 (padded to 8), 16, 32
SHAPES = [
    (2, 256, 256, 128, 8),
    (8, 256, 256, 768, 8),
    (1, 96, 3000, 64, 8),
    (2, 1024, 1024, 64, 5),
    (1, 40, 5000, 128, 16),
    (1, 64, 70000, 64, 8),
    (1, 2048, 2048, 192, 32),
    (3, 100, 1500, 64, 1),
]


@pytest.mark.parametrize("N,C,E,Dm,k", SHAPES)
def test_fused_equals_two_launch_form(N, C, E, Dm, k):
    lq, lk = _landmarks(N, C, E, Dm, 500 + C + k)
    _, ref_idx, ref_w, idx, w = _both(lq, lk, k)
    assert torch.equal(idx, ref_idx)
    assert torch.equal(w, ref_w)


@pytest.mark.parametrize("N,C,E,Dm,k", [(1, 300, 2500, 64, 8), (2, 256, 256, 64, 8), (1, 64, 66000, 64, 4)])
def test_fused_with_ties(N, C, E, Dm, k):
    lq, lk = _landmarks(N, C, E, Dm, 600 + C, ties=True)
    scores, ref_idx, ref_w, idx, w = _both(lq, lk, k)
    row = scores[0, -1].float()
    assert row[torch.isfinite(row)].unique().numel() < 0.5 * E          # the data really is tie-heavy
    assert torch.equal(idx, ref_idx)
    assert torch.equal(w, ref_w)


@pytest.mark.parametrize("N,C,E,Dm,k", [(2, 256, 256, 128, 8), (1, 128, 3000, 64, 16)])
def test_fused_with_noise(N, C, E, Dm, k):
    lq, lk = _landmarks(N, C, E, Dm, 700 + C)
    g = torch.Generator(device=DEV).manual_seed(701)
    noise = -torch.empty(N, C, E, device=DEV).exponential_(generator=g).log()       # model/DRT.py:616-620
    noise = noise.bfloat16()
    _, ref_idx, ref_w, idx, w = _both(lq, lk, k, noise=noise)
    assert torch.equal(idx, ref_idx)
    assert torch.equal(w, ref_w)
    # the noise really changes the selection, and the weights still come from the noise-free scores
    _, plain_idx, _, _, _ = _both(lq, lk, k)
    assert not torch.equal(plain_idx, ref_idx)


def test_fused_not_causal():
    lq, lk = _landmarks(2, 64, 1500, 64, 800)
    _, ref_idx, ref_w, idx, w = _both(lq, lk, 8, causal=False)
    assert torch.equal(idx, ref_idx)
    assert torch.equal(w, ref_w)


def test_size_rule_and_scores_on_request():
    """``fused=None``: score matrices below 2 GiB take the two launches even without scores; with scores the call
    returns the bits of ``landmark_scores``.  Either way the selection is the fused kernel's."""
    import gca_hip
    lq, lk = _landmarks(1, 200, 2300, 128, 900)
    _, ref_idx, ref_w, idx_f, w_f = _both(lq, lk, 8, hidden=96.0)
    scores = gca_hip.landmark_scores(lq, lk, 96.0, True)
    got, idx, w = gca_hip.landmark_score_topk(lq, lk, 8, 96.0, True, None, return_scores=True)
    assert torch.equal(got.view(torch.int16), scores.view(torch.int16))
    assert torch.equal(idx, ref_idx) and torch.equal(w, ref_w)
    none, idx2, w2 = gca_hip.landmark_score_topk(lq, lk, 8, 96.0, True, None, return_scores=False)
    assert none is None and torch.equal(idx2, idx_f) and torch.equal(w2, w_f)


def test_strided_landmark_store_and_fallback_shapes():
    import gca_hip
    # a landmark store with spare capacity is read in place
    store = torch.zeros(2, 4096, 64, device=DEV, dtype=torch.bfloat16)
    lq, lk = _landmarks(2, 64, 3000, 64, 950)
    store[:, :3000] = lk
    _, ref_idx, ref_w, _, _ = _both(lq, lk, 8)
    _, idx, w = gca_hip.landmark_score_topk(lq, store[:, :3000], 8, None, True, None, return_scores=False, fused=True)
    assert torch.equal(idx, ref_idx) and torch.equal(w, ref_w)
    # shapes the fused kernel does not take (fp32; a width that is no multiple of 64) still answer without scores
    for lq2, lk2 in ((lq.float(), lk.float()), (lq[..., :40].contiguous(), lk[..., :40].contiguous())):
        s2 = gca_hip.landmark_scores(lq2, lk2, None, True)
        r_idx, r_w = gca_hip.landmark_topk(s2, 8, True)
        none, idx2, w2 = gca_hip.landmark_score_topk(lq2, lk2, 8, None, True, None, return_scores=False, fused=True)
        assert none is None and torch.equal(idx2, r_idx) and torch.equal(w2, r_w)


def test_null_scores_refused_where_only_the_two_launch_form_exists():
    import ctypes
    from gca_hip import _lib
    from gca_hip.retrieval import _lmk_desc
    from gca_hip.gca import _ptr, _stream
    lq = torch.randn(1, 64, 64, device=DEV)
    lk = torch.randn(1, 64, 64, device=DEV)
    idx = torch.empty(1, 64, 8, device=DEV, dtype=torch.int64)
    w = torch.empty(1, 64, 8, device=DEV)
    desc = _lmk_desc(torch.float32, 8, 1, 64, 64, 64, True, 64.0)
    rc = _lib.lib().lmk_score_topk(ctypes.byref(desc), _ptr(lq), _ptr(lk), None, None, _ptr(idx), _ptr(w), None, 0,
                                   _stream(lq.device))
    assert rc == _lib.GCA_ERR_UNSUPPORTED
