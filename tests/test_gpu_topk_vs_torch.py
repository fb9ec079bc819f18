"""The selection kernel against ``torch.topk`` ON THE DEVICE (the call the reference makes, model/DRT.py:625).

``torch.topk`` leaves the order among equal values unspecified, so two statements are tested:
  * rows whose values are pairwise distinct (fp32 and bf16): the kernel's indices equal ``torch.topk(...).indices``
    slot for slot -- there is nothing to break ties on;
  * rows with exact ties (ordinary bf16 scores): the selected VALUES are the same multiset in the same order, and
    every index the two disagree on sits at a tied value.  How the library orders ties is recorded (printed and
    written to $GCA_TEST_RECORD_DIR/topk_ties.txt when that variable names a folder), not asserted: the kernels use the canonical rule
    "higher value first, then lower index".
"""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _masked(scores):
    C, E = scores.shape[-2:]
    vis = torch.arange(E, device=scores.device)[None, :] < (torch.arange(C, device=scores.device)[:, None] + (E - C))
    return scores.masked_fill(~vis, float("-inf"))


@pytest.mark.parametrize("N,C,k", [(2, 64, 8), (1, 700, 8), (1, 3000, 16), (1, 5000, 32)])
def test_distinct_fp32_rows_equal_torch_topk(N, C, k):
    import gca_hip
    g = torch.Generator(device=DEV).manual_seed(70 + C)
    # every row is a random permutation of C distinct values
    scores = (torch.rand(N, C, C, device=DEV, generator=g).argsort(-1).float() - C / 2) * 1e-3
    srt = scores.sort(-1).values
    assert (srt[..., 1:] != srt[..., :-1]).all()
    idx, w = gca_hip.landmark_topk(scores, k, causal=True)
    ref = torch.topk(_masked(scores), k, dim=-1)
    finite = torch.isfinite(ref.values)
    assert torch.equal(idx[finite], ref.indices[finite])
    assert (w[~finite] == 0).all()
    rw = torch.nan_to_num(torch.softmax(ref.values, -1))                      # model/DRT.py:626-627
    assert (w - rw).abs().max() <= 1e-6


@pytest.mark.parametrize("E,k", [(200, 8), (4000, 8), (30000, 16)])
def test_distinct_bf16_rows_equal_torch_topk(E, k):
    import gca_hip
    g = torch.Generator(device=DEV).manual_seed(80 + k)
    R = 16
    # distinct finite bf16 values per row: a random subset of the positive finite bit patterns, random signs kept apart
    bits = torch.stack([torch.randperm(0x7f00, device=DEV, generator=g)[:E] for _ in range(R)]) + 0x80
    scores = bits.to(torch.int16).view(torch.bfloat16).view(1, R, E)
    idx, _ = gca_hip.landmark_topk(scores, k, causal=False)
    ref = torch.topk(scores, k, dim=-1)
    assert torch.equal(idx, ref.indices)


def test_tied_bf16_rows_values_agree_and_tie_order_is_recorded():
    import gca_hip
    g = torch.Generator(device=DEV).manual_seed(90)
    N, C, k = 2, 3000, 8
    scores = torch.randn(N, C, C, device=DEV, generator=g).bfloat16()         # thousands of exact ties per row
    idx, _ = gca_hip.landmark_topk(scores, k, causal=True)
    m = _masked(scores)
    ref = torch.topk(m, k, dim=-1)
    mine = m.gather(-1, idx)
    finite = torch.isfinite(ref.values)
    assert torch.equal(mine[finite], ref.values[finite])                       # same values, same slot order
    differ = (idx != ref.indices) & finite
    # a disagreement is only possible where the value is tied with another selected or boundary value
    rows = differ.any(-1)
    if rows.any():
        mult = (m[rows].unsqueeze(-1) == ref.values[rows].unsqueeze(-2)).sum(-2)     # per slot: candidates holding its value
        assert (mult[differ[rows]] >= 2).all()
    # canonical rule: among equal values the kernel's indices ascend
    same = (mine[..., 1:] == mine[..., :-1]) & finite[..., 1:]
    assert (idx[..., 1:][same] > idx[..., :-1][same]).all()
    tie_slots = int(same.sum())
    lib_ascending = int((ref.indices[..., 1:][same] > ref.indices[..., :-1][same]).sum())
    line = (f"torch {torch.__version__} topk on device, bf16 rows with ties (N={N}, C={C}, k={k}): "
            f"{int(rows.sum())} of {int(finite.any(-1).sum())} rows differ from the canonical order in "
            f"{int(differ.sum())} slots; of {tie_slots} adjacent tied slot pairs the library returns "
            f"{lib_ascending} in ascending index order")
    print(line)
    out_dir = os.environ.get("GCA_TEST_RECORD_DIR")
    if out_dir and os.path.isdir(out_dir):
        with open(os.path.join(out_dir, "topk_ties.txt"), "w") as f:
            f.write(line + "\n")
