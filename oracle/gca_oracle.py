"""CPU oracle for the Grouped Cross-Attention (GCA) hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
check and the benchmark's ``cpu_baseline`` leg may import it; the product path
(``gca_hip``) never does and fails loudly when its HIP library is missing.

It restates, in plain fp32/fp64 PyTorch on the CPU, the arithmetic the reference
performs on this path.  Each function cites the reference lines it follows
(paths relative to the reference checkout):

* landmark scoring ............ model/DRT.py:612   (decode copy :838)
* strict-past causal mask ..... model/DRT.py:590-607, applied :613
* top-k + retrieval weights ... model/DRT.py:616-627
* gather + row shift + layout . model/DRT.py:193-200, :629-637, :320-332
* GCA forward ................. ltriton/gca.py:912-921 (the reference's own
                                 einsum statement of its kernel, :94-211)
* GCA backward ................ autograd of the forward (ltriton/gca.py:922-926)
                                 and the explicit formulas of :318-481, :839-840
* caller contract ............. model/DRT.py:345-398

How each function is pinned (the reference holds no golden vectors for this
path: its only kernel test draws inputs from the GPU RNG, ltriton/gca.py:895-908):

* ``landmark_scores``   closed form (dot product / sqrt(hidden)); checked against
                        a triple loop in numpy float64.
* ``causal_visible``    closed form ``dec_id > enc_id``; checked against loops.
* ``topk_canonical``    equals ``torch.topk`` wherever values are strictly
                        separated; on ties the rule "higher value first, then
                        lower index" is checked against a brute-force python sort.
* ``retrieval_weights`` library softmax + nan_to_num; invariants (non-negative,
                        row sums in {0, 1}, masked slots weigh 0).
* ``gather_chunks``     pure indexing; checked against python loops.
* ``gca_forward``       textbook softmax attention per retrieved chunk + weighted
                        sum; checked against per-(z, h, j)
                        ``F.scaled_dot_product_attention``, numpy float64 loops,
                        K=1/w=1 reduction to plain attention, constant-V.
                        ``sm_n`` ("softmax off by one"): closed form
                        ``softmax([s, 0])[..., :-1]`` == appending a zero key and a
                        zero value row (what model/DRT.py:772-779 does).
* ``gca_backward``      explicit formulas checked against autograd of
                        ``gca_forward`` and fp64 ``gradcheck``; invariant
                        ``sum_j w_j D_j == rowsum(O * dO)``.

Parity unpinned by any reference test: ``sm_n != 0`` (the reference kernel
multiplies it by zero, ltriton/gca.py:186-187 with :48-49, and its tests pass 0)
and the retrieval functions (no reference test calls them).  Both are pinned here
by the closed forms above only.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

LOG2E = 1.4426950408889634


# --------------------------------------------------------------------------- retrieval

def landmark_scores(lmk_q: torch.Tensor, lmk_k: torch.Tensor, hidden_size: Optional[int] = None) -> torch.Tensor:
    """scores[n, c, e] = <lmk_q[n, c], lmk_k[n, e]> / sqrt(hidden)   (model/DRT.py:612).

    The divisor is the model width (``self.input_dim``), not the head dim.
    """
    if hidden_size is None:
        hidden_size = lmk_q.shape[-1]
    return torch.einsum('ncd,ned->nce', lmk_q, lmk_k) / math.sqrt(hidden_size)


def causal_visible(dec_chunk_num: int, enc_chunk_num: int, max_chunk_win: int = -1, device=None) -> torch.Tensor:
    """Boolean (dec, enc) matrix, True where a decoder row may see an encoder chunk.

    model/DRT.py:596-603: decoder ids are the LAST ``dec_chunk_num`` of
    ``arange(enc_chunk_num)``; visible iff ``dec_id > enc_id`` (strictly past),
    optionally also ``dec_id <= enc_id + max_chunk_win``.
    """
    dec = torch.arange(enc_chunk_num, device=device)[-dec_chunk_num:] if dec_chunk_num > 0 else torch.arange(0, device=device)
    enc = torch.arange(enc_chunk_num, device=device)
    vis = dec.unsqueeze(1) > enc.unsqueeze(0)
    if max_chunk_win != -1:
        vis = vis & (dec.unsqueeze(1) <= enc.unsqueeze(0) + max_chunk_win)
    return vis


def mask_scores(scores: torch.Tensor, max_chunk_win: int = -1) -> torch.Tensor:
    """Fill the non-visible entries with -inf   (model/DRT.py:613)."""
    vis = causal_visible(scores.shape[1], scores.shape[2], max_chunk_win, scores.device)
    return scores.masked_fill(~vis, float('-inf'))


def topk_canonical(values: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k along the last dim: higher value first, ties by LOWER index first.

    model/DRT.py:625 calls ``torch.topk`` (sorted), whose order among equal
    values is unspecified; this rule equals ``torch.topk`` whenever the values
    involved are strictly separated and fixes the choice otherwise.
    """
    vals, idx = torch.sort(values, dim=-1, descending=True, stable=True)
    return vals[..., :k].contiguous(), idx[..., :k].contiguous()


def retrieval_weights(masked_scores: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """softmax over the selected (noise-free) scores, NaN -> 0   (model/DRT.py:626-627)."""
    w = F.softmax(masked_scores.gather(dim=2, index=indices).float(), dim=-1)
    return torch.nan_to_num(w, nan=0.0)


def retrieve(lmk_q: torch.Tensor, lmk_k: torch.Tensor, chunk_topk: int, hidden_size: Optional[int] = None,
             noise: Optional[torch.Tensor] = None, max_chunk_win: int = -1):
    """Rows R1-R3: returns (masked scores, indices (N,C,k'), weights (N,C,k')).

    ``noise`` is the Gumbel perturbation used for the SELECTION only in training
    (model/DRT.py:616-625); weights always come from the noise-free scores.
    """
    scores = mask_scores(landmark_scores(lmk_q, lmk_k, hidden_size), max_chunk_win)
    k = min(scores.shape[-1], chunk_topk)                       # model/DRT.py:623
    sel = scores if noise is None else scores + noise
    _, indices = topk_canonical(sel, k)
    return scores, indices, retrieval_weights(scores, indices)


def gather_chunks(chunk_k: torch.Tensor, chunk_v: torch.Tensor, indices: torch.Tensor, weights: torch.Tensor,
                  num_kv_heads: int):
    """Row R4: advanced-index gather, drop the last retrieval row, kernel layout.

    chunk_k/v (N, C, S, Hkv*d); indices/weights (N, C, K).  Row c of the
    retrieval feeds the queries of chunk c+1, so the last row is dropped
    (model/DRT.py:629, :636).  Returns k, v as ((N (C-1)), Hkv, K, S, d) and
    weights as ((N (C-1)), K)   (model/DRT.py:198-199, :328-330).
    """
    N, C, S, Dm = chunk_k.shape
    K = indices.shape[-1]
    d = Dm // num_kv_heads
    idx = indices[:, :-1, :].reshape(N, (C - 1) * K)
    bidx = torch.arange(N, device=chunk_k.device).unsqueeze(1)
    k = chunk_k[bidx, idx]                                       # (N, (C-1)K, S, Dm)
    v = chunk_v[bidx, idx]
    k = k.reshape(N, C - 1, K, S, num_kv_heads, d).permute(0, 1, 4, 2, 3, 5).reshape(N * (C - 1), num_kv_heads, K, S, d)
    v = v.reshape(N, C - 1, K, S, num_kv_heads, d).permute(0, 1, 4, 2, 3, 5).reshape(N * (C - 1), num_kv_heads, K, S, d)
    w = weights[:, :-1, :].reshape(N * (C - 1), K)
    return k.contiguous(), v.contiguous(), w.contiguous()


# --------------------------------------------------------------------------- attention

def softmax_n(s: torch.Tensor, sm_n: float) -> torch.Tensor:
    """P = exp(s) / (sm_n + sum exp(s)) along the last dim, computed stably.

    sm_n == 0 is ordinary softmax; sm_n == 1 equals softmax([s, 0])[..., :-1].
    """
    if sm_n == 0:
        return torch.softmax(s, dim=-1)
    m = s.amax(dim=-1, keepdim=True).clamp_min(0.0)
    e = torch.exp(s - m)
    return e / (sm_n * torch.exp(-m) + e.sum(dim=-1, keepdim=True))


def _expand_kv(x: torch.Tensor, group: int) -> torch.Tensor:
    # query head h reads kv head h // group  (ltriton/gca.py:115-117, :912-913)
    return x if group == 1 else torch.repeat_interleave(x, repeats=group, dim=1)


def gca_forward(q, k, v, weights, sm_scale: float, sm_n: float = 0.0, p_dtype: Optional[torch.dtype] = None,
                return_parts: bool = False):
    """Row R5.  q (Z,Hq,Q,d); k, v (Z,Hkv,K,S,d); weights (Z,K)  ->  o (Z,Hq,Q,d).

    O_j = softmax_n(sm_scale * Q K_j^T) V_j ;  O = sum_j weights[z, j] * O_j
    (ltriton/gca.py:914-921).  ``p_dtype`` optionally rounds P before P.V the way
    the reference's bf16 oracle does (:917).
    """
    G = q.shape[1] // k.shape[1]
    k_, v_ = _expand_kv(k, G), _expand_kv(v, G)
    s = torch.einsum('zhmd,zhknd->zhkmn', q, k_) * sm_scale
    p = softmax_n(s, sm_n)
    if p_dtype is not None:
        p = p.to(p_dtype).to(s.dtype)
    o_k = torch.einsum('zhkmn,zhknd->zhkmd', p, v_)
    o = torch.einsum('zhkmd,zk->zhmd', o_k, weights.to(o_k.dtype))
    if return_parts:
        return o, o_k, p, s
    return o


def gca_lse2(q, k, sm_scale: float, sm_n: float = 0.0) -> torch.Tensor:
    """Base-2 log of the softmax denominator of the log2-scaled scores,
    lse2[z,h,j,m] = log2(sm_n + sum_n exp(s[z,h,j,m,n])), laid out (Z,Hq,K,Q).
    (The reference keeps the same quantity as M[z,h,m,j], ltriton/gca.py:197.)"""
    G = q.shape[1] // k.shape[1]
    s = torch.einsum('zhmd,zhknd->zhkmn', q, _expand_kv(k, G)) * sm_scale
    if sm_n == 0:
        lse = torch.logsumexp(s, dim=-1)
    else:
        z = torch.full_like(s[..., :1], math.log(sm_n))
        lse = torch.logsumexp(torch.cat([s, z], dim=-1), dim=-1)
    return lse * LOG2E


def gca_backward(q, k, v, weights, do, sm_scale: float, sm_n: float = 0.0):
    """Row R6, explicit formulas (ltriton/gca.py:379-404, :468-479, :839-840):

    D_j = rowsum(O_j * dO) = rowsum(P_j * dP_j);  dw[z,j] = sum_{h,m} D_j
    dV_j = w_j P_j^T dO;  dP_j = dO V_j^T;  dS_j = w_j P_j * (dP_j - D_j)
    dK_j = sm_scale dS_j^T Q;  dQ = sm_scale sum_j dS_j K_j
    Gradients of kv heads sum over the query heads of their group.
    Returns (dq, dk, dv, dw).
    """
    Z, Hq, Q, d = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    k_, v_ = _expand_kv(k, G), _expand_kv(v, G)
    o, o_k, p, _ = gca_forward(q, k, v, weights, sm_scale, sm_n, return_parts=True)
    w = weights.to(o_k.dtype)
    delta = torch.einsum('zhkmd,zhmd->zhkm', o_k, do)            # D_j
    dw = delta.sum(dim=(1, 3))
    dp = torch.einsum('zhmd,zhknd->zhkmn', do, v_)
    ds = p * (dp - delta.unsqueeze(-1)) * w[:, None, :, None, None]
    dq = sm_scale * torch.einsum('zhkmn,zhknd->zhmd', ds, k_)
    dk_ = sm_scale * torch.einsum('zhkmn,zhmd->zhknd', ds, q)
    dv_ = torch.einsum('zhkmn,zhmd->zhknd', p * w[:, None, :, None, None], do)
    K, S = k.shape[2], k.shape[3]
    dk = dk_.reshape(Z, Hkv, G, K, S, d).sum(dim=2)
    dv = dv_.reshape(Z, Hkv, G, K, S, d).sum(dim=2)
    return dq, dk, dv, dw


def gca_forward_backward_autograd(q, k, v, weights, do, sm_scale, sm_n=0.0, p_dtype=None):
    """What the reference test does to get its expected gradients
    (ltriton/gca.py:922-926): autograd through the einsum forward."""
    q, k, v, weights = [t.detach().clone().requires_grad_(True) for t in (q, k, v, weights)]
    o = gca_forward(q, k, v, weights, sm_scale, sm_n, p_dtype=p_dtype)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad, weights.grad


# --------------------------------------------------------------------------- caller contract

def gca_layer(q_all, chunk_k, chunk_v, lmk_q, lmk_k, chunk_topk: int, num_kv_heads: int, sm_n: float = 0.0,
              hidden_size: Optional[int] = None, noise=None):
    """Rows R1-R5 + the caller's conventions (model/DRT.py:345-398, :609-641).

    q_all (N, C, Hq, S, d) holds the projected queries of every chunk; chunk 0
    has nothing to retrieve, so its output is zero (model/DRT.py:369, :387-394)
    and retrieval row c feeds query chunk c+1.  sm_scale = 1/sqrt(d)
    (model/DRT.py:380).  Returns (out (N, C, Hq, S, d), indices, weights).
    """
    N, C, Hq, S, d = q_all.shape
    _, indices, weights = retrieve(lmk_q, lmk_k, chunk_topk, hidden_size, noise)
    k, v, w = gather_chunks(chunk_k, chunk_v, indices, weights, num_kv_heads)
    q = q_all[:, 1:].reshape(N * (C - 1), Hq, S, d)
    o = gca_forward(q, k, v, w, 1.0 / math.sqrt(d), sm_n)
    out = torch.zeros_like(q_all)
    out[:, 1:] = o.reshape(N, C - 1, Hq, S, d)
    return out, indices, weights


# --------------------------------------------------------------------------- the sub-layer around the kernel

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last dim (the RMSNorm of model/DRT.py:314, :353)."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def gca_module_forward(hidden, chunk_k, chunk_v, indices, weights, norm_w, eps, wq, bq, wo, bo, num_heads: int,
                       num_kv_heads: int, sm_n: float = 0.0, sm_n_functional: bool = False):
    """TritonGroupCrossAttention.forward for chunk_size > 1, step by step (model/DRT.py:345-398):
    pre_norm -> q_proj -> 'N D S (h d) -> N D h S d' -> drop chunk 0 -> '(N D) h S d' -> kernel with
    sm_scale = 1/sqrt(d) -> '(N D) h S d -> N (D S) (h d)' -> o_proj -> zero-filled result whose last
    (C-1)*S rows are the output.  hidden (N, C, S, dim); indices/weights (N, C, kk) from the retrieval.

    ``sm_n`` is what the module passes to its kernel (1.0 with enable_softmax_one, model/DRT.py:317-318).  Inside
    the reference's kernels it is numerically inert: the denominator starts at sm_n and is multiplied by
    exp2(m_i - m_ij) = exp2(-inf) = 0 on the first key tile (ltriton/gca.py:186-187, :48-49); the model's "+1"
    is the zeroed landmark row the caller stores in chunk_k / chunk_v (model/DRT.py:771-779).  So the
    restatement evaluates the plain softmax whatever sm_n is; ``sm_n_functional=True`` states the other
    reading (denominator sm_n + sum exp) for caches stored without that row."""
    N, C, S, dim = hidden.shape
    d = dim // num_heads
    x = rms_norm(hidden, norm_w, eps)
    q = F.linear(x, wq, bq)                                             # (N, C, S, h*d)
    q = q.reshape(N, C, S, num_heads, d).permute(0, 1, 3, 2, 4)         # N D h S d
    q = q[:, 1:].reshape(N * (C - 1), num_heads, S, d)                  # model/DRT.py:369-372
    k, v, w = gather_chunks(chunk_k, chunk_v, indices, weights, num_kv_heads)
    vals = gca_forward(q, k, v, w, 1.0 / math.sqrt(d), sm_n if sm_n_functional else 0.0)   # ((N D), h, S, d)
    vals = vals.reshape(N, C - 1, num_heads, S, d).permute(0, 1, 3, 2, 4).reshape(N, (C - 1) * S, num_heads * d)
    o = F.linear(vals, wo, bo)
    ret = torch.zeros((N, C * S, dim), dtype=o.dtype, device=o.device)
    ret[:, -o.shape[1]:, :] = o                                         # model/DRT.py:387-394
    return ret
