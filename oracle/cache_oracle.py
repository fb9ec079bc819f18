"""CPU oracle for the chunk cache and the decode flow around the GCA kernels.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE (same rule as gca_oracle.py: only the tests, the smoke
check and the benchmark's CPU leg may import it).

It restates, with plain torch ops on the CPU, what the reference does between two kernel calls while
it generates (paths relative to the reference checkout):

* ``landmark_row``      model/DRT.py:769-779 (decode copy :804-813): a 64-row chunk gets its last row
                        (the landmark position) zeroed, a 65-row chunk loses it.
* ``ChunkCacheOracle``  model/DRT.py:75-232, non-offloading branches: append by ``torch.cat``,
                        ``update_current_retrieved_chunk`` keeps the LAST retrieval row's gathered chunks
                        and weights, ``retrieve_chunks`` is advanced indexing.
* ``prefill``           model/DRT.py:609-641 with ``use_cache`` (:638-639).
* ``end_of_chunk``      model/DRT.py:835-848: the landmark state of the chunk just appended is scored
                        against every stored landmark, row id = E-1 sees e < E-1 (:590-607 with one row).
* ``decode_attention``  model/DRT.py:825-831 + :320-332 + :382: the current gathered chunks in kernel
                        layout and the inference kernel (ltriton/gca.py:846-888), stated as gca_forward.

How it is pinned: these are indexing and concatenation only, on top of functions pinned in
gca_oracle.py.  The one property that a wrong row shift, a wrong mask row or a stale state would break
is checked in tests/test_oracle.py: generating a sequence chunk by chunk (1-token and 2-token steps)
reproduces, position for position, the batch form ``gca_layer`` of the whole sequence - the same
self-consistency the reference's tests/generation_unittest.py asserts on its model.  No reference test
holds vectors for this flow: parity unpinned beyond that property.
"""
from __future__ import annotations

import math

import torch

from . import gca_oracle as O


def landmark_row(chunk: torch.Tensor, mode: str) -> torch.Tensor:
    """chunk (..., S or S+1, Dm) -> stored form (model/DRT.py:769-779)."""
    if mode == "keep":
        return chunk
    if mode == "zero":
        out = chunk.clone()
        out[..., -1, :] = 0
        return out
    if mode == "drop":
        return chunk[..., :-1, :]
    raise ValueError(mode)


class ChunkCacheOracle:
    def __init__(self, group_size: int = 1):
        self.chunk_k = self.chunk_v = self.lmk_embs = None
        self.cur = [None] * group_size      # (k (N,K,S,Dm), v, weights (N,1,K), indices (N,K))

    def append(self, chunk_k, chunk_v, lmk_embs):                      # model/DRT.py:87-132
        if self.chunk_k is None:
            self.chunk_k, self.chunk_v, self.lmk_embs = chunk_k, chunk_v, lmk_embs
        else:
            assert chunk_k.shape[-2] == self.chunk_k.shape[-2]
            self.chunk_k = torch.cat([self.chunk_k, chunk_k], dim=1)
            self.chunk_v = torch.cat([self.chunk_v, chunk_v], dim=1)
            self.lmk_embs = torch.cat([self.lmk_embs, lmk_embs], dim=1)

    def retrieve_chunks(self, indices):                                # model/DRT.py:193-200
        b = torch.arange(indices.shape[0]).unsqueeze(1)
        return self.chunk_k[b, indices], self.chunk_v[b, indices]

    def update_current_retrieved_chunk(self, indices, weights, group_idx):   # model/DRT.py:158-185
        if indices.dim() == 3:
            indices = indices[:, -1, :]
        k, v = self.retrieve_chunks(indices)
        self.cur[group_idx] = (k, v, weights[:, -1:, :], indices)


def prefill(cache: ChunkCacheOracle, lmk_q, topk: int, group_idx: int = 0, hidden_size=None):
    """Retrieval of a whole prompt, last row kept as decode state (model/DRT.py:609-641)."""
    _, indices, weights = O.retrieve(lmk_q, cache.lmk_embs, topk, hidden_size)
    cache.update_current_retrieved_chunk(indices, weights, group_idx)
    return indices, weights


def end_of_chunk(cache: ChunkCacheOracle, lmk_q_row, topk: int, group_idx: int = 0, hidden_size=None):
    """lmk_q_row (N, 1, Dl): landmark state of the chunk appended last (model/DRT.py:835-848)."""
    scores = O.landmark_scores(lmk_q_row, cache.lmk_embs, hidden_size)        # model/DRT.py:838
    E = scores.shape[2]
    dec_ids = torch.arange(E)[-1:]                                     # model/DRT.py:596-597
    visible = dec_ids.unsqueeze(1) > torch.arange(E).unsqueeze(0)
    scores = scores.masked_fill(~visible, float("-inf"))
    kk = min(E, topk)
    _, indices = O.topk_canonical(scores, kk)
    weights = O.retrieval_weights(scores, indices)
    cache.update_current_retrieved_chunk(indices.squeeze(1), weights[:, :1, :], group_idx)
    return indices, weights


def decode_attention(cache: ChunkCacheOracle, q, num_kv_heads: int, group_idx: int = 0, sm_n: float = 0.0):
    """q (N, Hq, Q, d) -> (N, Hq, Q, d) against the group's current chunks (model/DRT.py:825-831, :382)."""
    k, v, w, _ = cache.cur[group_idx]
    N, K, S, Dm = k.shape
    d = Dm // num_kv_heads
    k = k.reshape(N, K, S, num_kv_heads, d).permute(0, 3, 1, 2, 4)      # 'N (D K) S (h d) -> (N D) h K S d', D = 1
    v = v.reshape(N, K, S, num_kv_heads, d).permute(0, 3, 1, 2, 4)
    return O.gca_forward(q, k, v, w.reshape(N, K), 1.0 / math.sqrt(q.shape[-1]), sm_n)


def generate(q_all, chunk_k, chunk_v, lmk_q, lmk_k, topk: int, num_kv_heads: int, prompt_chunks: int,
             sm_n: float = 0.0, hidden_size=None, steps=(1,)):
    """Chunk-by-chunk generation over given per-position tensors.

    The first ``prompt_chunks`` chunks are the prompt (batch retrieval, model/DRT.py:609-641); every later
    chunk c is attended token by token (query steps of the sizes cycled from ``steps``, the last step of a
    chunk takes whatever rows are left) with the state left by chunk c-1, then appended and scored.
    q_all (N, C, Hq, S, d); chunk_k/v (N, C, S, Dm); lmk_q/lmk_k (N, C, Dl).
    Returns (out (N, C, Hq, S, d) with the prompt's chunks left zero, list of per-chunk indices (N, kk))."""
    N, C, Hq, S, d = q_all.shape
    cache = ChunkCacheOracle()
    P = prompt_chunks
    cache.append(chunk_k[:, :P], chunk_v[:, :P], lmk_k[:, :P])
    prefill(cache, lmk_q[:, :P], topk, 0, hidden_size)
    out = torch.zeros_like(q_all)
    picked = []
    for c in range(P, C):
        picked.append(cache.cur[0][3].clone())
        s, i = 0, 0
        while s < S:
            n = min(steps[i % len(steps)], S - s)
            out[:, c, :, s:s + n] = decode_attention(cache, q_all[:, c, :, s:s + n], num_kv_heads, 0, sm_n)
            s += n
            i += 1
        cache.append(chunk_k[:, c:c + 1], chunk_v[:, c:c + 1], lmk_k[:, c:c + 1])
        end_of_chunk(cache, lmk_q[:, c:c + 1], topk, 0, hidden_size)
    return out, picked
