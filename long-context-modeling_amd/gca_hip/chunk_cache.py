"""Device-resident chunk cache: the storage the indexed GCA kernels read.

Mirrors ``ChunkKVManager`` of the reference (model/DRT.py:75-232) method for method, with a different
storage policy.  The reference grows its cache with ``torch.cat`` (the whole cache is copied on every
append) and keeps a gathered copy of the currently retrieved chunks per layer group.  Here K, V and the
landmarks live in buffers allocated with spare capacity (doubling), an append is one copy of the new chunks
(kernel ``chunk_cache_append``, which can zero or drop the landmark row on the way,
model/DRT.py:769-779), and the decode state per group is the retrieved chunk *ids* and weights: the
indexed kernels read the chunks from the cache itself.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib
from .gca import _DT, _ptr, _stream, gca_kv_cache, gca_kv_cache_indexed
from .retrieval import gather_rows, landmark_retrieve

_LMK_ROW = {"keep": _lib.CHUNK_LMK_KEEP, "zero": _lib.CHUNK_LMK_ZERO, "drop": _lib.CHUNK_LMK_DROP}


def chunk_cache_append(src_k, src_v, src_lmk, k_store, v_store, lmk_store, count, landmark_row="keep"):
    """Copy ``src_k/src_v`` (N, n_new, S or S+1, Dm) and ``src_lmk`` (N, n_new, Dl) into slots
    ``count .. count+n_new-1`` of stores shaped (N, capacity, S, Dm) / (N, capacity, Dl)."""
    assert src_k.is_cuda and src_k.dtype in _DT and src_k.dim() == 4 and src_v.shape == src_k.shape
    assert k_store.dtype == src_k.dtype and v_store.dtype == src_k.dtype and k_store.shape == v_store.shape
    assert k_store.is_contiguous() and v_store.is_contiguous()
    src_k, src_v = src_k.contiguous(), src_v.contiguous()
    N, n_new, S_src, Dm = src_k.shape
    _, capacity, S, _ = k_store.shape
    assert k_store.shape[0] == N and k_store.shape[3] == Dm
    assert S_src == (S + 1 if landmark_row == "drop" else S), "source chunk rows do not match the store"
    Dl = 0
    if src_lmk is not None:
        assert lmk_store is not None and lmk_store.is_contiguous() and lmk_store.dtype == src_k.dtype
        assert src_lmk.dtype == src_k.dtype and src_lmk.shape[:2] == (N, n_new) and lmk_store.shape[:2] == (N, capacity)
        src_lmk = src_lmk.contiguous()
        Dl = src_lmk.shape[2]
        assert lmk_store.shape[2] == Dl
    desc = _lib.ChunkCacheDesc(dtype=_DT[src_k.dtype], lmk_row=_LMK_ROW[landmark_row], N=N, capacity=capacity,
                               count=int(count), n_new=n_new, S=S, Dm=Dm, Dl=Dl, reserved=0)
    with torch.cuda.device(src_k.device):
        rc = _lib.lib().chunk_cache_append(ctypes.byref(desc), _ptr(src_k), _ptr(src_v), _ptr(src_lmk), _ptr(k_store),
                                           _ptr(v_store), _ptr(lmk_store) if src_lmk is not None else None,
                                           _stream(src_k.device))
    _lib.check(rc, "chunk_cache_append")


class ChunkKVManager:
    """Chunk K/V cache + landmark store + per-group decode state (model/DRT.py:75-232).

    ``chunk_k``, ``chunk_v`` (N, C, S, Dm) and ``lmk_embs`` (N, C, Dl) are views of the filled part of
    the stores; ``k_store`` / ``v_store`` (N, capacity, S, Dm) are what the indexed kernels take.

    A first append of tensors that carry gradients (training: one append per forward, DRT.py:779) adopts
    them without a copy, so autograd reaches the projections that produced them, exactly like the
    reference; stores with spare capacity start with the second append or with ``capacity=``.

    ``offloading=True`` keeps K and V in pinned host memory like the reference's list-of-CPU-tensors
    (DRT.py:90-128), landmarks stay on the GPU, and retrieved chunks are copied back on demand.
    """

    def __init__(self, offloading=False, group_size=1, capacity=0):
        self.group_size = group_size
        self._offloading = offloading
        self._min_capacity = int(capacity)
        self._k = self._v = self._lmk = None     # stores
        self._count = 0
        self._device = None
        self._cur_idx = [None] * group_size       # (N, K) int64
        self._cur_w = [None] * group_size         # (N, 1, K)
        self._cur_all = [False] * group_size      # "the whole one-chunk cache" state of DRT.py:186-191
        self._current_hidden_states = None

    # ---- storage -----------------------------------------------------------------------------
    @property
    def count(self):
        return self._count

    @property
    def capacity(self):
        return 0 if self._k is None else self._k.shape[1]

    @property
    def k_store(self):
        return self._k

    @property
    def v_store(self):
        return self._v

    @property
    def chunk_k(self):
        return None if self._k is None else self._k[:, :self._count]

    @property
    def chunk_v(self):
        return None if self._v is None else self._v[:, :self._count]

    @property
    def lmk_embs(self):
        return None if self._lmk is None else self._lmk[:, :self._count]

    @property
    def past_lmk_embeds(self):
        return self.lmk_embs

    def _new_store(self, like, capacity, pinned):
        shape = (like.shape[0], capacity) + tuple(like.shape[2:])
        if pinned:
            return torch.empty(shape, dtype=like.dtype, device="cpu", pin_memory=True)
        return torch.empty(shape, dtype=like.dtype, device=like.device)

    def _grow(self, need, like_k, like_lmk):
        cap = max(need, 2 * self.capacity, self._min_capacity)
        k = self._new_store(like_k, cap, self._offloading)
        v = self._new_store(like_k, cap, self._offloading)
        lmk = self._new_store(like_lmk, cap, False)
        if self._count:
            k[:, :self._count].copy_(self._k[:, :self._count])
            v[:, :self._count].copy_(self._v[:, :self._count])
            lmk[:, :self._count].copy_(self._lmk[:, :self._count])
        self._k, self._v, self._lmk = k, v, lmk

    def append(self, chunk_k, chunk_v, lmk_embs, landmark_row="keep"):
        """chunk_k, chunk_v (N, n_new, S, Dm) (S+1 rows with ``landmark_row="drop"``), lmk_embs (N, n_new, Dl)
        (DRT.py:87-132).  ``landmark_row="zero"`` stores each chunk's last row as zeros, the softmax-off-by-one
        trick of DRT.py:771-772, without touching the caller's tensor."""
        assert chunk_k.dim() == 4 and chunk_v.shape == chunk_k.shape and lmk_embs.dim() == 3
        n_new = chunk_k.shape[1]
        S = chunk_k.shape[2] - (1 if landmark_row == "drop" else 0)
        if self._k is not None:
            assert S == self._k.shape[2], "chunk length differs from the cache's"    # DRT.py:103
        self._device = chunk_k.device
        adopt = (self._k is None and not self._offloading and self._min_capacity <= n_new and
                 torch.is_grad_enabled() and (chunk_k.requires_grad or chunk_v.requires_grad or lmk_embs.requires_grad))
        if adopt:
            if landmark_row == "zero":
                keep = torch.ones(S, 1, device=chunk_k.device, dtype=chunk_k.dtype)
                keep[-1] = 0
                chunk_k, chunk_v = chunk_k * keep, chunk_v * keep
            elif landmark_row == "drop":
                chunk_k, chunk_v = chunk_k[:, :, :-1], chunk_v[:, :, :-1]
            self._k, self._v, self._lmk = chunk_k.contiguous(), chunk_v.contiguous(), lmk_embs.contiguous()
            self._count = n_new
            return
        chunk_k, chunk_v, lmk_embs = chunk_k.detach(), chunk_v.detach(), lmk_embs.detach()
        if self._count + n_new > self.capacity:
            self._grow(self._count + n_new, chunk_k[:, :, :S], lmk_embs)
        if self._offloading:
            if landmark_row == "drop":
                chunk_k, chunk_v = chunk_k[:, :, :-1], chunk_v[:, :, :-1]
            sl = slice(self._count, self._count + n_new)
            self._k[:, sl].copy_(chunk_k)      # blocking: the host reads these rows when chunks are retrieved
            self._v[:, sl].copy_(chunk_v)
            if landmark_row == "zero":
                self._k[:, sl, -1].zero_()
                self._v[:, sl, -1].zero_()
            self._lmk[:, sl].copy_(lmk_embs)
        else:
            chunk_cache_append(chunk_k, chunk_v, lmk_embs, self._k, self._v, self._lmk, self._count, landmark_row)
        self._count += n_new

    # ---- lower-layer hidden states of the chunk being generated (DRT.py:141-156) -------------------
    @property
    def lower_hidden_states(self):
        return self._current_hidden_states

    def clear_lower_hidden_states(self):
        self._current_hidden_states = None

    def cache_lower_hidden_states(self, hidden_states):
        if self._current_hidden_states is None:
            self._current_hidden_states = hidden_states
        else:
            self._current_hidden_states = torch.cat([self._current_hidden_states, hidden_states], dim=1)

    # ---- retrieval state ---------------------------------------------------------------------------
    def update_current_retrieved_chunk(self, indices, weights, group_idx):
        """Remember what the chunk being generated attends to (DRT.py:158-191): the last row of
        ``indices`` (N, C, K) or (N, K) and of ``weights`` (N, C, K).  Only ids and weights are kept."""
        if indices.shape[1] > 0:
            if indices.dim() == 3:
                indices = indices[:, -1, :]
            self._cur_idx[group_idx] = indices.contiguous()
            self._cur_w[group_idx] = weights[:, -1:, :]
            self._cur_all[group_idx] = False
        else:
            assert self._count == 1      # DRT.py:186-187
            self._cur_idx[group_idx] = torch.zeros((indices.shape[0], 1), dtype=torch.int64, device=self._device)
            self._cur_w[group_idx] = weights
            self._cur_all[group_idx] = True

    def current_retrieved_indices(self, group_idx=0):
        """(indices (N, K) int64, weights (N, 1, K)) of the chunk being generated."""
        return self._cur_idx[group_idx], self._cur_w[group_idx]

    def current_retrieved_chunk(self, group_idx=0):
        """Gathered form (k, v (N, K, S, Dm), weights (N, 1, K)) as the reference keeps it
        (DRT.py:138-139); the decode path of this package does not need it."""
        idx = self._cur_idx[group_idx]
        if idx is None:
            return None, None, None
        if self._cur_all[group_idx]:
            k, v = self.chunk_k, self.chunk_v
            if self._offloading:
                k, v = k.to(self._device), v.to(self._device)
            return k, v, self._cur_w[group_idx]
        k, v = self.retrieve_chunks(idx)
        return k, v, self._cur_w[group_idx]

    def retrieve_chunks(self, indices):
        """k, v = cache[n, indices[n, i]] -> (N, len, S, Dm) (DRT.py:193-220)."""
        N = indices.shape[0]
        if not self._offloading:
            return gather_rows(self.chunk_k, self.chunk_v, indices)
        ci = indices.cpu()
        b = torch.arange(N).unsqueeze(1)
        # gather into pinned staging so the copy to the device is one asynchronous transfer per tensor
        out = []
        for store in (self._k, self._v):
            stage = torch.empty((N, ci.shape[1]) + tuple(store.shape[2:]), dtype=store.dtype, pin_memory=True)
            torch.index_select(store.view(-1, *store.shape[2:]), 0, (b * store.shape[1] + ci).reshape(-1),
                               out=stage.view(-1, *store.shape[2:]))
            out.append(stage.to(self._device, non_blocking=True))
        return out[0], out[1]

    def reorder(self, beam_idx):
        """Beam-search reordering of every per-sequence tensor (DRT.py:222-232)."""
        for name in ("_k", "_v", "_lmk"):
            t = getattr(self, name)
            if t is not None:
                setattr(self, name, t.index_select(0, beam_idx.to(t.device)))
        for g in range(self.group_size):
            if self._cur_idx[g] is not None:
                self._cur_idx[g] = self._cur_idx[g].index_select(0, beam_idx.to(self._cur_idx[g].device))
                self._cur_w[g] = self._cur_w[g].index_select(0, beam_idx.to(self._cur_w[g].device))

    # ---- the two retrieval sites of the model and the decode-step attention ----------------------------
    def batch_retrieval(self, lmk_q, topk, group_idx=0, hidden_size=None, noise=None, use_cache=False,
                        max_chunk_win=-1):
        """Scoring, mask, top-k and weights of ``lmk_q`` (N, C, Dl) against all stored landmarks
        (DRT._perform_batch_retrieval, DRT.py:609-641, without the gather).  With ``use_cache`` the last
        row becomes the decode state of the group (DRT.py:638-639).  ``max_chunk_win`` is the mask's window
        (DRT.py:590-603; the model leaves it at -1).  Returns (indices, weights) (N, C, kk)."""
        _, indices, weights = landmark_retrieve(lmk_q, self.lmk_embs, topk, hidden_size, True, noise, True,
                                                max_chunk_win)
        if use_cache and not torch.is_grad_enabled():
            self.update_current_retrieved_chunk(indices, weights, group_idx)
        return indices, weights

    def step_retrieval(self, lmk_q, topk, group_idx=0, hidden_size=None):
        """End of a generated chunk (DRT.py:835-848): ``lmk_q`` (N, 1, Dl) is the landmark state of the chunk
        that was just appended; it sees every chunk before that one.  Updates the group's decode state."""
        assert lmk_q.shape[1] == 1
        _, indices, weights = landmark_retrieve(lmk_q, self.lmk_embs, topk, hidden_size, True, None)
        self.update_current_retrieved_chunk(indices.squeeze(1), weights[:, :1, :], group_idx)
        return indices, weights

    def decode_attention(self, q, group_idx=0, sm_n=0.0):
        """GCA of the tokens being generated, q (N, Hq, Q, d) with Q = 1 or 2 (any Q works), against the
        group's retrieved chunks (DRT.py:825-831 + :382, kernel ltriton/gca.py:846-888).  Returns (N, Hq, Q, d)."""
        idx, w = self._cur_idx[group_idx], self._cur_w[group_idx]
        assert idx is not None, "no retrieval state: call batch_retrieval(use_cache=True) or step_retrieval first"
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
        w2 = w.reshape(w.shape[0], w.shape[-1]).contiguous()
        if self._offloading:
            k, v, _ = self.current_retrieved_chunk(group_idx)
            N, K, S, Dm = k.shape
            d = q.shape[-1]
            k = k.view(N, K, S, Dm // d, d).permute(0, 3, 1, 2, 4).contiguous()
            v = v.view(N, K, S, Dm // d, d).permute(0, 3, 1, 2, 4).contiguous()
            return gca_kv_cache(q.contiguous(), k, v, w2, sm_scale, sm_n)
        return gca_kv_cache_indexed(q.contiguous(), self._k, self._v, idx, w2, sm_scale, sm_n)
