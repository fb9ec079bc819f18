"""Drop-in for the reference's ``ltriton/gca.py``: put this directory's parent on ``sys.path``
ahead of the reference checkout and ``from ltriton.gca import attention, gca_kv_cache``
(model/DRT.py:36-37) binds the MI355X HIP kernels instead of the Triton ones.

``sm_n`` handling.  In the reference's kernels the ``sm_n`` argument has no numerical effect:
the running denominator starts at ``sm_n`` but is multiplied by ``exp2(-inf) = 0`` on the first
key tile (ltriton/gca.py:186-187 with :48-49), and the backward never reads it.  The model gets
its "+1" from zeroing the landmark row of K and V instead (model/DRT.py:772-779).  To keep a
model that calls these two functions numerically where it was, this module ignores ``sm_n`` by
default (mode "reference").  Set ``ltriton.gca.SM_N_MODE = "functional"`` (or the environment
variable ``GCA_SM_N_MODE=functional``) to get P = exp(s) / (sm_n + sum exp(s)) from the same calls;
``gca_hip.attention`` always has the functional meaning.
"""
import os

from gca_hip import gca as _impl

SM_N_MODE = os.environ.get("GCA_SM_N_MODE", "reference")


def _sm_n(sm_n):
    assert SM_N_MODE in ("reference", "functional"), SM_N_MODE
    return float(sm_n) if SM_N_MODE == "functional" else 0.0


def attention(q, k, v, weights, sm_scale, sm_n):
    return _impl.attention(q, k, v, weights, sm_scale, _sm_n(sm_n))


def gca_kv_cache(q, k, v, weights, sm_scale, sm_n):
    return _impl.gca_kv_cache(q, k, v, weights, sm_scale, _sm_n(sm_n))
