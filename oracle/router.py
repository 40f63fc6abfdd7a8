"""CPU restatement of the router top-k reference (test infrastructure only; never on a product path).

Follows ``router_topk_torch_ref`` (src/nkilib_src/nkilib/core/router_topk/router_topk_torch.py:23-135):
logits = x @ w (+ bias); the k largest logits per token (``argsort(-logits)[:, :k]``, :83-84); then either
  * ``router_pre_norm`` (:87-107): activate all E logits (softmax :90 / sigmoid :92); with ``norm_topk_prob``
    keep the selected experts' values and divide by their sum (:97-105), otherwise return the full activation;
  * else (:108-129): activate only the k selected logits (softmax over the k values / sigmoid) and scatter them
    into zeros.
Arithmetic is fp32 on the bf16-valued inputs (the reference's bf16 tensors make torch round the logits to bf16
before the argsort, which ties many experts; which of tied experts ``argsort`` returns is unspecified, so that
behaviour is parity unpinned and this restatement breaks ties towards the lower expert index).
"""

import numpy as np

SIGMOID, SOFTMAX = 0, 1  # RouterActFnType, src/nkilib_src/nkilib/core/utils/common_types.py:39-43


def router_topk_ref(x, w, w_bias, act_fn, k, router_pre_norm=True, norm_topk_prob=False):
    """x [T,H], w [H,E], w_bias [E] or None (float arrays holding bf16 values).  Returns a dict with
    ``router_logits`` [T,E] fp32, ``expert_index`` [T,k] int32 (descending logit, ties to the lower index) and
    ``expert_affinities`` [T,E] fp32."""
    x = np.asarray(x, dtype=np.float32)
    w = np.asarray(w, dtype=np.float32)
    logits = (x.astype(np.float64) @ w.astype(np.float64)).astype(np.float32)
    if w_bias is not None:
        logits = logits + np.asarray(w_bias, dtype=np.float32).reshape(1, -1)
    T, E = logits.shape
    idx = np.argsort(-logits, axis=-1, kind="stable")[:, :k].astype(np.int32)
    rows = np.arange(T)[:, None]
    if router_pre_norm:
        if act_fn == SOFTMAX:
            z = np.exp(logits - logits.max(axis=1, keepdims=True))
            full = z / z.sum(axis=1, keepdims=True)
        elif act_fn == SIGMOID:
            full = 1.0 / (1.0 + np.exp(-logits))
        else:
            raise NotImplementedError(act_fn)
        if norm_topk_prob:
            sel = np.zeros((T, E), dtype=np.float32)
            sel[rows, idx] = full[rows, idx]
            aff = sel / sel.sum(axis=1, keepdims=True)
        else:
            aff = full
    else:
        top = logits[rows, idx]
        if act_fn == SOFTMAX:
            z = np.exp(top - top.max(axis=1, keepdims=True))
            act = z / z.sum(axis=1, keepdims=True)
        elif act_fn == SIGMOID:
            act = 1.0 / (1.0 + np.exp(-top))
        else:
            raise NotImplementedError(act_fn)
        aff = np.zeros((T, E), dtype=np.float32)
        aff[rows, idx] = act
    return {"router_logits": logits, "expert_index": idx, "expert_affinities": aff.astype(np.float32)}


def topk_gap(logits, k):
    """Per token: the difference between its k-th and (k+1)-th largest logit (how far the selection is from a tie)."""
    s = -np.sort(-np.asarray(logits, dtype=np.float64), axis=-1)
    return s[:, k - 1] - s[:, k] if s.shape[1] > k else np.full(s.shape[0], np.inf)
