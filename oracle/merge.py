"""Log-sum-exp merge of partial attention results.

Follows the running-max / rescaled-sum update with guards for non-finite maxima of
``_online_logsumexp_and_weighted_update``
(arctic_platform/model/implementations/qwen35/models/layers/lm_head.py:190-202):
m' = max(m, m_i); old terms are rescaled by exp(m - m') only where m is finite; an
empty partial (lse = -inf) contributes nothing.
"""

from __future__ import annotations

import torch


def merge_partials(outs, lses):
    """outs ``[P, ..., D]``, lses ``[P, ...]`` -> (out ``[..., D]``, lse ``[...]``).

    Each partial is a normalised attention output over a disjoint token set together
    with the natural-log sum of its exponentiated scores.  All partials empty gives
    out = 0 and lse = -inf.
    """
    m = torch.full_like(lses[0], float("-inf"))
    s = torch.zeros_like(lses[0])
    acc = torch.zeros_like(outs[0])
    for o, l in zip(outs, lses):
        m_new = torch.maximum(m, l)
        old = torch.where(torch.isfinite(m), torch.exp(m - m_new), torch.zeros_like(m))
        live = torch.isfinite(l)
        w = torch.where(live, torch.exp(torch.where(live, l - m_new, torch.zeros_like(l))), torch.zeros_like(l))
        s = s * old + w
        acc = acc * old[..., None] + torch.where(live[..., None], o, torch.zeros_like(o)) * w[..., None]
        m = m_new
    safe = torch.where(s > 0, s, torch.ones_like(s))
    out = acc / safe[..., None]
    lse = torch.where(s > 0, m + torch.log(safe), torch.full_like(m, float("-inf")))
    return out, lse
