"""Split attention with a sliding window and with attention dropout, on the GPU: the kernel
instances of their own that a window or a dropout rate selects, forward and the three
gradients against the oracle.  Collected after ``tests/test_split_attention.py``, whose cases
(no window, no dropout) run the instances that take neither."""

import pytest
import torch

from arctic_platform_amd.split_attention import SplitLayout, dropout_keep_mask, split_attention
from oracle.split_attention import split_attention as oracle_split, total_tokens
from tests.test_split_attention import LAYOUTS, _close, _inputs, _run_case


@pytest.mark.gpu
@pytest.mark.parametrize("window", [1, 20, 32, 100, 4096])
@pytest.mark.parametrize("heads", [(8, 2, 128), (6, 2, 64), (4, 4, 128)])
def test_sliding_window_matches_the_oracle(heads, window):
    """The window of the trainer's attention calls (qwen_attention_patcher.py:1206, :1226):
    shorter than a tile, a tile, across tiles, longer than every sample; the kernels that share
    their operands through LDS and the per-wave ones."""
    for layout in LAYOUTS:
        _run_case(layout, *heads, seed=51, window=window)


@pytest.mark.gpu
@pytest.mark.parametrize("dropout,window", [(0.1, None), (0.5, None), (0.25, 40)])
@pytest.mark.parametrize("heads", [(8, 2, 128), (6, 2, 64), (4, 4, 128)])
def test_attention_dropout_matches_the_oracle(heads, dropout, window):
    """Attention dropout (the trainer's calls pass module.attention_dropout while training,
    qwen_attention_patcher.py:1204, :1224): forward and the three gradients against the oracle
    under the same mask, which the host restates from the seed; alone and with a window."""
    for layout in LAYOUTS:
        _run_case(layout, *heads, seed=71, window=window, dropout=dropout)


@pytest.mark.gpu
def test_attention_dropout_through_autograd_repeats_under_a_seed():
    layout = [(70, [40, 33]), (20, [50])]
    hq, hkv, d = 8, 2, 128
    q, k, v = (x.cuda().requires_grad_() for x in _inputs(layout, hq, hkv, d, 81, torch.bfloat16))
    L = SplitLayout(layout)
    torch.manual_seed(5)
    a = split_attention(q, k, v, L, d**-0.5, dropout=0.2)
    torch.manual_seed(5)
    b = split_attention(q, k, v, L, d**-0.5, dropout=0.2)
    c = split_attention(q, k, v, L, d**-0.5, dropout=0.2)
    assert torch.equal(a, b) and not torch.equal(a, c)
    a.float().sum().backward()
    assert all(bool(torch.isfinite(x.grad.float()).all()) for x in (q, k, v))
    # the forward's seed reaches the backward: an explicit seed against the oracle
    q.grad = k.grad = v.grad = None
    out = split_attention(q, k, v, L, d**-0.5, dropout=0.2, seed=1234)
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(82)).bfloat16()
    (out.float() * w.cuda().float()).sum().backward()
    q64, k64, v64 = (x.detach().cpu().double().requires_grad_() for x in (q, k, v))
    keep = dropout_keep_mask(1234, 0.2, hq, total_tokens(layout))
    ro, _ = oracle_split(q64, k64, v64, layout, d**-0.5, keep=keep, dropout=0.2)
    (ro * w.double()).sum().backward()
    grow = 1.0 / (1.0 - 0.2)  # the bounds grow with the scale of the kept probabilities (see _run_case)
    _close("out", out, ro, grow * 2e-2 / max(1.0, float(ro.detach().abs().max())))
    for name, got, ref in (("dq", q.grad, q64.grad), ("dk", k.grad, k64.grad), ("dv", v.grad, v64.grad)):
        _close(name, got, ref, grow * 1e-2)


@pytest.mark.gpu
def test_sliding_window_through_autograd_and_on_long_responses():
    """Long responses over a long prompt with a window much shorter than either (most tiles of
    the walks are left out), through the autograd function with the window passed on the call."""
    layout = [(700, [400, 260]), (300, [500])]
    hq, hkv, d, window = 8, 2, 128, 128
    q, k, v = (x.cuda().requires_grad_() for x in _inputs(layout, hq, hkv, d, 61, torch.bfloat16))
    L = SplitLayout(layout, sliding_window=window)
    out = split_attention(q, k, v, L, d**-0.5, dropout=0.0, sliding_window=window)
    w = torch.randn(out.shape, generator=torch.Generator().manual_seed(62)).bfloat16()
    (out.float() * w.cuda().float()).sum().backward()
    q64, k64, v64 = (x.detach().cpu().double().requires_grad_() for x in (q, k, v))
    ro, _ = oracle_split(q64, k64, v64, layout, d**-0.5, window=window)
    (ro * w.double()).sum().backward()
    _close("out", out, ro, 2e-2 / max(1.0, float(ro.detach().abs().max())))
    for name, got, ref in (("dq", q.grad, q64.grad), ("dk", k.grad, k64.grad), ("dv", v.grad, v64.grad)):
        _close(name, got, ref, 1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("window", [1, 20, 64, 300])
def test_chunks_behind_a_context_under_a_window(window):
    """A layout of response rows only (a prefill chunk behind a cached context) made with a
    window: the chunk's rows equal the response rows of the whole computation under that window."""
    from arctic_platform_amd.split_attention import split_attention_forward

    layout = [(70, [45]), (0, [33]), (200, [64]), (16, [1])]
    hq, hkv, d = 8, 2, 128
    scale = d**-0.5
    q_all, k, v = _inputs(layout, hq, hkv, d, 5, torch.bfloat16)
    ro, _ = oracle_split(q_all.double(), k.double(), v.double(), layout, scale, window=window)
    L = SplitLayout(layout, responses_only=True, sliding_window=window)
    rows = torch.tensor(L.q_index()[: L.num_tokens] >= 0)
    out, _ = split_attention_forward(q_all[rows].cuda(), k.cuda(), v.cuda(), L, scale)
    _close("out", out, ro[rows], 2e-2 / max(1.0, float(ro.abs().max())))
