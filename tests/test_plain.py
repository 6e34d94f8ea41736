"""What fixes the plain implementation besides the reference's text: library routines it must
reduce to, invariants, and vectors from the reference's own tests (no GPU)."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain_model import (plain_apply_mrope, plain_attention, plain_filtered_probs, plain_forward, plain_inv_freq,
                         plain_layer_windows, plain_mlp, plain_model_logits, plain_mrope_cos_sin, plain_penalties,
                         plain_read_config, plain_read_weights, plain_rmsnorm)


def test_rmsnorm_is_the_library_routine_and_scale_free():
    torch.manual_seed(0)
    x, w = torch.randn(5, 37), torch.randn(37)
    assert torch.allclose(plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (37,), w, 1e-5), atol=1e-6)
    ones = torch.ones(37)
    y = plain_rmsnorm(x, ones, 1e-6)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5), atol=1e-4)        # unit mean square
    assert torch.allclose(plain_rmsnorm(7.5 * x, ones, 1e-12), plain_rmsnorm(x, ones, 1e-12), atol=1e-5)
    # eps sits inside the root: for x = 0 the result is 0, for tiny x it damps
    tiny = torch.full((1, 4), 1e-4)
    assert torch.allclose(plain_rmsnorm(tiny, torch.ones(4), 1e-6), tiny / math.sqrt(1e-8 + 1e-6), rtol=1e-5)
    # the weight multiplies as stored, not as 1 + w
    assert torch.allclose(plain_rmsnorm(x, torch.zeros(37), 1e-6), torch.zeros(5, 37))


def _rotate_complex(x, pos, theta):
    """Standard 1-D rotary embedding in the rotate-half pairing: (x[f], x[f + hd/2]) as a complex
    number times e^{i pos inv_freq[f]}."""
    hd = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd))
    ang = pos.to(torch.float64)[:, None] * inv[None, :]
    z = torch.complex(x[..., : hd // 2].double(), x[..., hd // 2:].double()) * torch.polar(torch.ones_like(ang), ang)
    return torch.cat([z.real, z.imag], dim=-1).float()


def test_mrope_with_equal_rows_is_plain_rope():
    torch.manual_seed(1)
    hd, t = 16, 9
    q, k = torch.randn(3, t, hd), torch.randn(2, t, hd)
    pos = torch.tensor([0, 1, 2, 5, 9, 100, 1000, 4095, 7])
    cos, sin = plain_mrope_cos_sin(pos[None].expand(3, t), plain_inv_freq(hd, 10000.0))
    qr, kr = plain_apply_mrope(q, k, cos, sin, [2, 3, 3])
    assert torch.allclose(qr, _rotate_complex(q, pos, 10000.0), atol=2e-4)
    assert torch.allclose(kr, _rotate_complex(k, pos, 10000.0), atol=2e-4)
    assert torch.allclose(qr[:, 0], q[:, 0])                                   # position 0: identity
    assert torch.allclose(qr.norm(dim=-1), q.norm(dim=-1), atol=1e-5)          # a rotation


def test_mrope_scores_depend_on_distance_only():
    torch.manual_seed(2)
    hd = 24
    q, k = torch.randn(1, 1, hd), torch.randn(1, 1, hd)
    inv = plain_inv_freq(hd, 1e6)

    def score(pq, pk):
        cq = plain_mrope_cos_sin(torch.tensor([[pq]] * 3), inv)
        ck = plain_mrope_cos_sin(torch.tensor([[pk]] * 3), inv)
        a, _ = plain_apply_mrope(q, q, *cq, [4, 4, 4])
        _, b = plain_apply_mrope(k, k, *ck, [4, 4, 4])
        return (a * b).sum()

    assert torch.allclose(score(17, 5), score(112, 100), atol=1e-4)
    assert not torch.allclose(score(17, 5), score(17, 6), atol=1e-4)


def test_mrope_each_frequency_reads_its_own_row():
    """Sections [2, 3, 3] over half = 8: frequencies 0-1 read row t, 2-4 row h, 5-7 row w, and
    channel f + 8 follows channel f.  Doubling each entry instead of repeating the list
    ([2,2,3,3,3,3]) would fail this (reference rope.py:83-86)."""
    torch.manual_seed(3)
    hd = 16
    q = torch.randn(1, 1, hd)
    inv = plain_inv_freq(hd, 100.0)
    base = torch.tensor([[3], [3], [3]])
    ref, _ = plain_apply_mrope(q, q, *plain_mrope_cos_sin(base, inv), [2, 3, 3])
    owners = {0: [0, 1], 1: [2, 3, 4], 2: [5, 6, 7]}
    for row, freqs in owners.items():
        pos = base.clone()
        pos[row] = 11
        out, _ = plain_apply_mrope(q, q, *plain_mrope_cos_sin(pos, inv), [2, 3, 3])
        changed = ((out - ref).abs() > 1e-6)[0, 0]
        want = torch.zeros(hd, dtype=torch.bool)
        for f in freqs:
            want[f] = want[f + 8] = True
        assert torch.equal(changed, want), (row, changed)
    with pytest.raises(ValueError):
        plain_apply_mrope(q, q, *plain_mrope_cos_sin(base, inv), [2, 3, 4])    # reference rope.py:89-93


def test_attention_is_the_library_routine():
    torch.manual_seed(4)
    t, hd = 13, 8
    q, k, v = torch.randn(6, t, hd), torch.randn(2, t, hd), torch.randn(2, t, hd)
    got = plain_attention(q, k, v, hd ** -0.5)
    lib = F.scaled_dot_product_attention(q[None], k.repeat_interleave(3, 0)[None], v.repeat_interleave(3, 0)[None],
                                         is_causal=True)[0]
    assert torch.allclose(got, lib, atol=1e-5)
    # query head h reads key head h // groups
    alone = plain_attention(q[3:6], k[1:2], v[1:2], hd ** -0.5)
    assert torch.allclose(got[3:6], alone, atol=1e-6)
    assert torch.allclose(got[:, 0], v.repeat_interleave(3, 0)[:, 0], atol=1e-6)  # the first token sees itself only
    # one head, no mask effect on the last row: plain softmax(q k^T) v
    last = torch.softmax((q[0, -1] @ k[0].T) * hd ** -0.5, -1) @ v[0]
    assert torch.allclose(got[0, -1], last, atol=1e-5)
    # a sequence longer than the slice of queries the function takes at a time, with a window that
    # reaches across slices
    t = 1100
    q, k, v = torch.randn(2, t, hd), torch.randn(1, t, hd), torch.randn(1, t, hd)
    i, j = torch.arange(t)[:, None], torch.arange(t)[None, :]
    for window in (None, 90):
        mask = (j <= i) if window is None else (j <= i) & (i - j < window)
        lib = F.scaled_dot_product_attention(q[None], k.repeat_interleave(2, 0)[None], v.repeat_interleave(2, 0)[None],
                                             attn_mask=mask)[0]
        assert torch.allclose(plain_attention(q, k, v, hd ** -0.5, window), lib, atol=1e-5)


def test_window_edges():
    torch.manual_seed(5)
    t, hd = 11, 8
    q, k, v = torch.randn(2, t, hd), torch.randn(2, t, hd), torch.randn(2, t, hd)
    full = plain_attention(q, k, v, 1.0)
    assert torch.allclose(plain_attention(q, k, v, 1.0, window=t), full)          # window >= length: full
    assert torch.allclose(plain_attention(q, k, v, 1.0, window=1), v, atol=1e-6)  # window 1: own value
    w4 = plain_attention(q, k, v, 1.0, window=4)
    assert torch.allclose(w4[:, :4], full[:, :4], atol=1e-6)                      # the first 4 see everything
    # query 7 with window 4 sees keys 4..7 exactly
    want = torch.softmax(q[0, 7] @ k[0, 4:8].T, -1) @ v[0, 4:8]
    assert torch.allclose(w4[0, 7], want, atol=1e-6)
    # the reference's mask vector (tests/test_components.py:571-576): 2 queries after 3 cached keys;
    # query 0 sits at index 3 and sees keys 0..3, query 1 sees 0..4
    scores = torch.zeros(5, 5).masked_fill(~(torch.arange(5)[None] <= torch.arange(5)[:, None]), float("-inf"))
    assert scores[3, 3] == 0 and scores[3, 4] == float("-inf") and scores[4, 4] == 0


def test_swiglu():
    torch.manual_seed(6)
    x, g, u, d = torch.randn(4, 10), torch.randn(7, 10), torch.randn(7, 10), torch.randn(10, 7)
    assert torch.allclose(plain_mlp(x, g, u, d), (F.silu(x @ g.T) * (x @ u.T)) @ d.T, atol=1e-6)
    assert torch.equal(plain_mlp(torch.zeros(1, 10), g, u, d), torch.zeros(1, 10))  # silu(0) = 0, no biases


def test_layer_windows_rule():
    base = {"num_hidden_layers": 4, "sliding_window": 16}
    assert plain_layer_windows(dict(base, use_sliding_window=False)) == [None] * 4
    assert plain_layer_windows(dict(base, use_sliding_window=True, max_window_layers=1)) == [None, 16, 16, 16]
    assert plain_layer_windows(dict(base, use_sliding_window=True)) == [None] * 4
    assert plain_layer_windows(dict(base, layer_types=["sliding_attention", "full_attention"] * 2)) == [16, None] * 2


def test_whole_model_invariants(model_dirs):
    for name, vocab in (("A", 256), ("B", 509)):
        d = model_dirs[name]
        cfg, w = plain_read_config(d), plain_read_weights(d)
        ids = torch.randint(0, vocab, (23,), generator=torch.Generator().manual_seed(1)).tolist()
        logits = plain_forward(cfg, w, ids)
        assert logits.shape == (23, vocab)
        # causal: a prefix's logits do not depend on what follows
        assert torch.allclose(plain_forward(cfg, w, ids[:10]), logits[:10], atol=1e-5)
        # only distances count: shifting every position changes nothing
        shifted = (torch.arange(23) + 50)[None].expand(3, 23)
        assert torch.allclose(plain_forward(cfg, w, ids, shifted), logits, atol=2e-4)
        # but the rows matter: a different h row changes the result
        rows = torch.arange(23)[None].repeat(3, 1)
        rows[1, 5:] += 3
        assert not torch.allclose(plain_forward(cfg, w, ids, rows), logits, atol=1e-4)
    # the window matters in B: without it the late logits differ
    cfg_full = dict(cfg, use_sliding_window=False, layer_types=None)
    assert not torch.allclose(plain_forward(cfg_full, w, ids), logits, atol=1e-5)
    assert torch.allclose(plain_forward(cfg_full, w, ids)[:16], logits[:16], atol=1e-5)
    # tied head in A, stored head in B
    assert "lm_head.weight" not in plain_read_weights(model_dirs["A"]) and "lm_head.weight" in w


def test_sampling_formulas():
    # reference tests/test_components.py:590-626, 716-732
    logits = torch.tensor([4.0, 3.0, 2.0, 1.0, 0.0])
    probs = plain_filtered_probs(logits, 1.0, top_p=0.5)
    assert (probs > 0).tolist() == [True, False, False, False, False]          # 0.636 alone reaches 0.5
    probs = plain_filtered_probs(logits, 1.0, top_p=0.7)
    assert (probs > 0).tolist() == [True, True, False, False, False]           # the crossing token stays
    assert (plain_filtered_probs(logits, 1.0, top_k=1) > 0).tolist() == [True] + [False] * 4
    assert (plain_filtered_probs(logits, 1.0, top_k=3) > 0).sum() == 3
    assert (plain_filtered_probs(logits, 1.0, min_p=0.2) > 0).tolist() == [True, True, False, False, False]
    assert torch.allclose(plain_filtered_probs(logits, 2.0), torch.softmax(logits / 2, -1))
    out = plain_penalties(torch.zeros(3), [0, 0, 1], presence=1.0, frequency=0.5)
    assert out.tolist() == [-2.0, -1.5, 0.0]
    out = plain_penalties(torch.tensor([1.0, -1.0, 1.0]), [0, 1], repetition=2.0)
    assert out.tolist() == [0.5, -2.0, 1.0]
