"""Each HIP kernel alone against a plain float32 formula, at sizes other than the engine's."""

import math

import pytest
import torch

from plain_model import (plain_apply_mrope, plain_attention, plain_inv_freq, plain_mrope_cos_sin, plain_rmsnorm)

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype):
    return dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed_gather(dtype):
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(0)
    table = torch.randn(301, 100).to(dtype).cuda()
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32).cuda()
    out = kernels.embed_gather(ids, table)
    assert out.dtype == torch.float32 and torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("width", [97, 3584, 8200])
@pytest.mark.parametrize("delta_dtype, out_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                                    (torch.bfloat16, torch.bfloat16), (None, torch.bfloat16)])
def test_add_rmsnorm(width, delta_dtype, out_dtype):
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(width)
    n, eps = 5, 1e-5
    h = torch.randn(n, width) * 3
    delta = torch.randn(n, width).to(delta_dtype) if delta_dtype is not None else None
    w = 1 + 0.1 * torch.randn(width)
    total = h + (delta.float() if delta is not None else 0)
    want = plain_rmsnorm(total, w, eps)
    hd = h.cuda()
    out = kernels.add_rmsnorm(hd, None if delta is None else delta.cuda(), w.cuda(), eps, out_dtype)
    assert out.dtype == out_dtype
    assert torch.allclose(out.float().cpu(), want, **_tol(out_dtype))
    assert torch.allclose(hd.cpu(), total, atol=1e-6), "the sum is written back in float32"
    # selected rows: h stays as it was
    hd = h.cuda()
    rows = torch.tensor([4, 0, 4], dtype=torch.int32).cuda()
    out = kernels.add_rmsnorm(hd, None if delta is None else delta.cuda(), w.cuda(), eps, out_dtype, rows=rows)
    assert torch.allclose(out.float().cpu(), want[[4, 0, 4]], **_tol(out_dtype)) and torch.equal(hd.cpu(), h)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, nkv, hd, sections, ps", [(6, 2, 24, (4, 4, 4), 16), (5, 1, 48, (10, 6, 8), 16),
                                                       (4, 4, 128, (16, 24, 24), 16), (6, 2, 24, (4, 4, 4), 48),
                                                       (4, 4, 128, (16, 24, 24), 32)])
def test_rope_kv_write(dtype, nq, nkv, hd, sections, ps):
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(hd)
    n, pages, theta = 11, 5, 1e4
    x = torch.randn(n, (nq + 2 * nkv) * hd)
    bias = torch.randn((nq + 2 * nkv) * hd) * 0.1
    pos = torch.stack([torch.randint(0, 5000, (n,)) for _ in range(3)])
    slots = torch.randperm(pages * ps)[:n].to(torch.int32)
    inv = plain_inv_freq(hd, theta)
    rows = torch.tensor(sum(([r] * c for r, c in enumerate(sections)), []), dtype=torch.int32)
    kc = torch.zeros(pages, nkv, ps, hd, dtype=dtype).cuda()
    vc = torch.zeros(pages, nkv, hd, ps, dtype=dtype).cuda()
    q = kernels.rope_kv_write(x.cuda(), bias.cuda(), pos.to(torch.int32).cuda(), inv.cuda(), rows.cuda(), slots.cuda(),
                              kc, vc, nq, nkv, hd, ps, out_dtype=dtype)
    xb = x + bias
    qs, ks, vs = xb.split([nq * hd, nkv * hd, nkv * hd], dim=1)
    cos, sin = plain_mrope_cos_sin(pos, inv)
    qr, kr = plain_apply_mrope(qs.view(n, nq, hd).transpose(0, 1), ks.view(n, nkv, hd).transpose(0, 1), cos, sin, sections)
    tol = dict(atol=2e-4, rtol=1e-4) if dtype == torch.float32 else _tol(dtype)   # sin/cos of angles up to 5000
    assert torch.allclose(q.float().cpu().view(n, nq, hd), qr.transpose(0, 1), **tol)
    kflat = kc.float().cpu().permute(0, 2, 1, 3).reshape(pages * ps, nkv, hd)          # [slot, kv head, hd]
    vflat = vc.float().cpu().permute(0, 3, 1, 2).reshape(pages * ps, nkv, hd)
    assert torch.allclose(kflat[slots.long()], kr.transpose(0, 1), **tol)
    assert torch.allclose(vflat[slots.long()], vs.view(n, nkv, hd), **_tol(dtype))
    untouched = torch.ones(pages * ps, dtype=torch.bool)
    untouched[slots.long()] = False
    assert kflat[untouched].abs().max() == 0 and vflat[untouched].abs().max() == 0
    # with the step's table of cosines and sines in hand the kernel gives the very same values
    cs = kernels.rope_table(pos.to(torch.int32).cuda(), inv.cuda(), rows.cuda(), n)
    want_cs = torch.stack([torch.cos(pos[rows.long()].T.float() * inv), torch.sin(pos[rows.long()].T.float() * inv)], dim=-1)
    assert torch.allclose(cs.cpu(), want_cs, atol=2e-4)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2 = kernels.rope_kv_write(x.cuda(), bias.cuda(), pos.to(torch.int32).cuda(), inv.cuda(), rows.cuda(), slots.cuda(),
                               kc2, vc2, nq, nkv, hd, ps, out_dtype=dtype, cs=cs)
    if dtype == torch.float32:
        assert torch.equal(q2, q) and torch.equal(kc2, kc) and torch.equal(vc2, vc)
    else:   # float32 sums to bfloat16 with the table: the kernel with 16-byte loads
        for a, b in ((q2, q), (kc2, kc), (vc2, vc)):
            assert torch.allclose(a.float(), b.float(), atol=2e-2, rtol=1e-2)
        assert torch.equal(vc2, vc)
    # position 0 leaves a head as it is; a negative slot writes nothing; rot < hd leaves the tail alone
    kc.zero_()
    q0 = kernels.rope_kv_write(x.cuda(), None, torch.zeros(3, n, dtype=torch.int32).cuda(), inv.cuda(), rows.cuda(),
                               torch.full((n,), -1, dtype=torch.int32).cuda(), kc, vc, nq, nkv, hd, ps, out_dtype=dtype)
    assert torch.allclose(q0.float().cpu(), x[:, :nq * hd].to(dtype).float(), atol=1e-6) and kc.abs().max() == 0
    half = hd // 4
    qp = kernels.rope_kv_write(x[:, :nq * hd].contiguous().cuda(), None, pos.to(torch.int32).cuda(),
                               plain_inv_freq(2 * half, theta).cuda(), torch.zeros(half, dtype=torch.int32).cuda(),
                               None, None, None, nq, 0, hd, ps, out_dtype=dtype)
    qp = qp.float().cpu().view(n, nq, hd)
    assert torch.allclose(qp[..., 2 * half:], x[:, :nq * hd].view(n, nq, hd)[..., 2 * half:].to(dtype).float(), atol=1e-6)
    c1, s1 = plain_mrope_cos_sin(pos[:1].expand(3, n), plain_inv_freq(2 * half, theta))
    want, _ = plain_apply_mrope(x[:, :nq * hd].view(n, nq, hd)[..., :2 * half].transpose(0, 1),
                                x[:, :nq * hd].view(n, nq, hd)[..., :2 * half].transpose(0, 1), c1, s1, (half, 0, 0))
    assert torch.allclose(qp[..., :2 * half], want.transpose(0, 1), **tol)


def test_rope_kv_write_from_slabs():
    """The projection as slabs of partial sums: the rotation's kernel adds them in order and gives
    what it gives for their sum."""
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(3)
    n, nq, nkv, hd, ps, pages = 40, 6, 2, 48, 16, 9
    cols = (nq + 2 * nkv) * hd
    slabs = torch.randn(3, n, cols).cuda()
    total = slabs[0] + slabs[1]
    total = total + slabs[2]
    bias = torch.randn(cols).cuda()
    pos = torch.randint(0, 500, (3, n), dtype=torch.int32).cuda()
    inv_freq = plain_inv_freq(hd, 10000.0).cuda()
    freq_row = torch.tensor([0] * 8 + [1] * 8 + [2] * 8, dtype=torch.int32).cuda()
    slots = torch.randperm(pages * ps)[:n].to(torch.int32).cuda()
    cs = kernels.rope_table(pos, inv_freq, freq_row, n)
    outs = []
    for x in (slabs, total):
        kc = torch.zeros(pages, nkv, ps, hd, dtype=torch.bfloat16).cuda()
        vc = torch.zeros(pages, nkv, hd, ps, dtype=torch.bfloat16).cuda()
        q = kernels.rope_kv_write(x, bias, pos, inv_freq, freq_row, slots, kc, vc, nq, nkv, hd, ps,
                                  out_dtype=torch.bfloat16, cs=cs)
        outs.append((q, kc, vc))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert outs[0][0].abs().sum() > 0 and outs[0][1].abs().sum() > 0
    with pytest.raises(kernels.KernelError):      # slabs are taken with the table in hand only
        kernels.rope_kv_write(slabs, bias, pos, inv_freq, freq_row, slots, outs[0][1], outs[0][2], nq, nkv, hd, ps,
                              out_dtype=torch.bfloat16)


def _paged(k, v, ps, pages, dtype, seed):
    """Scatter per-request keys/values [nkv, T, hd] into shuffled pages; returns caches and tables."""
    g = torch.Generator().manual_seed(seed)
    nkv, hd = k[0].shape[0], k[0].shape[2]
    kc = torch.randn(pages, nkv, ps, hd, generator=g).to(dtype)          # stale values everywhere
    vc = torch.randn(pages, nkv, hd, ps, generator=g).to(dtype)
    order = torch.randperm(pages, generator=g).tolist()
    width = max((x.shape[1] + ps - 1) // ps for x in k)
    table = torch.full((len(k), width), -1, dtype=torch.int32)
    for r, (kr, vr) in enumerate(zip(k, v)):
        for i in range((kr.shape[1] + ps - 1) // ps):
            page = order.pop()
            table[r, i] = page
            n = min(ps, kr.shape[1] - i * ps)
            kc[page, :, :n] = kr[:, i * ps:i * ps + n].to(dtype)
            vc[page, :, :, :n] = vr[:, i * ps:i * ps + n].transpose(1, 2).to(dtype)
    return kc, vc, table


# the last shape has more query heads to a key/value head (20) than a column tile has columns: a
# token's heads span two tiles
ATTN_SHAPES = [(6, 2, 24, None), (5, 1, 48, 40), (8, 8, 16, 7), (14, 2, 128, None), (4, 2, 80, 130), (40, 2, 64, None)]


def _attention_case(dtype, nq, nkv, hd, window, lens=(333, 17, 64, 1), qlens=(5, 17, 1, 1), ps=16):
    """Prompt portions and single tokens of several requests in one call, pages shuffled, stale
    values in every unused slot.  One query and one far key are scaled so that a single score
    dominates: a kernel that misses that key (a page, a window edge) fails by far."""
    torch.manual_seed(nq * hd)
    lens, qlens = list(lens), list(qlens)   # context of each request after this step; its last qlen tokens are this step's
    last = lens[0] - 1
    k = [torch.randn(nkv, t, hd).to(dtype).float() for t in lens]
    v = [torch.randn(nkv, t, hd).to(dtype).float() for t in lens]
    q_all = [torch.randn(nq, t, hd) for t in lens]
    far = 2 if window is None else max(0, last - window + 1)      # the first key the last query still sees
    kf = k[0][:, far].repeat_interleave(nq // nkv, 0)
    q_all[0][:, last] = kf * (30.0 / (kf.pow(2).sum(-1, keepdim=True) * hd ** -0.5))      # that score is 30
    q_all = [x.to(dtype).float() for x in q_all]
    scale = hd ** -0.5
    kc, vc, table = _paged(k, v, ps, sum((t + ps - 1) // ps for t in lens) + 11, dtype, 1)
    qs, req, seqpos, want = [], [], [], []
    for r, (t, ql) in enumerate(zip(lens, qlens)):
        full = plain_attention(q_all[r], k[r], v[r], scale, window)      # [nq, t, hd]
        for p in range(t - ql, t):
            qs.append(q_all[r][:, p].reshape(-1))
            req.append(r)
            seqpos.append(p)
            want.append(full[:, p].reshape(-1))
    want = torch.stack(want)
    # the dominated row (request 0, its last position) really is the far key's value
    assert torch.allclose(want[qlens[0] - 1].view(nq, hd), v[0][:, far].repeat_interleave(nq // nkv, 0), atol=1e-3)
    return dict(q=torch.stack(qs).to(dtype).cuda(), kc=kc.cuda(), vc=vc.cuda(), table=table.cuda(),
                req=torch.tensor(req, dtype=torch.int32).cuda(), seqpos=torch.tensor(seqpos, dtype=torch.int32).cuda(),
                want=want, scale=scale, lens=lens, qlens=qlens)


# other page sizes than 16 (the reference tests 32, reference tests/test_paged_attn_kernel.py:89);
# 48 is the one where a 32-key block straddles pages at changing places
PAGE_SIZES = [(14, 2, 128, None, 32), (5, 1, 48, 40, 48), (4, 2, 80, 130, 64), (6, 2, 24, None, 32), (14, 2, 128, 70, 48),
              (7, 1, 128, None, 64)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq, nkv, hd, window, ps", [(*s, 16) for s in ATTN_SHAPES] + PAGE_SIZES)
def test_paged_attention_generic(dtype, nq, nkv, hd, window, ps):
    from qwen25vl_lite_amd.ops import kernels
    c = _attention_case(dtype, nq, nkv, hd, window, ps=ps)
    out = kernels.paged_attention_generic(c["q"], c["kc"], c["vc"], c["table"], c["req"], c["seqpos"], nq, window,
                                          c["scale"])
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=1.5e-2, rtol=2e-2)
    assert torch.allclose(out.float().cpu(), c["want"], **tol), (out.float().cpu() - c["want"]).abs().max()


@pytest.mark.parametrize("split", ["tile", "tile_two_groups", "coop", "coop_split", "coop_split_two_kernels"])
@pytest.mark.parametrize("nq, nkv, hd, window, ps", [(*s, 16) for s in ATTN_SHAPES if s[2] % 16 == 0]
                         + [s for s in PAGE_SIZES if s[2] % 16 == 0])
def test_paged_attention_matrix_cores(nq, nkv, hd, window, ps, split, monkeypatch):
    """The matrix-core kernels on the same case: blocks that own several tiles and share the keys
    through LDS (one group of waves, or two that take the key blocks in turn and merge), the waves
    of a block sharing one tile, and the keys further split among blocks, whose partial results the
    last block to finish merges (or a second kernel, for callers without counters)."""
    from qwen25vl_lite_amd.ops import attention_mfma
    from qwen25vl_lite_amd.parts import StepContext
    c = _attention_case(torch.bfloat16, nq, nkv, hd, window, ps=ps)
    plan = {"tile": ("tile", 1, 0), "tile_two_groups": ("tile", 1, 0), "coop": ("coop", 1, 0),
            "coop_split": ("coop", 6, 64), "coop_split_two_kernels": ("coop", 6, 64)}[split]
    if split == "coop_split_two_kernels":
        monkeypatch.setattr(attention_mfma, "MERGE_COUNTERS", 0)
    groups = {"tile": 1, "tile_two_groups": 2}.get(split)
    if groups == 2 and hd > 128:
        pytest.skip("two groups of waves are built for head sizes up to 128")
    monkeypatch.setattr(attention_mfma, "plan_splits", lambda t, n, m, d=None: plan)
    cu = [0]
    for ql in c["qlens"]:
        cu.append(cu[-1] + ql)
    none = torch.zeros(0, dtype=torch.int32).cuda()
    step = StepContext(num_tokens=cu[-1], num_reqs=4, token_ids=none, positions=none, token_req=c["req"],
                       token_seqpos=c["seqpos"], cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
                       ctx_len=torch.tensor(c["lens"], dtype=torch.int32).cuda(), req_slots=none, groups=[],
                       logit_rows=none, cu_q_host=cu, ctx_len_host=c["lens"], max_q_len=17, max_ctx_len=333,
                       dtype=torch.bfloat16)
    out = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"],
                                       force_groups=groups)
    assert out is not None
    err = (out.float().cpu() - c["want"]).abs().max()
    assert torch.allclose(out.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2), err
    if split == "coop_split":
        # the counters are back at zero, and a second launch right behind the first finds them so
        again = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"])
        assert torch.equal(again, out)
        torch.cuda.synchronize()
        assert int(attention_mfma._counters(c["q"].device).abs().sum()) == 0


@pytest.mark.parametrize("split", ["coop", "coop_split", "coop_split_two_kernels"])
@pytest.mark.parametrize("nq, nkv, hd, window", [(14, 2, 128, None), (6, 2, 48, 100), (8, 8, 16, 7)])
def test_a_step_of_decoded_tokens_only(nq, nkv, hd, window, split, monkeypatch):
    """Every request brings one token: the kernel is not handed the lists of tiles and of run
    starts (tile i is request i's, its token is token i) and gives what it gives with them."""
    from qwen25vl_lite_amd.ops import attention_mfma
    from qwen25vl_lite_amd.parts import StepContext
    lens = (333, 17, 64, 1, 200)
    c = _attention_case(torch.bfloat16, nq, nkv, hd, window, lens, (1,) * len(lens))
    plan = ("coop", 1, 0) if split == "coop" else ("coop", 6, 64)
    if split == "coop_split_two_kernels":
        monkeypatch.setattr(attention_mfma, "MERGE_COUNTERS", 0)
    monkeypatch.setattr(attention_mfma, "plan_splits", lambda t, n, m, d=None: plan)
    cu = list(range(len(lens) + 1))
    none = torch.zeros(0, dtype=torch.int32).cuda()
    step = StepContext(num_tokens=len(lens), num_reqs=len(lens), token_ids=none, positions=none, token_req=c["req"],
                       token_seqpos=c["seqpos"], cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
                       ctx_len=torch.tensor(lens, dtype=torch.int32).cuda(), req_slots=none, groups=[],
                       logit_rows=none, cu_q_host=cu, ctx_len_host=list(lens), max_q_len=1, max_ctx_len=max(lens),
                       dtype=torch.bfloat16)
    handed = []
    real = attention_mfma._fn

    def spy(stem, name, *a, **k):
        fn = real(stem, name, *a, **k)
        if not name.startswith("qvl_attn_mfma_coop"):
            return fn
        return lambda *args: (handed.append((args[5], args[7], args[8])), fn(*args))[1]   # cu_q, tile_req, tile_ct

    monkeypatch.setattr(attention_mfma, "_fn", spy)
    out = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"])
    assert handed == [(None, None, None)]
    assert torch.allclose(out.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2), (out.float().cpu() - c["want"]).abs().max()
    # the same step declared as one that might hold portions: the lists are handed over, the result is the same bits
    step.max_q_len = 2
    handed.clear()
    with_lists = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"])
    assert handed and handed[0][0] is not None and torch.equal(with_lists, out)


@pytest.mark.parametrize("nq, nkv, hd, window", [(14, 2, 128, None), (6, 2, 48, 100)])
def test_mixed_step_with_few_long_decoded_tokens(nq, nkv, hd, window, monkeypatch):
    """A prompt portion beside two decoded tokens whose contexts are long: the decoded tokens go to
    the kernel that splits a context among blocks, in a launch of their own, the portion to the
    kernel for many tiles; both write into the same output.  (The limits are set low here so that
    contexts of a few hundred keys count as long.)"""
    from qwen25vl_lite_amd.ops import attention_mfma, kernels
    from qwen25vl_lite_amd.parts import StepContext
    lens, qlens = (333, 300, 17, 280), (40, 1, 17, 1)
    c = _attention_case(torch.bfloat16, nq, nkv, hd, window, lens, qlens)
    monkeypatch.setattr(attention_mfma, "TARGET_BLOCKS", 8)    # the two decoded tokens make 4 blocks, the portions 24 or more
    monkeypatch.setattr(attention_mfma, "MIN_KEYS_PER_SPLIT", 64)
    monkeypatch.setattr(attention_mfma, "SPLIT_FROM_KEYS", 64)
    monkeypatch.setattr(attention_mfma, "ALONE_KEYS", 128)
    cu = [0]
    for ql in qlens:
        cu.append(cu[-1] + ql)
    none = torch.zeros(0, dtype=torch.int32).cuda()
    step = StepContext(num_tokens=cu[-1], num_reqs=len(lens), token_ids=none, positions=none, token_req=c["req"],
                       token_seqpos=c["seqpos"], cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
                       ctx_len=torch.tensor(lens, dtype=torch.int32).cuda(), req_slots=none, groups=[],
                       logit_rows=none, cu_q_host=cu, ctx_len_host=list(lens), max_q_len=max(qlens),
                       max_ctx_len=max(lens), dtype=torch.bfloat16)
    assert attention_mfma.long_single_tiles(step, nq // nkv, nkv) == (0, 1, 0, 1)
    called = []
    real = attention_mfma._fn
    monkeypatch.setattr(attention_mfma, "_fn", lambda stem, name, *a, **k: (called.append(name), real(stem, name, *a, **k))[1])
    out = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"])
    assert "qvl_attn_mfma_coop_merged" in called and "qvl_attn_mfma_block" in called
    err = (out.float().cpu() - c["want"]).abs().max()
    assert torch.allclose(out.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2), err


@pytest.mark.parametrize("nq, nkv, hd, window, ps", [(28, 4, 128, None, 16), (6, 2, 48, 100, 16), (4, 4, 256, 257, 16),
                                                     (5, 1, 16, None, 16), (28, 4, 128, None, 48), (6, 2, 48, 100, 32),
                                                     (4, 4, 256, 257, 64), (4, 2, 32, None, 16), (8, 2, 64, 70, 32),
                                                     (3, 1, 96, None, 16), (6, 3, 112, 200, 48)])
def test_paged_attention_long_portions(nq, nkv, hd, window, ps):
    """Prompt portions long enough for several blocks of several waves per request, next to a
    short portion and a decoded token: the kernel that shares keys through LDS walks the union of
    its waves' ranges, with blocks that some of its waves skip.  Every head size in steps of 16 up to
    128 lays its stages out differently (loads per part, the second half's offset): all of them run."""
    from qwen25vl_lite_amd.ops import attention_mfma, kernels
    from qwen25vl_lite_amd.parts import StepContext
    lens, qlens = (413, 150, 90), (380, 3, 1)
    c = _attention_case(torch.bfloat16, nq, nkv, hd, window, lens, qlens, ps=ps)
    cu = [0]
    for ql in qlens:
        cu.append(cu[-1] + ql)
    none = torch.zeros(0, dtype=torch.int32).cuda()
    step = StepContext(num_tokens=cu[-1], num_reqs=len(lens), token_ids=none, positions=none, token_req=c["req"],
                       token_seqpos=c["seqpos"], cu_q=torch.tensor(cu, dtype=torch.int32).cuda(),
                       ctx_len=torch.tensor(lens, dtype=torch.int32).cuda(), req_slots=none, groups=[],
                       logit_rows=none, cu_q_host=cu, ctx_len_host=list(lens), max_q_len=max(qlens),
                       max_ctx_len=max(lens), dtype=torch.bfloat16)
    import unittest.mock as mock
    for groups in (1, 2) if hd <= 128 else (1,):   # an odd and an even number of key blocks among the walks
        with mock.patch.object(attention_mfma, "plan_splits", lambda t, n, m, d=None: ("tile", 1, 0)):
            out = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"],
                                               force_groups=groups, force_wide=False)
        err = (out.float().cpu() - c["want"]).abs().max()
        assert torch.allclose(out.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2), (groups, err)
    if hd in (128, 48):   # the kind whose waves carry three column tiles (its operands pass through a few registers)
        with mock.patch.object(attention_mfma, "plan_splits", lambda t, n, m, d=None: ("tile", 1, 0)):
            out = attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"],
                                               force_groups=1, force_wide=True)
        err = (out.float().cpu() - c["want"]).abs().max()
        assert torch.allclose(out.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2), ("wide", err)
        assert attention_mfma.block_tiles(hd, True) == 12 and attention_mfma.block_tiles(hd) == 8
    # every launch leaves the work-queue counters at zero for the next one
    torch.cuda.synchronize()
    assert int(attention_mfma._work_queue(c["q"].device)[0].abs().sum()) == 0
    assert attention_mfma.block_groups(10, 512, hd) == (2 if hd <= 128 else 1)
    assert attention_mfma.block_groups(513, 512, hd) == 1
    with mock.patch.object(attention_mfma, "plan_splits", lambda t, n, m, d=None: ("tile", 1, 0)), pytest.raises(kernels.KernelError):
        attention_mfma.try_attention(c["q"], c["kc"], c["vc"], c["table"], step, nq, window, c["scale"], force_groups=3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows, inter", [(7, 353), (5, 352), (70, 18944)])
def test_swiglu(dtype, rows, inter):
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(3)
    x = (torch.randn(rows, 2 * inter) * 3).to(dtype)
    want = torch.nn.functional.silu(x[:, :inter].float()) * x[:, inter:].float()
    out = kernels.swiglu(x.cuda())
    assert torch.allclose(out.float().cpu(), want, **_tol(dtype))
    if inter % 8 == 0:   # the same values with gate and up columns in alternating groups of 8
        g = torch.stack([x[:, :inter].reshape(rows, -1, 8), x[:, inter:].reshape(rows, -1, 8)], dim=2)
        out = kernels.swiglu(g.reshape(rows, 2 * inter).contiguous().cuda(), grouped=True)
        assert torch.allclose(out.float().cpu(), want, **_tol(dtype))


@pytest.mark.parametrize("m, n, k", [(1, 5, 3), (7, 509, 144), (65, 130, 353), (130, 64, 1000)])
def test_gemm_f32_is_exact_and_row_independent(m, n, k):
    from qwen25vl_lite_amd.ops import kernels
    torch.manual_seed(m)
    x, w, b = torch.randn(m, k), torch.randn(n, k), torch.randn(n)
    want = (x.double() @ w.double().T + b.double()).float()
    out = kernels.gemm_f32(x.cuda(), w.cuda(), b.cuda())
    assert torch.allclose(out.cpu(), want, atol=1e-4 * math.sqrt(k), rtol=1e-5)
    # no reduced-precision input format: products of values that bfloat16/tf32 would round
    xe = torch.full((1, 4), 1 + 2 ** -20)
    we = torch.tensor([[1.0, -1.0, 1.0, -1.0 + 2 ** -19]])
    assert kernels.gemm_f32(xe.cuda(), we.cuda()).item() == pytest.approx((xe.double() @ we.double().T).item(), abs=1e-12)
    # a row's result does not depend on what else is in the batch
    alone = kernels.gemm_f32(x[m // 2:m // 2 + 1].contiguous().cuda(), w.cuda(), b.cuda())
    assert torch.equal(alone[0], out[m // 2])


@pytest.mark.parametrize("m, n, k", [(1, 509, 144), (8, 300, 200), (16, 17, 8), (9, 100, 8200), (17, 1000, 4104),
                                     (31, 130, 352), (64, 509, 3584), (5, 40, 100), (300, 64, 1000),
                                     (17, 4700, 3584), (32, 300, 3840), (24, 509, 3848), (20, 33, 8),
                                     (30, 4104, 4000), (16, 4104, 4104), (33, 300, 200), (64, 4700, 3584),
                                     (48, 509, 3848), (41, 130, 8200), (64, 3584, 18944), (65, 300, 200)])
def test_linear_bfloat16(m, n, k):
    """Up to 64 rows go through the resident matrix-core kernel (inner sizes in steps of 8): up to 32
    rows always if the inner size fits one pass of a block (4096, or 3840 with 17 to 32 rows), and
    with a longer one while each compute unit has one tile at most; 33 to 64 rows if it fits one pass
    (teams of blocks); the rest through the library; all accumulate in float32."""
    from qwen25vl_lite_amd.ops import skinny
    from qwen25vl_lite_amd.ops.linear import linear
    torch.manual_seed(k)
    x, w = torch.randn(m, k).bfloat16(), (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    b = torch.randn(n)
    want = x.float() @ w.float().T
    units = torch.cuda.get_device_properties(0).multi_processor_count
    assert skinny.takes_resident(m, k, w.cuda()) == (
        k % 8 == 0 and m <= 64 and (k <= 4096 if m > 32 else (k <= (4096 if m <= 16 else 3840) or n <= 16 * units)))
    out32 = linear(x.cuda(), w.cuda(), out_dtype=torch.float32)
    assert out32.dtype == torch.float32 and torch.allclose(out32.cpu(), want, atol=2e-3, rtol=2e-3)
    out16 = linear(x.cuda(), w.cuda())
    assert out16.dtype == torch.bfloat16 and torch.allclose(out16.float().cpu(), want, atol=2e-2, rtol=2e-2)
    outb = linear(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32)
    assert torch.allclose(outb.cpu(), want + b, atol=2e-3, rtol=2e-3)
    # a row's result does not depend on the rows beside it
    if m > 1:
        alone = linear(x[m // 2:m // 2 + 1].contiguous().cuda(), w.cuda(), out_dtype=torch.float32)
        assert torch.allclose(alone[0], out32[m // 2], atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("m, n, k", [(1, 48, 64), (7, 1000, 3584), (16, 130, 4096), (3, 64, 144),
                                     (17, 1000, 3584), (32, 130, 3840), (29, 64, 144), (24, 48, 4096),
                                     (33, 1000, 3584), (64, 64, 144)])
def test_product_with_the_norm_folded_in(m, n, k):
    """rmsnorm(h) * w formed inside the product equals the norm kernel followed by the product."""
    from qwen25vl_lite_amd.ops import kernels
    from qwen25vl_lite_amd.ops.linear import NormedRows, linear
    torch.manual_seed(n)
    h = (torch.randn(m, k) * 2).cuda()
    g = (1 + 0.1 * torch.randn(k)).cuda()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16().cuda()
    fused = linear(NormedRows(h, g, 1e-5, torch.bfloat16), w, out_dtype=torch.float32)
    apart = linear(kernels.add_rmsnorm(h, None, g, 1e-5, torch.bfloat16), w, out_dtype=torch.float32)
    want = plain_rmsnorm(h.cpu(), g.cpu(), 1e-5).bfloat16().float() @ w.float().cpu().T
    assert torch.allclose(fused.cpu(), want, atol=3e-3, rtol=3e-3)
    assert (fused - apart).abs().max() < 0.02 * want.abs().max()   # the same up to a bfloat16 rounding of x here and there
    if m > 32:   # teams of blocks: `linear` leaves these to the library, the kernel itself takes them
        from qwen25vl_lite_amd.ops import skinny
        assert skinny.folds_norm(m, k)
        team = skinny.resident_product(w, h=h, norm_weight=g, eps=1e-5, out_dtype=torch.float32)
        assert torch.allclose(team.cpu(), want, atol=3e-3, rtol=3e-3)
        both = skinny.resident_product(w, x=kernels.add_rmsnorm(h, None, g, 1e-5, torch.bfloat16), out_dtype=torch.float32)
        assert torch.allclose(both.cpu(), want, atol=3e-3, rtol=3e-3)
    # a longer row than one pass of the block holds is computed by the norm's own kernel first
    h2, g2 = torch.randn(2, 4104).cuda(), torch.ones(4104).cuda()
    w2 = (torch.randn(24, 4104) / 64).bfloat16().cuda()
    out = linear(NormedRows(h2, g2, 1e-6, torch.bfloat16), w2, out_dtype=torch.float32)
    assert torch.allclose(out.cpu(), plain_rmsnorm(h2.cpu(), g2.cpu(), 1e-6).bfloat16().float() @ w2.float().cpu().T,
                          atol=3e-3, rtol=3e-3)


@pytest.mark.parametrize("m, n, k", [(1, 144, 352), (8, 3584, 18944), (16, 100, 4104), (24, 144, 352), (40, 144, 352),
                                     (32, 3584, 3584), (17, 100, 3840), (24, 144, 4104), (32, 3584, 18944),
                                     (64, 3584, 18944), (33, 3584, 3584), (57, 100, 4104), (70, 144, 352)])
def test_product_added_into_the_residual(m, n, k):
    from qwen25vl_lite_amd.ops.linear import linear_into
    torch.manual_seed(k)
    x = torch.randn(m, k).bfloat16().cuda()
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16().cuda()
    h = torch.randn(m, n).cuda()
    want = h.cpu() + x.float().cpu() @ w.float().cpu().T
    left = linear_into(h, x, w)
    if m <= 16 and k <= 4096:      # one block carries the rows for the whole inner size: added in place
        assert left is None and torch.allclose(h.cpu(), want, atol=3e-3, rtol=3e-3)
    elif m <= 64:   # the split kernel: slabs of partial sums for the next norm to add
        assert left.dtype == torch.float32 and left.dim() == 3 and tuple(left.shape[1:]) == (m, n)
        assert torch.allclose(h.cpu() + left.sum(0).cpu(), want, atol=3e-3, rtol=3e-3)
    else:   # the library's product comes back in bfloat16 for the next norm to add
        assert left is not None and left.dtype == torch.bfloat16 and left.dim() == 2
        assert torch.allclose(h.cpu() + left.float().cpu(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m, inter, k", [(1, 352, 144), (8, 18944, 3584), (16, 40, 4104), (50, 352, 144),
                                         (4, 2072, 64), (3, 5136, 72), (2, 8 * 320, 40),
                                         (32, 18944, 3584), (17, 2072, 64), (25, 5136, 72), (64, 18944, 3584),
                                         (33, 2072, 64), (47, 5136, 72), (70, 352, 144)])
def test_gate_up_product_with_the_activation_folded_in(dtype, m, inter, k):
    """Grouped gate | up rows: few bfloat16 rows get silu(gate) * up from the product's own kernel,
    everything else from the product followed by the activation kernel on the grouped columns."""
    from qwen25vl_lite_amd.ops.linear import gate_up_swiglu
    torch.manual_seed(inter)
    x = torch.randn(m, k).to(dtype)
    gate = (torch.randn(inter, k) / math.sqrt(k)).to(dtype)
    up = (torch.randn(inter, k) / math.sqrt(k)).to(dtype)
    grouped = torch.stack([gate.view(-1, 8, k), up.view(-1, 8, k)], dim=1).reshape(2 * inter, k).contiguous()
    out = gate_up_swiglu(x.cuda(), grouped.cuda(), True)
    want = torch.nn.functional.silu(x.float() @ gate.float().T) * (x.float() @ up.float().T)
    assert out.shape == (m, inter) and out.dtype == dtype
    tol = dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    assert torch.allclose(out.float().cpu(), want, **tol)
    plain = gate_up_swiglu(x.cuda(), torch.cat([gate, up]).cuda(), False)
    assert torch.allclose(plain.float().cpu(), want, **tol)


@pytest.mark.parametrize("m, n, k", [(64, 3584, 18944), (17, 509, 352), (33, 130, 200), (48, 1000, 3584), (40, 144, 352),
                                     (64, 37, 8), (25, 4700, 1248), (57, 300, 1256), (1, 3584, 18944), (8, 2048, 11008),
                                     (16, 37, 4104), (3, 5000, 2056), (49, 8, 2048 * 300 + 8), (4, 512, 29568), (33, 260, 29568)])
def test_split_product_and_the_norm_that_adds_its_slabs(m, n, k):
    """Up to 64 rows against a weight cut along its inner size: the slabs of partial sums add up to
    the product (inner sizes that are no multiple of 32, row counts that fill no tile, more chunks
    than compute units refused), twice the same bits; and the norm kernel that takes the slabs as
    its addend gives what it gives for their sum."""
    from qwen25vl_lite_amd.ops import kernels, skinny
    torch.manual_seed(n + k)
    w = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    x = torch.randn(m, k).bfloat16()
    want = x.float() @ w.float().T
    if k > 2048 * 256:
        assert not skinny.takes_split(m, k, w.cuda())
        with pytest.raises(ValueError):
            skinny.split_product(w.cuda(), x.cuda())
        return
    assert skinny.takes_split(m, k, w.cuda()) and not skinny.takes_split(65, k, w.cuda())
    slabs = skinny.split_product(w.cuda(), x.cuda())
    assert slabs.dtype == torch.float32 and slabs.dim() == 3 and tuple(slabs.shape[1:]) == (m, n)
    assert torch.allclose(slabs.sum(0).cpu(), want, atol=3e-3, rtol=3e-3), (slabs.sum(0).cpu() - want).abs().max()
    assert torch.equal(slabs, skinny.split_product(w.cuda(), x.cuda()))
    if n % 4 == 0:
        h = torch.randn(m, n).cuda()
        g = (1 + 0.1 * torch.randn(n)).cuda()
        h1, h2 = h.clone(), h.clone()
        a = kernels.add_rmsnorm(h1, slabs, g, 1e-6, torch.bfloat16)
        total = slabs[0].clone()
        for c in range(1, slabs.shape[0]):
            total += slabs[c]
        b = kernels.add_rmsnorm(h2, total, g, 1e-6, torch.bfloat16)
        assert torch.equal(h1, h2), "the slabs are added in their order"
        # (the two kernels add the squares up in different orders: the scale may differ in its last bit)
        assert torch.allclose(a.float(), b.float(), atol=1e-2, rtol=1e-2)
        rows = torch.tensor([m - 1, 0], dtype=torch.int32).cuda()
        h3 = h.clone()
        c3 = kernels.add_rmsnorm(h3, slabs, g, 1e-6, torch.float32, rows=rows)
        assert torch.equal(h3, h) and torch.allclose(c3, kernels.add_rmsnorm(h.clone(), total, g, 1e-6, torch.float32)[[m - 1, 0]])


def test_few_row_products_at_random_sizes():
    """The resident kernel (both builds: inner sizes up to and beyond 2,048) and the split kernel at
    sizes drawn at random: any row count up to 64, widths that fill no tile, inner sizes in steps of 8
    on either side of a pass, of a chunk and of a build; every one against the float32 product."""
    import random
    from qwen25vl_lite_amd.ops import skinny
    from qwen25vl_lite_amd.ops.linear import linear, linear_into
    rng = random.Random(5)
    edges = [8, 120, 128, 136, 1016, 1024, 2040, 2048, 2056, 3832, 3840, 3848, 4088, 4096, 4104, 6144, 8200]
    for case in range(48):
        m = rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64])
        n = rng.choice([1, 5, 15, 16, 17, 100, 255, 256, 257, 1000])
        k = rng.choice(edges) if case % 2 else 8 * rng.randint(1, 700)
        torch.manual_seed(case)
        x = torch.randn(m, k).bfloat16().cuda()
        w = (torch.randn(n, k) / math.sqrt(k)).bfloat16().cuda()
        want = x.float() @ w.float().T
        got = linear(x, w, out_dtype=torch.float32)
        assert torch.allclose(got, want, atol=5e-3, rtol=5e-3), (m, n, k, (got - want).abs().max().item())
        slabs = skinny.split_product(w, x)
        assert torch.allclose(slabs.sum(0), want, atol=5e-3, rtol=5e-3), (m, n, k, (slabs.sum(0) - want).abs().max().item())
        h = torch.randn(m, n).cuda()
        before = h.clone()
        left = linear_into(h, x, w)
        total = h if left is None else h + (left.sum(0) if left.dim() == 3 else left.float())
        assert torch.allclose(total, before + want, atol=2e-2, rtol=2e-2), (m, n, k)


def test_no_cpu_path():
    from qwen25vl_lite_amd.ops import kernels
    from qwen25vl_lite_amd.ops.linear import linear
    with pytest.raises(kernels.KernelError):
        kernels.swiglu(torch.zeros(2, 4))
    with pytest.raises(kernels.KernelError):
        linear(torch.zeros(2, 4), torch.zeros(3, 4))
    with pytest.raises(kernels.KernelError):
        kernels.swiglu(torch.zeros(2, 4, dtype=torch.float16).cuda())


@pytest.mark.parametrize("ps", [16, 32, 48])
@pytest.mark.parametrize("m, nq, nkv, hd, k, bias, lazy", [(1, 4, 2, 16, 64, True, False), (8, 28, 4, 128, 3584, True, True),
                                                         (16, 6, 3, 48, 136, False, True), (5, 3, 0, 80, 104, True, False),
                                                         (32, 28, 4, 128, 3584, True, True), (17, 6, 3, 48, 136, False, True),
                                                         (27, 4, 2, 16, 64, True, False), (64, 28, 4, 128, 3584, True, False),
                                                         (33, 6, 3, 48, 136, False, False), (50, 4, 2, 16, 64, True, False)])
def test_projection_with_rotation_and_cache_write_folded_in(m, nq, nkv, hd, k, bias, lazy, ps):
    """The stacked q | k | v projection of a few rows that rotates and stores inside the product's
    kernel equals the product followed by the rotation kernel: queries, and every slot of the
    cache (the slots of other tokens keep their stale values)."""
    from qwen25vl_lite_amd.ops import kernels, skinny
    from qwen25vl_lite_amd.ops.linear import linear
    torch.manual_seed(hd + m)
    pages = 7
    n_out = (nq + 2 * nkv) * hd
    w = (torch.randn(n_out, k) / math.sqrt(k)).bfloat16().cuda()
    b = torch.randn(n_out).cuda() if bias else None
    h = (torch.randn(m, k) * 2).cuda()
    g = (1 + 0.1 * torch.randn(k)).cuda()
    x = kernels.add_rmsnorm(h, None, g, 1e-6, torch.bfloat16)
    half = hd // 2
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))).cuda()
    freq_row = (torch.arange(half) % 3).int().cuda()
    if half > 3:
        freq_row[3] = -1                        # a frequency that is not rotated
    pos = torch.randint(0, 40000, (3, m), dtype=torch.int32).cuda()
    slots = torch.randperm(pages * ps)[:m].int().cuda()
    if m > 2:
        slots[1] = -1                           # a token without a slot writes nothing
    kc0 = torch.randn(pages, max(nkv, 1), ps, hd).bfloat16().cuda()
    vc0 = torch.randn(pages, max(nkv, 1), hd, ps).bfloat16().cuda()
    kc_a, vc_a, kc_b, vc_b = kc0.clone(), vc0.clone(), kc0.clone(), vc0.clone()
    qkv = linear(x, w, out_dtype=torch.float32)
    q_a = kernels.rope_kv_write(qkv, b, pos, inv_freq, freq_row, slots if nkv else None, kc_a if nkv else None,
                                vc_a if nkv else None, nq, nkv, hd, ps, out_dtype=torch.bfloat16)
    assert skinny.takes_qkv_rope(m, k, w, hd, half, torch.bfloat16, norm=lazy)
    cs = kernels.rope_table(pos, inv_freq, freq_row, m)
    src = dict(h=h, norm_weight=g, eps=1e-6) if lazy else dict(x=x)
    q_b = skinny.qkv_rope_product(w, cs, bias=b, slots=slots if nkv else None, k_cache=kc_b if nkv else None,
                                  v_cache=vc_b if nkv else None, num_q_heads=nq, num_kv_heads=nkv, head_dim=hd,
                                  page_size=ps, **src)
    tol = dict(atol=2e-2, rtol=2e-2)           # one bfloat16 rounding of values of a few units
    assert torch.allclose(q_b.float(), q_a.float(), **tol), (q_b.float() - q_a.float()).abs().max()
    assert torch.allclose(kc_b.float(), kc_a.float(), **tol) and torch.allclose(vc_b.float(), vc_a.float(), **tol)
    if nkv:   # something was written, and only in the tokens' slots
        assert not torch.equal(kc_b, kc0) and not torch.equal(vc_b, vc0)
        touched = (kc_b != kc0).any(dim=3).any(dim=1).flatten().nonzero().flatten().tolist()
        assert set(touched) <= set(s for s in slots.tolist() if s >= 0)
    # And against the plain formulas themselves (not another path of the engine): the frequencies'
    # rows laid out by sections, the product in float32 on the host, the reference's rotation.
    sections = (half - 2 * (half // 3), half // 3, half // 3)
    rows = torch.tensor(sum(([r] * c for r, c in enumerate(sections)), []), dtype=torch.int32).cuda()
    kc_c, vc_c = kc0.clone(), vc0.clone()
    q_c = skinny.qkv_rope_product(w, kernels.rope_table(pos, inv_freq, rows, m), bias=b, slots=slots if nkv else None,
                                  k_cache=kc_c if nkv else None, v_cache=vc_c if nkv else None, num_q_heads=nq,
                                  num_kv_heads=nkv, head_dim=hd, page_size=ps, **src)
    xb = x.float().cpu() @ w.float().cpu().T + (b.cpu() if bias else 0.0)
    qs, ks, vs = xb.split([nq * hd, nkv * hd, nkv * hd], dim=1)
    cos, sin = plain_mrope_cos_sin(pos.cpu(), inv_freq.cpu())
    heads = lambda t, n: t.reshape(m, n, hd).transpose(0, 1)
    qr, kr = plain_apply_mrope(heads(qs, nq), heads(ks, nkv) if nkv else heads(qs, nq), cos, sin, sections)
    plain_tol = dict(atol=3e-2, rtol=2e-2)     # the norm's output and the result each rounded to bfloat16 once
    assert torch.allclose(q_c.float().cpu().view(m, nq, hd), qr.transpose(0, 1), **plain_tol)
    if nkv:
        kflat = kc_c.float().cpu().permute(0, 2, 1, 3).reshape(pages * ps, nkv, hd)
        vflat = vc_c.float().cpu().permute(0, 3, 1, 2).reshape(pages * ps, nkv, hd)
        live = (slots >= 0).cpu()
        at = slots.cpu().long()[live]
        assert torch.allclose(kflat[at], kr.transpose(0, 1)[live], **plain_tol)
        assert torch.allclose(vflat[at], vs.view(m, nkv, hd)[live], **plain_tol)
    # a head size whose rotation the kernel does not take, or a cache of another type, is refused
    assert not skinny.takes_qkv_rope(m, k, w, 24, 12, torch.bfloat16)
    assert not skinny.takes_qkv_rope(m, k, w, hd, half - 1, torch.bfloat16)
    assert not skinny.takes_qkv_rope(m, k, w, hd, half, torch.float32)
