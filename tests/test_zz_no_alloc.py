"""The attention entry point that allocates nothing (``qvl_attn_mfma_coop_static``), called
through ctypes as a caller outside the package would, against the entry point that takes the
caller's scratch buffer (``qvl_attn_mfma_coop``): two calls in a row, the second with a smaller
input, so that what the first left in the library's array must not matter."""

import ctypes

import pytest
import torch

from test_gpu_kernels import _attention_case

pytestmark = pytest.mark.gpu

HD = 128
_int, _float, _ptr, _ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong


def _library():
    from qwen25vl_lite_amd.ops.library import load_library
    lib = load_library("attention_mfma", {"HD": HD})
    head = [_ptr] * 4 + [_int] + [_ptr] * 4 + [_int, _ptr]
    tail = [_int] * 4 + [_float, _int, _int, _ptr]
    lib.qvl_attn_mfma_coop.argtypes = head + [_ptr] + tail
    lib.qvl_attn_mfma_coop_static.argtypes = head + tail
    lib.qvl_attn_mfma_scratch_floats.argtypes = [_int] * 3
    lib.qvl_attn_mfma_scratch_floats.restype = _ll
    lib.qvl_attn_mfma_static_scratch_floats.restype = _ll
    for name in ("qvl_attn_mfma_coop", "qvl_attn_mfma_coop_static", "qvl_attn_mfma_coop_static_init"):
        getattr(lib, name).restype = _int
    return lib


def _case(lens, nq, nkv, window, nsplit):
    """Single decoded tokens of requests with long contexts; everything both entry points take."""
    from qwen25vl_lite_amd.ops.attention_mfma import tiles_for
    c = _attention_case(torch.bfloat16, nq, nkv, HD, window, lens, (1,) * len(lens))
    cu = list(range(len(lens) + 1))
    req, ct = tiles_for(cu, nq // nkv)
    most = max(lens)
    per = ((most + 31 + nsplit - 1) // nsplit + 31) // 32 * 32
    dev = lambda a: torch.tensor(a, dtype=torch.int32).cuda()
    c.update(cu_q=dev(cu), ctx=dev(list(lens)), tile_req=dev(req.tolist()), tile_ct=dev(ct.tolist()), tiles=len(req),
             nsplit=(most + 31 + per - 1) // per, per=per, nq=nq, nkv=nkv, window=window or 0)
    return c


def _head(c, out):
    return [c["q"].data_ptr(), c["kc"].data_ptr(), c["vc"].data_ptr(), c["table"].data_ptr(), c["table"].shape[1],
            c["cu_q"].data_ptr(), c["ctx"].data_ptr(), c["tile_req"].data_ptr(), c["tile_ct"].data_ptr(), c["tiles"],
            out.data_ptr()]


def _tail(c, stream):
    return [c["nq"], c["nkv"], 16, c["window"], c["scale"], c["nsplit"], c["per"], stream]


def test_the_entry_point_that_allocates_nothing_matches_the_one_with_a_scratch_argument():
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.qvl_attn_mfma_coop_static_init() == 0
    limit = lib.qvl_attn_mfma_static_scratch_floats()
    assert limit == 2 * 1024 * 1024
    big = _case((2100, 700, 1300, 33), 14, 2, None, 4)
    small = _case((1500, 90), 4, 2, 1200, 2)       # fewer requests, heads and splits, and a window
    assert big["nsplit"] > small["nsplit"] > 1
    for c in (big, small):                         # the second call finds the first one's partial results
        need = lib.qvl_attn_mfma_scratch_floats(c["tiles"], c["nkv"], c["nsplit"])
        assert 0 < need <= limit
        scratch = torch.full((need,), float("nan"), device="cuda")
        want = torch.zeros_like(c["q"])
        got = torch.zeros_like(c["q"])
        assert lib.qvl_attn_mfma_coop(*_head(c, want), scratch.data_ptr(), *_tail(c, stream)) == 0
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        assert lib.qvl_attn_mfma_coop_static(*_head(c, got), *_tail(c, stream)) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before, "the call took device memory"
        assert torch.equal(got, want), (got.float() - want.float()).abs().max()
        assert torch.allclose(got.float().cpu(), c["want"], atol=1.5e-2, rtol=2e-2)


def test_a_call_beyond_the_array_is_refused_and_launches_nothing():
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    c = _case((600, 40), 4, 2, None, 2)
    out = torch.full_like(c["q"], 3.0)
    tiles_too_many = dict(c, tiles=10_000, nsplit=64, per=32)
    assert lib.qvl_attn_mfma_scratch_floats(10_000, 2, 64) > lib.qvl_attn_mfma_static_scratch_floats()
    assert lib.qvl_attn_mfma_coop_static(*_head(tiles_too_many, out), *_tail(tiles_too_many, stream)) == 4
    torch.cuda.synchronize()
    assert torch.all(out == 3.0)
