"""The HIP path against the committed fixture tests/golden/layer_small.npz (a small layer pass: one cached
chunk + two denoising chunks, 4 query heads over 2 KV heads, text cross-attention with one empty segment).

Bars as elsewhere: prologue within one bf16 ulp, V rows bit exact, attention max-abs <= 2e-2 and
cosine >= 0.9999 against the stored fp32 output."""
import os

import numpy as np
import pytest
import torch

import magi_attn as M

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _bf(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def _close(out, ref, what):
    o, r = out.double().cpu().flatten(), ref.double().flatten()
    assert (o - r).abs().max().item() <= 2e-2, what
    assert (torch.dot(o, r) / (o.norm() * r.norm()).clamp_min(1e-30)).item() >= 0.9999, what


def test_layer_small_fixture(dev):
    z = np.load(os.path.join(GOLDEN, "layer_small.npz"))
    T, H, W, prefix, dn, Hq, Hkv, D = (int(x) for x in z["dims"])
    L = T * H * W
    S = dn * L
    to = lambda a: (a if isinstance(a, torch.Tensor) else torch.from_numpy(a)).to(dev)
    # the cache holds the prefix chunk; the prologue appends the new rows in place
    cache = torch.zeros((prefix + dn) * L, Hkv, 2 * D, dtype=torch.bfloat16, device=dev)
    cache[: prefix * L] = to(_bf(z["prefix_kv"]))
    q, _, _ = M.qk_prologue(to(_bf(z["q_raw"])).view(S, Hq * D), to(_bf(z["k_raw"])).view(S, Hkv * D),
                            to(_bf(z["v_raw"])).view(S, Hkv * D), to(z["rope"]), to(z["gq"]), to(z["bq"]), to(z["gk"]),
                            to(z["bk"]), Hq=Hq, Hkv=Hkv, kv_out=cache[prefix * L:], n_cache_rows=S)
    q_ref, kv_ref = _bf(z["q"]), _bf(z["kv"])
    new = cache[prefix * L:].cpu()
    for got, ref, what in ((q.cpu(), q_ref, "q"), (new[..., :D], kv_ref[..., :D], "k")):
        ulp = torch.clamp(ref.float().abs() * 2.0 ** -7, min=1e-5)
        assert torch.all((got.float() - ref.float()).abs() <= ulp), what
        assert (got != ref).float().mean().item() < 1e-3, what
    assert torch.equal(new[..., D:], kv_ref[..., D:])
    assert torch.equal(cache[: prefix * L].cpu(), _bf(z["prefix_kv"]))  # the prefix rows are untouched

    k_ranges = z["k_ranges"]
    out, lse = M.flex_flash_attn_func(q, cache[..., :D], cache[..., D:], to(z["q_ranges"]), to(k_ranges), L,
                                      int(k_ranges[:, 1].max() - k_ranges[:, 0].min()))
    _close(out, torch.from_numpy(z["out"]), "core attention")
    assert (lse.cpu() - torch.from_numpy(z["lse"])).abs().max() < 5e-3

    cu_q, cu_k = z["cu_q"], z["cu_k"]
    xout = M.flash_attn_varlen_func(q, to(_bf(z["xk"])), to(_bf(z["xv"])), to(cu_q), to(cu_k), L, int(np.diff(cu_k).max()))
    _close(xout, torch.from_numpy(z["xout"]), "cross attention")
    assert torch.count_nonzero(xout[L:]).item() == 0  # empty text segment -> zeros
