"""GPU parity of the fused projection GEMM + prologue (magi_qkv_proj_prologue) against the CPU oracle.

Expected values: the projections in float64, rounded once to bf16 (the reference's linear layers return bf16,
dit_module.py:390-425), then the oracle's prologue (get_q / get_k / get_v, dit_module.py:953-996).  The kernel
accumulates in fp32 in its own order, so a raw value that lies within ~1e-6 relative of a bf16 rounding boundary may
round the other way (as it may in any library GEMM); after the norm such an element is off by up to about two bf16
ulps of ITS magnitude, which after the rotation (x1 cos - x2 sin may cancel) can be many ulps of a small result.
Bar: v and the raw cross-attention q equal to the rounded float64 product up to one bf16 ulp; q and k within one bf16
ulp of the oracle (absolute floor 1e-5 where the rotation cancels) for all but 1 in 1000 elements, and everywhere
within 2^-6 of the largest magnitude of the same (token, head) row (one ulp of a raw value that large plus the
roundings of the result)."""
import math

import pytest
import torch

import magi_attn as M
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu


def _problem(S, K, Hq, Hkv, Hqx, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(S, K, generator=g).bfloat16()
    w = (torch.randn((Hq + 2 * Hkv + Hqx) * 128, K, generator=g) * K ** -0.5).bfloat16()
    par = [torch.randn(128, generator=g) * 0.2 for _ in range(4)]
    return x, w, par


def _raw(x, w):
    return (x.double() @ w.double().T).bfloat16()


def _close(got, ref, what, exact_share=1e-3, max_ulps=None):
    gf, rf = got.float().cpu(), ref.float()
    ulp = torch.clamp(rf.abs() * 2.0 ** -7, min=1e-5)
    d = (gf - rf).abs()
    if max_ulps is None:
        bound = torch.maximum(ulp, rf.abs().amax(dim=-1, keepdim=True) * 2.0 ** -6)
        assert torch.all(d <= bound), f"{what}: {(d / bound).max().item():.2f} x the row-scaled bound"
    else:
        assert torch.all(d <= max_ulps * ulp), f"{what}: more than {max_ulps} bf16 ulps off ({(d / ulp).max().item():.1f})"
    share = (d > ulp).float().mean().item()
    assert share < exact_share, f"{what}: {share:.2e} of the elements are more than one ulp off"


@pytest.mark.parametrize("S,K,Hq,Hkv,Hqx,keep,T,H,W", [
    (2 * 4 * 6 * 6, 256, 6, 2, 6, 1, 12, 4, 6),     # 288 tokens: a ragged second token tile
    (2 * 8 * 8 * 4, 512, 2, 1, 2, 2, 8, 8, 8),      # 512 tokens, 3 column tiles
    (6 * 5 * 7, 1024, 24, 8, 24, 0, 6, 5, 7),       # 210 tokens (less than a tile), 32 column tiles, all rows to the side buffer
    (2 * 16 * 20, 6144, 4, 2, 4, 2, 2, 16, 20),     # the layer's K
])
def test_fused_projection_and_prologue(dev, S, K, Hq, Hkv, Hqx, keep, T, H, W):
    D = 128
    x, w, (gq, bq, gk, bk) = _problem(S, K, Hq, Hkv, Hqx, seed=S + K)
    dn = 2 if T % 2 == 0 else 1
    rope = O.rope_for_forward(T, H, W, 1, dn)[-S:].contiguous()
    assert rope.shape == (S, 96)
    cs = D ** -0.5 * math.log2(math.e)
    raw = _raw(x, w)
    nq, nk = Hq * D, Hkv * D
    q_raw, k_raw, v_raw, qx_raw = raw[:, :nq], raw[:, nq:nq + nk], raw[:, nq + nk:nq + 2 * nk], raw[:, nq + 2 * nk:]
    q_ref, kv_ref = O.prologue(q_raw.reshape(S, Hq, D), k_raw.reshape(S, Hkv, D), v_raw.reshape(S, Hkv, D), rope, gq, bq,
                               gk, bk, q_premul=cs)
    to = lambda t: t.to(dev)
    L = S // dn
    n_keep = keep * L if keep * L <= S else S
    cache = torch.full((S + 3, Hkv, 2 * D), 7.0, dtype=torch.bfloat16, device=dev)
    side = torch.full((S, Hkv, 2 * D), 7.0, dtype=torch.bfloat16, device=dev)
    q, _, _, qx = M.qkv_proj_prologue(to(x), to(w), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv, Hqx=Hqx,
                                      q_premul=cs, kv_out=cache[3:], n_cache_rows=n_keep, kv_tail=side)
    kv = torch.cat([cache[3:3 + n_keep], side[:S - n_keep]])
    _close(q, q_ref, "q")
    _close(kv[..., :D], kv_ref[..., :D], "k")
    _close(kv[..., D:], kv_ref[..., D:], "v", max_ulps=1)
    _close(qx, qx_raw.reshape(S, Hqx, D), "qx", max_ulps=1)
    assert torch.all(cache[:3] == 7.0) and torch.all(cache[3 + n_keep:] == 7.0) and torch.all(side[S - n_keep:] == 7.0)
    # against the two-step path of the library on the device (a library GEMM, then the prologue kernel): same bar
    raw_dev = torch.nn.functional.linear(to(x), to(w))
    q2, kv2, _ = M.qk_prologue(raw_dev[:, :nq], raw_dev[:, nq:nq + nk], raw_dev[:, nq + nk:nq + 2 * nk], to(rope), to(gq),
                               to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv, q_premul=cs)
    _close(q, q2.cpu(), "q vs two-step")
    _close(kv, kv2.cpu(), "kv vs two-step")


def test_fused_projection_variants_and_argument_checks(dev):
    D, S, K, Hq, Hkv = 128, 100, 128, 2, 1
    x, w, (gq, bq, gk, bk) = _problem(S, K, Hq, Hkv, 2, seed=3)
    to = lambda t: t.to(dev)
    raw = _raw(x, w)
    # RMS norm, no rotary, batch 2 ordering is irrelevant without a table; strided x rows
    xs = torch.zeros(S, K + 64, dtype=torch.bfloat16)
    xs[:, :K] = x
    q, kv, _, qx = M.qkv_proj_prologue(to(xs)[:, :K], to(w), None, to(gq), None, to(gk), None, Hq=Hq, Hkv=Hkv, Hqx=2,
                                       norm_kind=M.MAGI_NORM_RMSNORM_1P)
    q_ref = O.rmsnorm(raw[:, :Hq * D].reshape(S, Hq, D).float(), gq + 1).bfloat16()
    k_ref = O.rmsnorm(raw[:, Hq * D:(Hq + Hkv) * D].reshape(S, Hkv, D).float(), gk + 1).bfloat16()
    _close(q, q_ref, "q rms")
    _close(kv[..., :D], k_ref, "k rms")
    # no norm at all: the plain projections
    q, kv, _, qx = M.qkv_proj_prologue(to(x), to(w), None, None, None, None, None, Hq=Hq, Hkv=Hkv, Hqx=2,
                                       norm_kind=M.MAGI_NORM_NONE)
    _close(q, raw[:, :Hq * D].reshape(S, Hq, D), "q plain", max_ulps=1)
    _close(qx, raw[:, (Hq + 2 * Hkv) * D:].reshape(S, 2, D), "qx plain", max_ulps=1)
    # rotary table per position with two batch rows per position
    rope = O.rope_for_forward(2, 5, 5, 0, 1)
    q, kv, _, _ = M.qkv_proj_prologue(to(x), to(w), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv, Hqx=2, batch=2)
    q_ref, kv_ref = O.prologue(raw[:, :Hq * D].reshape(S, Hq, D), raw[:, Hq * D:(Hq + Hkv) * D].reshape(S, Hkv, D),
                               raw[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].reshape(S, Hkv, D),
                               rope.repeat_interleave(2, dim=0), gq, bq, gk, bk)
    _close(q, q_ref, "q batch 2")
    _close(kv, kv_ref, "kv batch 2")
    with pytest.raises(M.MagiError):  # an odd number of heads
        M.qkv_proj_prologue(to(x), to(w)[:5 * D], None, to(gq), None, to(gk), None, Hq=Hq, Hkv=Hkv, Hqx=1)
    with pytest.raises(M.MagiError):  # K not a multiple of 64
        M.qkv_proj_prologue(to(x)[:, :96].contiguous(), to(w)[:, :96].contiguous(), None, to(gq), None, to(gk), None,
                            Hq=Hq, Hkv=Hkv, Hqx=2)
    with pytest.raises(M.MagiError):  # a rotary width other than 96
        M.qkv_proj_prologue(to(x), to(w), torch.zeros(S, 64, device=dev), to(gq), None, to(gk), None, Hq=Hq, Hkv=Hkv, Hqx=2)
