"""GPU tests of the measured score bound (MAGI_ATTN_AUTO_BOUND): a bf16 call that states no bound has the library
measure max|q| and max|k| and pick the kernel on the device.  Whichever kernel the measurement selects must give, bit
for bit, what a direct call of that kernel gives; the selection itself is checked through inputs on either side of
MAGI_SCORE_BOUND_MAX."""
import math

import numpy as np
import pytest
import torch

import magi_attn as M
from magi_attn import _lib as L
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu


def _ranges(dev, *arrs):
    return [torch.tensor(np.asarray(a), dtype=torch.int32, device=dev) for a in arrs]


def _case(dev, L_, dn, sp, Hq, Hkv, seed, gain=1.0):
    q, k, v = O.synthetic_qkv(dn * L_, (sp + dn) * L_, Hq, Hkv, 128, seed=seed)
    q, k = (q.float() * gain).bfloat16(), (k.float() * gain).bfloat16()
    qr, kr = O.q_ranges_for(dn, L_), O.default_kvrange(sp, dn, L_)
    tq, tk = _ranges(dev, qr, kr)
    return q, k, v, qr, kr, tq, tk


@pytest.mark.parametrize("L_,dn,sp,Hq,Hkv", [(200, 3, 1, 6, 2), (1, 3, 2, 6, 1), (333, 4, 3, 12, 4), (1536, 3, 0, 24, 8)])
def test_measured_bound_selects_the_bounded_kernel_on_normed_inputs(dev, L_, dn, sp, Hq, Hkv):
    """QK-normed q and k (lengths sqrt(128)): the measured bound is 16.5, the bounded-score kernel runs, scaling q
    while it loads it.  Bit-identical to the same call with a stated bound, five launches, parity with the oracle."""
    q, k, v, qr, kr, tq, tk = _case(dev, L_, dn, sp, Hq, Hkv, seed=99 + L_)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    before = L.lib().magi_launch_count()
    out, lse = M.range_attention(qd, kd, vd, tq, tk, L_, auto_bound=True)
    assert L.lib().magi_launch_count() - before == 5
    stated, lse_s = M.range_attention(qd, kd, vd, tq, tk, L_, score_bound=17.0)
    assert torch.equal(out, stated) and torch.equal(lse, lse_s)
    ref = O.range_attention(q, k, v, qr, kr)
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2
    # pre-scaled q: the bound is measured on q as it is
    qp = (q.float() * (128 ** -0.5 * math.log2(math.e))).bfloat16().to(dev)
    out_p, _ = M.range_attention(qp, kd, vd, tq, tk, L_, q_prescaled=True, auto_bound=True)
    stated_p, _ = M.range_attention(qp, kd, vd, tq, tk, L_, q_prescaled=True, score_bound=17.0)
    assert torch.equal(out_p, stated_p)


@pytest.mark.parametrize("gain", [2.0, 3.0])
def test_measured_bound_above_the_limit_runs_the_online_softmax(dev, gain):
    """Lengths of gain * sqrt(128) on both sides: bounds of 66 and 148, above MAGI_SCORE_BOUND_MAX, so the kernel with
    the running maximum has to produce the result: bit-identical to the plain call."""
    q, k, v, qr, kr, tq, tk = _case(dev, 150, 3, 1, 6, 2, seed=5, gain=gain)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out, lse = M.range_attention(qd, kd, vd, tq, tk, 150, auto_bound=True)
    plain, lse_p = M.range_attention(qd, kd, vd, tq, tk, 150)
    assert torch.equal(out, plain) and torch.equal(lse, lse_p)
    assert (out.float().cpu() - O.range_attention(q, k, v, qr, kr)).abs().max().item() <= 2e-2


def test_measured_bound_just_below_and_just_above_the_limit(dev):
    """One long key decides: k row 7 scaled so that max|q| max|k| scale log2(e) * 1.01 lands at 63.9 and at 64.1."""
    q, k, v, qr, kr, tq, tk = _case(dev, 100, 2, 1, 4, 2, seed=11)
    qd, vd = q.to(dev), v.to(dev)
    factor = 128 ** -0.5 * math.log2(math.e) * 1.01
    qmax = q.float().norm(dim=-1).max().item()
    base = k.float().norm(dim=-1)
    for target, bounded in ((63.0, True), (65.5, False)):
        k2 = k.clone()
        k2[7, 1] = (k[7, 1].float() * (target / (factor * qmax * base[7, 1].item()))).bfloat16()
        measured = factor * qmax * k2.float().norm(dim=-1).max().item()
        assert (measured <= 64.0) == bounded, measured
        out, _ = M.range_attention(qd, k2.to(dev), vd, tq, tk, 100, auto_bound=True)
        want, _ = M.range_attention(qd, k2.to(dev), vd, tq, tk, 100, **({"score_bound": 64.0} if bounded else {}))
        assert torch.equal(out, want), target


def test_measured_bound_sees_both_key_segments_and_nans(dev):
    """The long key sits in the side segment (k2); and a NaN in k sends the call to the online-softmax kernel, whose
    result (NaN in the rows that see that key, finite elsewhere) is what the plain call gives."""
    L_, sp, dn, Hq, Hkv = 90, 2, 2, 4, 2
    q, k, v, qr, kr, tq, tk = _case(dev, L_, dn, sp, Hq, Hkv, seed=3)
    qd = q.to(dev)
    split = sp * L_ + 30
    k_long = k.clone()
    k_long[split + 5, 0] *= 6.0  # bound 6 x 16.5: above the limit, and only the side segment shows it
    head, tail = k_long[:split].to(dev), k_long[split:].to(dev)
    vh, vt = v[:split].to(dev), v[split:].to(dev)
    out, _ = M.range_attention(qd, head, vh, tq, tk, L_, k2=tail, v2=vt, k_split=split, auto_bound=True)
    plain, _ = M.range_attention(qd, head, vh, tq, tk, L_, k2=tail, v2=vt, k_split=split)
    assert torch.equal(out, plain)
    assert (out.float().cpu() - O.range_attention(q, k_long, v, qr, kr)).abs().max().item() <= 2e-2
    # without the long key the same split call takes the bounded kernel
    out_b, _ = M.range_attention(qd, k[:split].to(dev), vh, tq, tk, L_, k2=k[split:].to(dev), v2=vt, k_split=split, auto_bound=True)
    stated, _ = M.range_attention(qd, k[:split].to(dev), vh, tq, tk, L_, k2=k[split:].to(dev), v2=vt, k_split=split, score_bound=17.0)
    assert torch.equal(out_b, stated)
    k_nan = k.clone()
    k_nan[3, 1, 17] = float("nan")
    out_n, _ = M.range_attention(qd, k_nan.to(dev), v.to(dev), tq, tk, L_, auto_bound=True)
    plain_n, _ = M.range_attention(qd, k_nan.to(dev), v.to(dev), tq, tk, L_)
    assert torch.equal(torch.isnan(out_n), torch.isnan(plain_n)) and torch.isnan(out_n).any()
    assert torch.equal(torch.nan_to_num(out_n), torch.nan_to_num(plain_n))


def test_reference_shaped_callables_measure_a_bound_where_it_pays(dev):
    """flex_flash_attn_func without any extra argument, as the reference calls it: on a launch that is large beside
    two passes over q and k it measures the bound (five launches) and equals the call with a stated bound; on a small
    one it launches the online-softmax kernel alone."""
    assert M.functional._measuring_a_bound_pays(torch.empty(86400, 48, 128, dtype=torch.bfloat16, device="meta"),
                                                torch.empty(259200, 8, 128, dtype=torch.bfloat16, device="meta"), 4, 21600, 259200)
    assert not M.functional._measuring_a_bound_pays(torch.empty(86400, 48, 128, dtype=torch.bfloat16, device="meta"),
                                                    torch.empty(2700, 8, 128, dtype=torch.bfloat16, device="meta"), 4, 21600, 800)
    L_, dn, sp, Hq, Hkv = 4096, 2, 2, 8, 2
    q, k, v, qr, kr, tq, tk = _case(dev, L_, dn, sp, Hq, Hkv, seed=21)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    before = L.lib().magi_launch_count()
    out, lse = M.flex_flash_attn_func(qd, kd, vd, tq, tk, L_, (sp + dn) * L_)
    launches = L.lib().magi_launch_count() - before
    assert launches == (5 if M.functional._measuring_a_bound_pays(qd, kd, dn, L_, (sp + dn) * L_) else 1)
    forced, _ = M.flex_flash_attn_func(qd, kd, vd, tq, tk, L_, (sp + dn) * L_, auto_bound=True)
    stated, _ = M.flex_flash_attn_func(qd, kd, vd, tq, tk, L_, (sp + dn) * L_, score_bound=17.0)
    assert torch.equal(forced, stated)
    if launches == 5:
        assert torch.equal(out, stated)
    small = M.flex_flash_attn_func(qd[:64], kd[:64], vd[:64], *_ranges(dev, [[0, 64]], [[0, 64]]), 64, 64)[0]
    before = L.lib().magi_launch_count()
    M.flex_flash_attn_func(qd[:64], kd[:64], vd[:64], *_ranges(dev, [[0, 64]], [[0, 64]]), 64, 64)
    assert L.lib().magi_launch_count() - before == 1 and small.shape == (64, Hq, 128)


def test_auto_bound_argument_checks(dev):
    q = torch.zeros(8, 2, 128, dtype=torch.bfloat16, device=dev)
    r = torch.tensor([[0, 8]], dtype=torch.int32, device=dev)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 8, auto_bound=True, score_bound=10.0)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 8, auto_bound=True, q_tile_rows=128)
    g = torch.zeros(128, device=dev)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 8, auto_bound=True, q_norm=(g, None, 1e-6))
    # the C entry refuses the flag without a workspace
    a = L.AttnArgs()
    a.q = a.k = a.v = a.out = q.data_ptr()
    a.q_ranges = a.k_ranges = r.data_ptr()
    a.q_stride_t = a.k_stride_t = a.v_stride_t = a.o_stride_t = 256
    a.q_stride_h = a.k_stride_h = a.v_stride_h = a.o_stride_h = 128
    a.total_q = a.total_k = a.k_split = 8
    a.n_ranges, a.max_seqlen_q, a.Hq, a.Hkv, a.D = 1, 8, 2, 2, 128
    a.flags = L.MAGI_ATTN_AUTO_BOUND
    assert L.lib().magi_attn_fwd(a, None) == -22 and b"workspace" in L.lib().magi_last_error()
