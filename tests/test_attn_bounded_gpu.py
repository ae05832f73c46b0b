"""GPU parity of the bounded-score attention path (64 query rows per wavefront, no running maximum; through
the C-ABI with magi_attn_args.score_bound) against the CPU oracle and against the online-softmax kernel.

The inputs are what the layer produces: q pre-multiplied by softmax_scale * log2(e) before its one rounding to
bf16, per-head normalised q and k, so that |q . k| <= |q| |k| is known.  Tolerance as for the other bf16 tests
(benchmark definition): max-abs <= 2e-2 and cosine >= 0.9999 against the fp32 reference."""
import math

import numpy as np
import pytest
import torch

import magi_attn as M
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MIN_COS = 0.9999
PREMUL = 128 ** -0.5 * math.log2(math.e)
LN2 = math.log(2.0)


def _cmp(out, ref, what=""):
    o = out.detach().double().cpu().flatten()
    r = ref.detach().double().cpu().flatten()
    err = (o - r).abs().max().item()
    cos = (torch.dot(o, r) / (o.norm() * r.norm()).clamp_min(1e-30)).item()
    assert err <= MAX_ABS, f"{what}: max-abs {err}"
    assert cos >= MIN_COS, f"{what}: cosine {cos}"
    return err, cos


def _ranges(dev, *arrs):
    return [torch.tensor(np.asarray(a), dtype=torch.int32, device=dev) for a in arrs]


def _inputs(Tq, Tk, Hq, Hkv, seed, gain=1.0):
    """q (pre-scaled, bf16), k, v and the Cauchy-Schwarz bound of |q . k| computed from the tensors themselves."""
    q, k, v = O.synthetic_qkv(Tq, Tk, Hq, Hkv, 128, seed=seed, dtype=torch.float32)
    q = (q * (gain * PREMUL)).bfloat16()
    k = (k * gain).bfloat16()
    v = v.bfloat16()
    bound = (q.float().norm(dim=-1).max() * k.float().norm(dim=-1).max()).item() if Tk else 1.0
    return q, k, v, bound


CASES = [
    # L, dn, sp, Hq, Hkv
    (128, 1, 0, 1, 1),      # half a q tile of the 256-row workgroup, two key tiles
    (64, 2, 0, 2, 1),       # one wave of the four
    (200, 3, 1, 6, 2),      # ragged everywhere, GQA 3
    (77, 2, 2, 3, 1),       # L below one tile; second row block of wave 1 partly filled
    (1, 3, 2, 6, 1),        # single-token chunks, GQA 6
    (333, 4, 3, 12, 4),     # two q tiles per range, 13 rows in the last wave
    (1536, 3, 0, 24, 8),    # the CPU-runnable benchmark configuration
]


@pytest.mark.parametrize("rows", [0, 256, 512, "mfma32"])
@pytest.mark.parametrize("L,dn,sp,Hq,Hkv", CASES)
def test_bounded_chunk_causal_parity(dev, L, dn, sp, Hq, Hkv, rows):
    """rows: the workgroup shape (magi_attn_args.q_tile_rows; 0 = the library's choice, 256 rows): 256 = 4 waves of 64
    query rows on the 16x16x32 MFMA, 512 = 8 waves on the 32x32x16 MFMA; "mfma32" = 4 waves on the 32x32x16 MFMA
    (MAGI_ATTN_BOUNDED_MFMA32)."""
    mfma32 = rows == "mfma32"
    rows = 0 if mfma32 else rows
    q, k, v, bound = _inputs(dn * L, (sp + dn) * L, Hq, Hkv, seed=4321 + L)
    assert bound <= M.MAGI_SCORE_BOUND_MAX
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    ref = O.range_attention(q, k, v, qr, kr, softmax_scale=LN2)  # q carries softmax_scale * log2(e)
    lse_ref = O.range_attention_lse(q, k, v, qr, kr, softmax_scale=LN2)
    tq, tk = _ranges(dev, qr, kr)
    out, lse = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, int(kr.max() - kr.min()),
                                 q_prescaled=True, score_bound=bound, q_tile_rows=rows, bounded_mfma32=mfma32)
    _cmp(out, ref, f"L={L}")
    assert (lse.cpu() - lse_ref).abs().max() < 5e-3
    # against the online-softmax kernel on the same inputs: the same softmax up to the rounding of p to bf16
    # (relative to the row maximum there, to 2^score here)
    base, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_prescaled=True)
    assert (out.float() - base.float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("gain", [0.25, 1.9])
def test_bounded_extreme_score_ranges(dev, gain):
    """Scores near the upper end of the allowed bound (2^+-59 next to each other in one row sum) and tiny ones."""
    L, dn, sp, Hq, Hkv = 160, 2, 1, 4, 2
    q, k, v, bound = _inputs(dn * L, (sp + dn) * L, Hq, Hkv, seed=99, gain=gain)
    assert bound <= M.MAGI_SCORE_BOUND_MAX
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    ref = O.range_attention(q, k, v, qr, kr, softmax_scale=LN2)
    tq, tk = _ranges(dev, qr, kr)
    out, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_prescaled=True, score_bound=bound)
    assert torch.isfinite(out).all()
    _cmp(out, ref, f"gain={gain}")


def test_bound_above_the_limit_falls_back_to_the_running_maximum(dev):
    L, Hq, Hkv = 96, 2, 1
    q, k, v, _ = _inputs(L, L, Hq, Hkv, seed=5, gain=4.0)  # |q . k| up to ~260: 2^score overflows fp32
    qr = kr = np.array([[0, L]])
    tq, tk = _ranges(dev, qr, kr)
    base, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_prescaled=True)
    out, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_prescaled=True, score_bound=300.0)
    assert torch.equal(out, base)


def test_bounded_varlen_segments_with_empty_and_ragged_keys(dev):
    """cu_seqlens ranges as the T5 cross attention uses them: key segments of 0, 1, 31, 32, 33, 64, 65, 800 tokens."""
    Lq, Hq, Hkv = 300, 6, 2
    lens = [0, 1, 31, 32, 33, 64, 65, 800]
    cu_q = np.arange(0, (len(lens) + 1) * Lq, Lq)
    cu_k = np.concatenate([[0], np.cumsum(lens)])
    q, k, v, bound = _inputs(int(cu_q[-1]), int(cu_k[-1]), Hq, Hkv, seed=17)
    ref = O.varlen_cross_attention(q, k, v, torch.tensor(cu_q), torch.tensor(cu_k), softmax_scale=LN2)
    tq, tk = _ranges(dev, cu_q, cu_k)
    out, lse = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, Lq, 800, ranges_mode=M.MAGI_RANGES_CU,
                                 q_prescaled=True, score_bound=bound)
    assert torch.all(out[:Lq] == 0) and torch.all(torch.isinf(lse[:, :Lq]))
    _cmp(out, ref)


@pytest.mark.parametrize("mode", ["prescaled", "scale_on_load", "mfma32"])
def test_bounded_every_key_tail_length(dev, mode):
    """Key segments of every length from 1 to 131 in one launch (every position of the ragged end inside a 64-key
    tile and inside its 16-key blocks, with one, two and three tiles), query segments of 3 to 67 rows (partly filled
    16-row blocks and waves), an offset start of the key axis; output and lse against the oracle per segment."""
    Hq, Hkv = 4, 2
    k_lens = np.arange(1, 132)
    q_lens = 3 + (np.arange(len(k_lens)) * 7) % 65
    qs = np.concatenate([[0], np.cumsum(q_lens)])
    ks = 5 + np.concatenate([[0], np.cumsum(k_lens)])       # keys start at row 5, not at a tile boundary
    qr = np.stack([qs[:-1], qs[1:]], 1)
    kr = np.stack([ks[:-1], ks[1:]], 1)
    q, k, v, bound = _inputs(int(qs[-1]), int(ks[-1]) + 9, Hq, Hkv, seed=23)
    tq, tk = _ranges(dev, qr, kr)
    if mode == "scale_on_load":
        q_in = (q.float() / PREMUL).bfloat16()                # unscaled q: the kernel applies softmax_scale * log2(e)
        kw, scale = dict(score_bound=1.01 * bound), None      # (oracle: default softmax scale, natural exponential)
    else:
        q_in, scale = q, LN2
        kw = dict(q_prescaled=True, score_bound=bound, bounded_mfma32=(mode == "mfma32"))
    out, lse = M.range_attention(q_in.to(dev), k.to(dev), v.to(dev), tq, tk, int(q_lens.max()), int(k_lens.max()), **kw)
    ref = O.range_attention(q_in, k, v, qr, kr, softmax_scale=scale)
    ref_lse = O.range_attention_lse(q_in, k, v, qr, kr, softmax_scale=scale)
    _cmp(out, ref, mode)
    # (the lse of a one-key segment IS its score; the second rounding of q moves a score by ~2e-3 r.m.s., so the
    # largest of 20000 rows lies around four times that)
    assert (lse.cpu() - ref_lse).abs().max().item() < (2e-2 if mode == "scale_on_load" else 5e-3)
    worst = max(((out[a:b].double().cpu() - ref[a:b].double()).abs().max().item(), int(n)) for (a, b), n in zip(qr, k_lens))
    assert worst[0] <= MAX_ABS, f"segment with {worst[1]} keys: {worst[0]}"


@pytest.mark.parametrize("mfma32", [False, True])
def test_bounded_cache_views_two_segments_and_grouped_output(dev, mfma32):
    """K / V read in place from an interleaved cache, the key axis split into [cache prefix | side buffer] at
    tile-unfriendly places, and the output written in the two-level head layout: all bit-identical to the plain call."""
    L, sp, dn, Hq, Hkv, D = 90, 2, 3, 8, 2, 128
    q, k, v, bound = _inputs(dn * L, (sp + dn) * L, Hq, Hkv, seed=8)
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    tq, tk = _ranges(dev, qr, kr)
    kw = dict(q_prescaled=True, score_bound=bound, bounded_mfma32=mfma32)
    base = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, **kw)[0]
    _cmp(base, O.range_attention(q, k, v, qr, kr, softmax_scale=LN2))
    cache = torch.cat([k, v], -1).to(dev)
    out = M.range_attention(q.to(dev), cache[..., :D], cache[..., D:], tq, tk, L, **kw)[0]
    assert torch.equal(out, base)
    for split in (0, sp * L, sp * L + 37, (sp + dn) * L):
        big = torch.full((split + 5, Hkv, 2 * D), float("nan"), dtype=torch.bfloat16, device=dev)
        big[:split] = cache[:split]
        tail = cache[split:].clone()
        o2 = M.range_attention(q.to(dev), big[:split, :, :D], big[:split, :, D:], tq, tk, L, k2=tail[..., :D],
                               v2=tail[..., D:], k_split=split, **kw)[0]
        assert torch.equal(o2, base), f"split={split}"
    grouped = torch.zeros(dn * L, 4, Hq // 4, D, dtype=torch.bfloat16, device=dev)[:, :, :, :]
    M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, out=grouped, return_lse=False, **kw)
    assert torch.equal(grouped.view(dn * L, Hq, D), base)


def test_score_bound_argument_checks(dev):
    q = torch.zeros(4, 1, 128, dtype=torch.bfloat16, device=dev)
    r = torch.tensor([[0, 4]], dtype=torch.int32, device=dev)
    q8 = q.view(torch.uint8)[..., :128].view(torch.float8_e4m3fn)
    one = torch.ones(1, 1, device=dev)
    with pytest.raises(M.MagiError):  # a promise about bf16 inputs
        M.range_attention(q8, q8, q8, r, r, 4, q_scale=one, k_scale=one, v_scale=one, scale_chunk_tokens=4, score_bound=8.0)
    with pytest.raises(M.MagiError):  # unscaled q with a bound: 256-row workgroups only
        M.range_attention(q, q, q, r, r, 4, score_bound=8.0, q_tile_rows=512)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 4, q_prescaled=True, score_bound=-1.0)
    with pytest.raises(M.MagiError):  # 384-row workgroups belong to the online-softmax kernel
        M.range_attention(q, q, q, r, r, 4, q_prescaled=True, score_bound=8.0, q_tile_rows=384)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 4, q_tile_rows=512)
    with pytest.raises(M.MagiError):  # the 32x32x16 form takes pre-scaled q and a bound
        M.range_attention(q, q, q, r, r, 4, score_bound=8.0, bounded_mfma32=True)
    with pytest.raises(M.MagiError):
        M.range_attention(q, q, q, r, r, 4, q_prescaled=True, bounded_mfma32=True)


@pytest.mark.parametrize("L,dn,sp,Hq,Hkv", CASES)
def test_bound_on_unscaled_q_scales_while_loading(dev, L, dn, sp, Hq, Hkv):
    """A score bound WITHOUT q_prescaled, as the reference-shaped callables pass it (the reference hands its
    attention functions unscaled q and softmax_scale=None): the kernel multiplies q by softmax_scale * log2(e) while
    loading it.  q is then rounded to bf16 twice (once by its producer, once after the scale), each 2^-9 relative
    per element, which moves a score by ~2e-3 exp2 units r.m.s.: well inside the bf16 bar against the oracle on the
    unscaled q, and close to the kernel fed with q pre-scaled ahead of its single rounding."""
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=4321 + L)
    bound = M.qk_norm_score_bound(q.float().norm(dim=-1).max().item(), k.float().norm(dim=-1).max().item() if k.numel() else 1.0)
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    ref = O.range_attention(q, k, v, qr, kr)
    lse_ref = O.range_attention_lse(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr, kr)
    out, lse = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, int(kr.max() - kr.min()),
                                      score_bound=bound)
    _cmp(out, ref, f"L={L}")
    assert (lse.cpu() - lse_ref).abs().max() < 5e-3
    online, _ = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, int(kr.max() - kr.min()))
    assert (out.float() - online.float()).abs().max().item() <= 2e-2
    # an explicit softmax_scale is honoured (the bound is stated in the units of the scaled scores)
    out2, _ = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, int(kr.max() - kr.min()),
                                     softmax_scale=0.05, score_bound=bound)
    _cmp(out2, O.range_attention(q, k, v, qr, kr, softmax_scale=0.05), f"L={L} scale 0.05")


def test_reference_shaped_callables_take_a_score_bound(dev):
    """flash_attn_func / flash_attn_varlen_func with score_bound=: batched and varlen forms, an empty segment, the
    interleaved cache read in place: same results as without the bound, to the rounding of the probabilities."""
    g = torch.Generator().manual_seed(9)
    B, Sq, Sk, Hq, Hkv, D = 3, 70, 150, 4, 2, 128
    q = O.rmsnorm(torch.randn(B, Sq, Hq, D, generator=g)).bfloat16()
    k = O.rmsnorm(torch.randn(B, Sk, Hkv, D, generator=g)).bfloat16()
    v = torch.randn(B, Sk, Hkv, D, generator=g).bfloat16()
    bound = M.qk_norm_score_bound(1.01 * D ** 0.5, 1.01 * D ** 0.5)
    out = M.flash_attn_func(q.to(dev), k.to(dev), v.to(dev), score_bound=bound)
    for b in range(B):
        _cmp(out[b], O.range_attention(q[b], k[b], v[b], [[0, Sq]], [[0, Sk]]), f"batch {b}")
    Lq = 130
    lens = [800, 0, 20, 413]
    qx = O.rmsnorm(torch.randn(len(lens) * Lq, Hq, D, generator=g)).bfloat16()
    kvx = torch.randn(sum(lens), Hkv, 2 * D, generator=g)
    kvx[..., :D] = O.rmsnorm(kvx[..., :D])
    kvx = kvx.bfloat16()
    cu_q = torch.arange(0, (len(lens) + 1) * Lq, Lq, dtype=torch.int32)
    cu_k = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32)
    kd = kvx.to(dev)
    ox = M.flash_attn_varlen_func(qx.to(dev), kd[..., :D], kd[..., D:], cu_q.to(dev), cu_k.to(dev), Lq, 800,
                                  score_bound=bound)
    assert torch.all(ox[Lq:2 * Lq] == 0)
    _cmp(ox, O.varlen_cross_attention(qx, kvx[..., :D], kvx[..., D:], cu_q, cu_k))


@pytest.mark.parametrize("kind", ["layernorm", "rmsnorm"])
def test_query_norm_inside_the_kernel(dev, kind):
    """q_norm: the kernel takes the RAW query projection (a row-strided view, as the fused projection GEMM leaves it),
    applies the per-head norm while loading it and scales by softmax_scale * log2(e) before the one rounding to
    bf16.  Oracle: the CPU restatement of the norm (fp32) followed by the range attention; also against the
    two-launch form (magi_head_norm, then attention on pre-scaled q) to the rounding of q."""
    Lq, Hq, Hkv, D = 210, 6, 2, 128
    lens = [0, 57, 800, 64]
    g = torch.Generator().manual_seed(31)
    wide = (torch.randn(len(lens) * Lq, Hq * D + 256, generator=g) * 3 + 0.5).bfloat16()
    q_raw = wide[:, 128:128 + Hq * D].view(-1, Hq, D)  # rows 2 * (Hq * D + 256) bytes apart
    gamma = torch.randn(D, generator=g) * 0.1
    beta = torch.randn(D, generator=g) * 0.1
    k = O.rmsnorm(torch.randn(sum(lens), Hkv, D, generator=g)).bfloat16()
    v = torch.randn(sum(lens), Hkv, D, generator=g).bfloat16()
    cu_q = np.arange(0, (len(lens) + 1) * Lq, Lq)
    cu_k = np.concatenate([[0], np.cumsum(lens)])
    eps = 1e-6
    qf = q_raw.float()
    if kind == "layernorm":
        qn = torch.nn.functional.layer_norm(qf, (D,), gamma + 1, beta, eps)
        code = M.MAGI_NORM_LAYERNORM_1P
    else:
        qn = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * (gamma + 1) + beta
        code = M.MAGI_NORM_RMSNORM_1P
    ref = O.varlen_cross_attention(qn, k, v, torch.tensor(cu_q), torch.tensor(cu_k))  # fp32 q, softmax scale D^-0.5
    bound = 1.01 * PREMUL * (qn.norm(dim=-1).max() * k.float().norm(dim=-1).max()).item()
    assert bound <= M.MAGI_SCORE_BOUND_MAX
    tq, tk = _ranges(dev, cu_q, cu_k)
    out, lse = M.range_attention(q_raw.to(dev), k.to(dev), v.to(dev), tq, tk, Lq, 800, ranges_mode=M.MAGI_RANGES_CU,
                                 score_bound=bound, q_norm=(gamma.to(dev), beta.to(dev), eps, code))
    assert torch.all(out[:Lq] == 0)
    _cmp(out, ref, kind)
    if kind == "layernorm":
        # the two-launch form rounds the normalised q to bf16 BEFORE the scale is applied inside the kernel
        qh = M.head_norm(q_raw.to(dev), gamma.to(dev), beta.to(dev), eps)
        two, _ = M.range_attention(qh, k.to(dev), v.to(dev), tq, tk, Lq, 800, ranges_mode=M.MAGI_RANGES_CU)
        assert (out.float() - two.float()).abs().max().item() <= 2e-2
    with pytest.raises(M.MagiError):  # needs the bound
        M.range_attention(q_raw.to(dev), k.to(dev), v.to(dev), tq, tk, Lq, 800, ranges_mode=M.MAGI_RANGES_CU,
                          q_norm=(gamma.to(dev), beta.to(dev), eps, code))
