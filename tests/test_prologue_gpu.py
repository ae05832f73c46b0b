"""GPU parity of the fused prologue and of the module-level layer against the CPU oracle.

The prologue computes in fp32 and rounds once to bf16, like the reference; summation order
inside the norm differs from the CPU library routine, so a value that lands on a bf16 rounding
boundary may differ by one bf16 ulp.  Bar: every element within one bf16 ulp of the oracle
(absolute floor 1e-5 where the rotation cancels) and fewer than 1 in 1000 elements different at all."""
import numpy as np
import pytest
import torch

import magi_attn as M
from magi_attn import module as MOD
from magi_attn import params as P
from magi_attn import ranges as R
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu


def _cosine(a, b):
    x, y = a.detach().double().cpu().flatten(), b.detach().double().cpu().flatten()
    if x.norm() == 0 and y.norm() == 0:  # e.g. the cross attention of a batch row without text
        return 1.0
    return (torch.dot(x, y) / (x.norm() * y.norm()).clamp_min(1e-30)).item()


def _ulp_check(a, ref, what=""):
    a, ref = a.cpu(), ref.cpu()
    af, rf = a.float(), ref.float()
    # one bf16 ulp of the reference value; where the rotation cancels to ~0 the fp32 rounding of the
    # O(1) operands (~1e-6) exceeds an ulp of the tiny result, hence the absolute floor
    ulp = torch.clamp(rf.abs() * 2.0 ** -7, min=1e-5)
    assert torch.all((af - rf).abs() <= ulp), f"{what}: more than one bf16 ulp off"
    frac = (a != ref).float().mean().item()
    assert frac < 1e-3, f"{what}: {frac:.2e} of the elements differ"


def _inputs(S, Hq, Hkv, seed):
    g = torch.Generator().manual_seed(seed)
    D = 128
    qr = torch.randn(S, Hq * D, generator=g).bfloat16()
    kr = torch.randn(S, Hkv * D, generator=g).bfloat16()
    vr = torch.randn(S, Hkv * D, generator=g).bfloat16()
    par = [torch.randn(D, generator=g) * 0.2 for _ in range(4)]
    return qr, kr, vr, par


@pytest.mark.parametrize("T,H,W,sp,dn,Hq,Hkv", [(2, 4, 6, 0, 1, 6, 2), (6, 5, 7, 2, 3, 24, 8), (4, 3, 3, 1, 2, 48, 8),
                                                (2, 2, 2, 0, 2, 3, 1),
                                                # few rows per token: 8, 4 and 2 tokens share a workgroup; odd S
                                                (1, 3, 3, 0, 1, 2, 1), (3, 5, 3, 1, 1, 6, 1), (1, 7, 3, 0, 1, 8, 4)])
def test_prologue_parity(dev, T, H, W, sp, dn, Hq, Hkv):
    S, D = T * H * W, 128
    qr, kr, vr, (gq, bq, gk, bk) = _inputs(S, Hq, Hkv, seed=S + Hq)
    rope = O.rope_for_forward(T, H, W, sp, dn)
    q_ref, kv_ref = O.prologue(qr.view(S, Hq, D), kr.view(S, Hkv, D), vr.view(S, Hkv, D), rope, gq, bq, gk, bk)
    to = lambda t: t.to(dev)
    q, kv, _ = M.qk_prologue(to(qr), to(kr), to(vr), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv)
    _ulp_check(q, q_ref, "q")
    _ulp_check(kv[..., :D], kv_ref[..., :D], "k")
    assert torch.equal(kv[..., D:].cpu(), kv_ref[..., D:])  # V is a copy: bit exact


def _e4m3_check(got, ref, what=""):
    """got / ref float8_e4m3fn: equal but for values on a rounding boundary, which the different summation order of
    the fp32 norm may push to the neighbouring code (bar: the neighbour at most, fewer than 2 in 1000 elements)."""
    gb, rb = got.cpu().view(torch.uint8).int(), ref.cpu().view(torch.uint8).int()
    assert gb.shape == rb.shape
    if gb.numel() == 0:
        return
    diff = gb != rb
    assert diff.float().mean().item() < 2e-3, f"{what}: {diff.float().mean().item():.2e} of the elements differ"
    # neighbouring codes: same sign and magnitude codes one apart, or +-0 against the smallest subnormal
    mag_g, mag_r = gb & 0x7f, rb & 0x7f
    near = ((gb & 0x80) == (rb & 0x80)) & ((mag_g - mag_r).abs() <= 1) | ((mag_g + mag_r) <= 1)
    assert torch.all(near | ~diff), f"{what}: more than one e4m3 code off"


@pytest.mark.parametrize("T,H,W,sp,dn,Hq,Hkv,keep", [(2, 4, 6, 0, 2, 6, 2, 1), (6, 5, 7, 2, 3, 24, 8, 3), (4, 3, 3, 1, 2, 48, 8, 0),
                                                     (1, 3, 3, 0, 1, 2, 1, 1), (3, 5, 3, 1, 3, 6, 1, 2)])
def test_prologue_e4m3_outputs(dev, T, H, W, sp, dn, Hq, Hkv, keep):
    """out_dtype e4m3: q and k leave the norm + rotary pass quantised with constant power-of-two scales, K straight
    into the rows of an fp8 cache (first `keep` chunks) and a side buffer (the rest).  Expected values: the
    oracle's prologue stopped ahead of its downcast, through the oracle's saturating e4m3 quantiser.  The scales
    come from the norm-parameter bound (nothing saturates); a second run with a scale 64 times too small checks
    the saturation to +-448."""
    import math

    S, D = T * H * W, 128
    L = S // dn
    cs = D ** -0.5 * math.log2(math.e)
    qr, kr, vr, (gq, bq, gk, bk) = _inputs(S, Hq, Hkv, seed=S + Hq + 1)
    rope = O.rope_for_forward(T, H, W, sp, dn)
    q_f, k_f = O.prologue(qr.view(S, Hq, D), kr.view(S, Hkv, D), vr.view(S, Hkv, D), rope, gq, bq, gk, bk, q_premul=cs,
                          downcast=False)
    bound = lambda g, b: math.sqrt(D) * (g + 1).abs().max().item() + b.norm().item()
    to = lambda t: t.to(dev)
    for shrink in (1.0, 64.0):
        qs = M.pow2_scale_for(cs * bound(gq, bq)) / shrink
        ks = M.pow2_scale_for(bound(gk, bk)) / shrink
        if shrink == 1.0:
            assert (q_f.abs().max() / qs <= 448) and (k_f.abs().max() / ks <= 448)
        cache_k = torch.zeros(S + 5, Hkv, D, device=dev).to(torch.float8_e4m3fn)
        side = torch.zeros(S, Hkv, D, device=dev).to(torch.float8_e4m3fn)
        n_keep = keep * L
        q8, k_out, k_tail = M.qk_prologue_fp8(to(qr), to(kr), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv,
                                              q_scale=qs, k_scale=ks, q_premul=cs, k_out=cache_k[5:], n_cache_rows=n_keep,
                                              k_tail=side)
        q_ref = O.quantize_e4m3(q_f, torch.tensor(qs))
        k_ref = O.quantize_e4m3(k_f, torch.tensor(ks))
        _e4m3_check(q8, q_ref, "q")
        _e4m3_check(cache_k[5:5 + n_keep], k_ref[:n_keep], "k (cache rows)")
        _e4m3_check(side[:S - n_keep], k_ref[n_keep:], "k (side rows)")
        assert torch.all(cache_k[:5].float() == 0) and torch.all(cache_k[5 + n_keep:].float() == 0)
        assert torch.all(side[S - n_keep:].float() == 0)
        assert not torch.isnan(q8.float()).any() and not torch.isnan(cache_k.float()).any()
        if shrink > 1.0:
            assert q8.float().abs().max() == 448
    # fresh outputs, strided raw rows (views of one projection result), no rotary, RMS norm
    big = torch.randn(S, (Hq + 2 * Hkv) * D + 64, generator=torch.Generator().manual_seed(5)).bfloat16().to(dev)
    qv, kv_ = big[:, :Hq * D], big[:, Hq * D:(Hq + Hkv) * D]
    q8, k8, _ = M.qk_prologue_fp8(qv, kv_, None, to(gq), None, to(gk), None, Hq=Hq, Hkv=Hkv, q_scale=2.0 ** -4,
                                  k_scale=2.0 ** -5, norm_kind=M.MAGI_NORM_RMSNORM_1P)
    qn = O.rmsnorm(qv.cpu().view(S, Hq, D).float(), gq + 1)
    kn = O.rmsnorm(kv_.cpu().view(S, Hkv, D).float(), gk + 1)
    _e4m3_check(q8, O.quantize_e4m3(qn, torch.tensor(2.0 ** -4)), "q rms")
    _e4m3_check(k8, O.quantize_e4m3(kn, torch.tensor(2.0 ** -5)), "k rms")
    with pytest.raises(M.MagiError):
        M.qk_prologue_fp8(qv, kv_, None, to(gq), None, to(gk), None, Hq=Hq, Hkv=Hkv, q_scale=0.0, k_scale=1.0)


def test_prologue_folds_a_factor_into_q_ahead_of_the_rounding(dev):
    """q_premul (softmax_scale * log2(e) for the pre-scaled attention path): applied in fp32 after norm and rotary,
    so q is rounded to bf16 once; K and V are untouched.  End to end: prologue with the factor + attention with
    q_prescaled against the oracle's unscaled prologue + attention."""
    import math

    T, H, W, sp, dn, Hq, Hkv = 4, 5, 6, 1, 2, 6, 2
    S, D = T * H * W, 128
    L = S // dn
    cs = D ** -0.5 * math.log2(math.e)
    qr, kr, vr, (gq, bq, gk, bk) = _inputs(S, Hq, Hkv, seed=99)
    rope = O.rope_for_forward(T, H, W, sp, dn)
    shaped = (qr.view(S, Hq, D), kr.view(S, Hkv, D), vr.view(S, Hkv, D), rope, gq, bq, gk, bk)
    q_ref, kv_ref = O.prologue(*shaped, q_premul=cs)
    q_plain, _ = O.prologue(*shaped)
    to = lambda t: t.to(dev)
    q, kv, _ = M.qk_prologue(to(qr), to(kr), to(vr), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv, q_premul=cs)
    _ulp_check(q, q_ref, "q * premul")
    _ulp_check(kv[..., :D], kv_ref[..., :D], "k")
    assert torch.equal(kv[..., D:].cpu(), kv_ref[..., D:])
    ranges = [[0, L], [L, S]], [[0, L], [0, S]]
    tq, tk = (torch.tensor(r, dtype=torch.int32, device=dev) for r in ranges)
    out, _ = M.range_attention(q, kv[..., :D], kv[..., D:], tq, tk, L, q_prescaled=True, return_lse=False)
    ref = O.range_attention(q_plain, kv_ref[..., :D], kv_ref[..., D:], *ranges)
    assert (out.float().cpu() - ref).abs().max() <= 2e-2


def test_prologue_rmsnorm_no_rope_and_strided_inputs(dev):
    S, Hq, Hkv, D = 50, 6, 2, 128
    qr, kr, vr, (gq, bq, gk, bk) = _inputs(S, Hq, Hkv, seed=3)
    z = torch.zeros(D)
    # one fused projection output [S, (Hq + 2 Hkv) * D] sliced into q / k / v column blocks
    fused = torch.cat([qr, kr, vr], 1).to(dev)
    qv, kv_, vv = fused[:, : Hq * D], fused[:, Hq * D:(Hq + Hkv) * D], fused[:, (Hq + Hkv) * D:]
    q, kv, _ = M.qk_prologue(qv, kv_, vv, None, gq.to(dev), None, gk.to(dev), None, Hq=Hq, Hkv=Hkv,
                             norm_kind=M.MAGI_NORM_RMSNORM_1P)
    q_ref = O.rmsnorm(qr.view(S, Hq, D).float(), gq + 1).bfloat16()
    k_ref = O.rmsnorm(kr.view(S, Hkv, D).float(), gk + 1).bfloat16()
    _ulp_check(q, q_ref, "q rms")
    _ulp_check(kv[..., :D], k_ref, "k rms")
    q2, _, _ = M.qk_prologue(qv, kv_, vv, None, None, None, None, None, Hq=Hq, Hkv=Hkv, norm_kind=M.MAGI_NORM_NONE)
    assert torch.equal(q2.cpu(), qr.view(S, Hq, D))


def test_prologue_writes_cache_in_place_and_tail(dev):
    S, Hq, Hkv, D = 40, 3, 2, 128
    qr, kr, vr, (gq, bq, gk, bk) = _inputs(S, Hq, Hkv, seed=4)
    rope = O.rope_table(1, 5, 8)
    _, kv_ref = O.prologue(qr.view(S, Hq, D), kr.view(S, Hkv, D), vr.view(S, Hkv, D), rope, gq, bq, gk, bk)
    to = lambda t: t.to(dev)
    cache = torch.full((100, Hkv, 2 * D), 7.0, dtype=torch.bfloat16, device=dev)
    tail = torch.full((20, Hkv, 2 * D), 9.0, dtype=torch.bfloat16, device=dev)
    start, keep = 30, 25
    M.qk_prologue(to(qr), to(kr), to(vr), to(rope), to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv,
                  kv_out=cache[start:], n_cache_rows=keep, kv_tail=tail)
    assert torch.all(cache[:start] == 7) and torch.all(cache[start + keep:] == 7)  # nothing else touched
    _ulp_check(cache[start:start + keep], kv_ref[:keep], "cache rows")
    _ulp_check(tail[: S - keep], kv_ref[keep:], "tail rows")
    assert torch.all(tail[S - keep:] == 9)


def test_head_norm_matches_bf16_layernorm(dev):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(33, 5, 256, generator=g).bfloat16()
    w = (torch.randn(128, generator=g) * 0.1).bfloat16()
    b = (torch.randn(128, generator=g) * 0.1).bfloat16()
    ln = MOD.FusedLayerNorm(128, dtype=torch.bfloat16)
    ln.weight.data.copy_(w)
    ln.bias.data.copy_(b)
    gg, bb = ln.gamma_beta_fp32()
    y = M.head_norm(x.to(dev)[..., :128], gg.to(dev), bb.to(dev))  # strided K half of an interleaved KV
    ref = torch.nn.functional.layer_norm(x[..., :128], (128,), w + 1, b, 1e-6)  # what the reference calls in bf16
    _ulp_check(y, ref, "xattn norm")


# ----------------------------------------------------------------------------- the layer
def _make_layer(dev, hidden, Hq, Hkv, seed):
    torch.manual_seed(seed)
    layer = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=3, device=dev)
    with torch.no_grad():
        for p in layer.parameters():
            if p.dim() == 1:
                p.copy_(torch.randn_like(p.float()) * 0.1)
            else:
                p.copy_(torch.randn_like(p.float()) * hidden ** -0.5)
        layer.linear_qkv.layer_norm.weight.add_(1.0)
    return layer


def _oracle_layer(layer, hidden_states, y, rope, sp, L, k_range, q_range, cache, update, distill, extra, cu_q, cu_k,
                  has_ip=True):
    """The reference's forward (dit_module.py:1138-1173) restated with the oracle pieces, on CPU."""
    D = 128
    cpu = lambda t: t.detach().cpu()
    lq = layer.linear_qkv
    mixed = torch.nn.functional.layer_norm(hidden_states, (hidden_states.shape[-1],), cpu(lq.layer_norm.weight),
                                           cpu(lq.layer_norm.bias), 1e-6)
    S = mixed.shape[0]
    lin = lambda m: torch.nn.functional.linear(mixed[:, 0], cpu(m.weight))
    Hq, Hkv = layer.num_attention_heads, layer.num_query_groups_per_partition
    q_raw, k_raw, v_raw, qx_raw = lin(lq.q), lin(lq.k), lin(lq.v), lin(lq.qx)
    q, kv = O.prologue(q_raw.view(S, Hq, D), k_raw.view(S, Hkv, D), v_raw.view(S, Hkv, D), rope,
                       cpu(layer.q_layernorm.weight), cpu(layer.q_layernorm.bias), cpu(layer.k_layernorm.weight),
                       cpu(layer.k_layernorm.bias))
    k, v = cache.adjust(kv, has_inference_params=has_ip, update_kv_cache=update, slice_point=sp, clip_token_nums=L,
                        fwd_extra_1st_chunk=extra, distill_nearly_clean_chunk=distill)
    core = O.range_attention(q, k, v, q_range, k_range).bfloat16()
    qx = torch.nn.functional.layer_norm(qx_raw.view(S, Hq, D), (D,), cpu(layer.q_layernorm_xattn.weight) + 1,
                                        cpu(layer.q_layernorm_xattn.bias), 1e-6)
    kvx = torch.nn.functional.linear(y, cpu(layer.linear_kv_xattn.weight)).view(y.shape[0], Hkv, 2 * D)
    kx = torch.nn.functional.layer_norm(kvx[..., :D], (D,), cpu(layer.k_layernorm_xattn.weight) + 1,
                                        cpu(layer.k_layernorm_xattn.bias), 1e-6)
    xo = O.varlen_cross_attention(qx, kx, kvx[..., D:], cu_q, cu_k).bfloat16()
    return core.reshape(S, 1, -1), xo.reshape(S, 1, -1)


def test_layer_forward_sequence_with_kv_cache(dev):
    """A short generation schedule (clean-chunk extraction, cached denoising with and without cache
    update, nearly-clean distillation, a cache-less pass) through the layer, compared step by
    step with the oracle's layer and with the oracle's cache contents."""
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    n_chunks = 6
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=0)
    rope_mod = M.rope.LearnableRotaryEmbeddingCat(128, device=dev) if hasattr(M, "rope") else None
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip = P.InferenceParams(1, n_chunks * L)
    cache_ref = O.KVCacheModel(n_chunks * L, Hkv, D)
    g = torch.Generator().manual_seed(1)
    #        sp dn update distill extra has_ip
    steps = [(0, 2, True, False, True, True),
             (0, 3, True, True, True, True),
             (2, 3, False, False, False, True),
             (2, 3, True, False, False, True),
             (1, 4, True, True, True, True),
             (3, 3, False, False, True, True),
             (0, 2, False, False, False, False)]
    for sp, dn, update, distill, extra, has_ip in steps:
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16()
        lens = torch.randint(0, 9, (dn,), generator=g)
        mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
        y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16()
        k_range = R.generate_default_kvrange(sp, dn, L) if has_ip else R.generate_kv_range_for_uncondition(dn, L)
        q_range = R.q_ranges_from_chunks(dn, L)
        core_p = P.build_core_attn_params(q_range.to(dev), k_range.to(dev), L)
        cross_p = P.build_cross_attn_params(mask.to(dev), L, 8)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=extra,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=core_p, cross_attn_params=cross_p)
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        ip.update_kv_cache = update
        with torch.no_grad():
            core, xo = layer(hs.to(dev), y.to(dev), ip if has_ip else None, rope, meta)
        assert core.shape == (S, 1, Hq * D) and xo.shape == (S, 1, Hq * D)
        core_ref, xo_ref = _oracle_layer(layer, hs, y, O.rope_for_forward(dn * fr, H, W, sp, dn), sp, L,
                                         k_range.numpy(), q_range.numpy(), cache_ref, update, distill, extra,
                                         cross_p.cu_seqlens_q.cpu(), cross_p.cu_seqlens_kv.cpu(), has_ip)
        for a, b, nm in ((core, core_ref, "core"), (xo, xo_ref, "xattn")):
            err = (a.float().cpu() - b.float()).abs().max().item()
            assert err <= 2e-2, f"step {(sp, dn, update, distill, extra)} {nm}: {err}"
            assert _cosine(a, b) >= 0.9999, f"step {(sp, dn, update, distill, extra)} {nm}: cosine {_cosine(a, b)}"
        # what the cache holds afterwards must be what the reference's cache would hold
        if has_ip and (extra or sp > 0) and update:
            keep = S - L if distill else S
            got = ip.key_value_memory_dict[3][sp * L: sp * L + keep].float().cpu()
            want = cache_ref.mem[sp * L: sp * L + keep].float()
            # (the two sides' projections come from different GEMM implementations, which may round a raw value to
            # the other neighbour: within 2^-6 of the row's largest magnitude, K and V halves apart)
            for half in (slice(0, D), slice(D, 2 * D)):
                d = (got[..., half] - want[..., half]).abs()
                assert torch.all(d <= want[..., half].abs().amax(dim=-1, keepdim=True) * 2.0 ** -6)


def test_reference_forward_written_out_method_by_method(dev):
    """The body of the reference's forward for cp_strategy "none" (dit_module.py:1166-1171), typed out with this
    module's methods of the same names: get_kv, get_q, adjust_key_and_value_for_inference, core_attention,
    cross_attention with get_xqkv.  This is the path a maintainer gets who swaps the class in but keeps a forward of
    their own; q stays unscaled here and nothing is appended in place.  Step by step against the oracle's layer and
    cache, and close to what this module's own forward returns (which pre-scales q: another rounding)."""
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    n_chunks = 6
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=17)
    twin = _make_layer(dev, hidden, Hq, Hkv, seed=17)          # same weights: runs the module's own forward
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip, ip_twin = P.InferenceParams(1, n_chunks * L), P.InferenceParams(1, n_chunks * L)
    cache_ref = O.KVCacheModel(n_chunks * L, Hkv, D)
    g = torch.Generator().manual_seed(3)
    #        sp dn update distill extra has_ip
    steps = [(0, 2, True, False, True, True), (2, 3, False, False, False, True), (2, 3, True, True, False, True),
             (4, 2, True, False, False, True), (0, 2, False, False, False, False)]
    for sp, dn, update, distill, extra, has_ip in steps:
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16()
        lens = torch.randint(0, 9, (dn,), generator=g)
        mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
        y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16()
        k_range = R.generate_default_kvrange(sp, dn, L) if has_ip else R.generate_kv_range_for_uncondition(dn, L)
        q_range = R.q_ranges_from_chunks(dn, L)
        cross_p = P.build_cross_attn_params(mask.to(dev), L, 8)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=extra,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(q_range.to(dev), k_range.to(dev), L),
                               cross_attn_params=cross_p)
        rotary_pos_emb = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        ip.update_kv_cache = ip_twin.update_kv_cache = update
        params = ip if has_ip else None
        with torch.no_grad():
            # ---- dit_module.py:1146-1171, line for line in meaning ----
            sin_emb, cos_emb = rotary_pos_emb.tensor_split(2, -1)
            batch_size = hs.shape[1]
            mixed_qqkv = layer.linear_qkv.forward_ln(hs.to(dev))
            key_and_value = layer.get_kv(mixed_qqkv, cos_emb, sin_emb)
            query = layer.get_q(mixed_qqkv, cos_emb, sin_emb)
            key, value = layer.adjust_key_and_value_for_inference(key_and_value, params, meta)
            core_attn_out = layer.core_attention(query, key, value, batch_size, meta)
            core_attn_out = core_attn_out.reshape(S, batch_size, Hq * D)       # "(sq b) hn hd -> sq b (hn hd)"
            xattn_out = layer.cross_attention(mixed_qqkv, y.to(dev), meta.cross_attn_params, layer.get_xqkv)
            own_core, own_x = twin(hs.to(dev), y.to(dev), ip_twin if has_ip else None, rotary_pos_emb, meta)
        assert query.shape == (S, Hq, D) and key_and_value.shape == (S, Hkv, 2 * D) and xattn_out.shape == (S, 1, Hq * D)
        core_ref, xo_ref = _oracle_layer(layer, hs, y, O.rope_for_forward(dn * fr, H, W, sp, dn), sp, L,
                                         k_range.numpy(), q_range.numpy(), cache_ref, update, distill, extra,
                                         cross_p.cu_seqlens_q.cpu(), cross_p.cu_seqlens_kv.cpu(), has_ip)
        for a, b, nm in ((core_attn_out, core_ref, "core"), (xattn_out, xo_ref, "xattn")):
            err = (a.float().cpu() - b.float()).abs().max().item()
            assert err <= 2e-2 and _cosine(a, b) >= 0.9999, f"step {(sp, dn, update, distill, extra)} {nm}: {err}"
        assert (core_attn_out.float() - own_core.float()).abs().max().item() <= 2e-2
        assert (xattn_out.float() - own_x.float()).abs().max().item() <= 2e-2
        if has_ip and (extra or sp > 0) and update:
            keep = S - L if distill else S
            rows = slice(sp * L, sp * L + keep)
            assert torch.equal(ip.key_value_memory_dict[3][rows], ip_twin.key_value_memory_dict[3][rows])  # same prologue
            got, want = ip.key_value_memory_dict[3][rows].float().cpu(), cache_ref.mem[rows].float()
            for half in (slice(0, D), slice(D, 2 * D)):
                d = (got[..., half] - want[..., half]).abs()
                assert torch.all(d <= want[..., half].abs().amax(dim=-1, keepdim=True) * 2.0 ** -6)
    # full_attention (dit_module.py:1068-1096): range i on its own gives range i's rows of core_attention
    with torch.no_grad():
        for i in range(dn):
            rows = slice(i * L, (i + 1) * L)
            o_i = layer.full_attention(1, meta, query[rows], key, value, i)
            assert torch.equal(o_i, core_attn_out.view(S, Hq, D)[rows]), i
    # get_qkv: the three pieces of the same prologue
    with torch.no_grad():
        q3, k3, v3 = layer.get_qkv(mixed_qqkv, cos_emb, sin_emb)
    assert torch.equal(q3, query) and torch.equal(k3, key_and_value[..., :D]) and torch.equal(v3, key_and_value[..., D:])


@pytest.mark.parametrize("proj_layout", [False, True])
def test_whole_layer_forward_captured_in_a_graph(dev, proj_layout):
    """The reference's enable_cuda_graph case at the level of the layer: one FullyParallelAttention.forward on the
    cached path (input LayerNorm, the projection GEMM, prologue with its in-place cache append, core attention over
    cache prefix + new rows, text projection, head norm, cross attention) captured into a HIP graph.  Replays on new
    hidden states and text states, with eager forwards in between, equal the eager results bit for bit."""
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    hidden, Hq, Hkv, D = 256, 8, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=23)
    sp, dn = 2, 2
    S = dn * L
    g = torch.Generator().manual_seed(5)
    hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
    y = (torch.randn(dn * 8, hidden, generator=g) * 0.5).bfloat16().to(dev)
    meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                           range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=True,
                           distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=True,
                           core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                     R.generate_default_kvrange(sp, dn, L).to(dev), L),
                           cross_attn_params=P.build_cross_attn_params(torch.ones(dn, 1, 1, 8).to(dev), L, 8))
    rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, sp, dn)
    ip = P.InferenceParams(1, 6 * L)
    ip.update_kv_cache = True
    ip.key_value_memory_dict[3] = torch.randn(6 * L, Hkv, 2 * D, generator=g).bfloat16().to(dev)
    run = lambda: layer(hs, y, ip, rope, meta, proj_layout=proj_layout)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run()  # warm-up outside the capture (norm-parameter caches, side buffers, GEMM workspaces)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = run()
        captured = captured if isinstance(captured, tuple) else (captured,)
        for rep in range(3):
            hs.copy_(torch.randn(S, 1, hidden, generator=g).bfloat16())
            y.copy_((torch.randn(dn * 8, hidden, generator=g) * 0.5).bfloat16())
            eager = run()
            eager = eager if isinstance(eager, tuple) else (eager,)
            rows = ip.key_value_memory_dict[3][sp * L:(sp + dn) * L].clone()
            torch.cuda.synchronize()
            for t in captured:
                t.fill_(7)
            ip.key_value_memory_dict[3][sp * L:(sp + dn) * L].zero_()
            graph.replay()
            torch.cuda.synchronize()
            for a, b in zip(captured, eager):
                assert torch.equal(a, b), f"replay {rep}"
            assert torch.equal(ip.key_value_memory_dict[3][sp * L:(sp + dn) * L], rows)  # the append is replayed too


def _cacheless_forward_vs_oracle(layer, dev, seed, tol=2e-2):
    """One cache-less batch-1 forward of two chunks (one of them without text) against the oracle's layer."""
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden = layer.linear_qkv.q.weight.shape[1]
    Hq, Hkv, D = layer.num_attention_heads, layer.num_query_groups_per_partition, 128
    fr, H, W, dn = 2, 3, 4, 2
    L = fr * H * W
    S = dn * L
    g = torch.Generator().manual_seed(seed)
    hs = torch.randn(S, 1, hidden, generator=g).bfloat16()
    lens = torch.tensor([7, 0])
    mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
    y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16()
    k_range, q_range = R.generate_kv_range_for_uncondition(dn, L), R.q_ranges_from_chunks(dn, L)
    cross_p = P.build_cross_attn_params(mask.to(dev), L, 8)
    meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=0, denoising_range_num=dn,
                           range_num=dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=False,
                           distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                           core_attn_params=P.build_core_attn_params(q_range.to(dev), k_range.to(dev), L),
                           cross_attn_params=cross_p)
    rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, 0, dn)
    with torch.no_grad():
        core, xo = layer(hs.to(dev), y.to(dev), None, rope, meta)
    core_ref, xo_ref = _oracle_layer(layer, hs, y, O.rope_for_forward(dn * fr, H, W, 0, dn), 0, L, k_range.numpy(),
                                     q_range.numpy(), O.KVCacheModel(S, Hkv, D), False, False, False,
                                     cross_p.cu_seqlens_q.cpu(), cross_p.cu_seqlens_kv.cpu(), has_ip=False)
    for a, b, nm in ((core, core_ref, "core"), (xo, xo_ref, "xattn")):
        assert torch.isfinite(a).all(), nm
        d = (a.float().cpu() - b.float()).abs()
        # (max-abs bar, or one bf16 ulp of the value where that is larger: outputs of magnitude 4 and more)
        assert torch.all(d <= torch.clamp(b.float().abs() * 2.0 ** -7, min=tol)), (nm, d.max().item())
        assert _cosine(a, b) >= 0.9999, (nm, _cosine(a, b))


def test_layer_follows_rewritten_norm_parameters_and_falls_back_above_the_bound(dev):
    """The score bounds (a promise to kernels that keep no running maximum) and the constant e4m3 scales are derived
    from the norm parameters and cached: after a parameter is rewritten, by copy_, by load_state_dict (in place and
    with assign=True, the reference loader's form, inference/infra/checkpoint/checkpointing.py:168) or through .data
    followed by invalidate_cached_parameters(), they must follow, and the forward must still match the oracle.
    Gains that push a bound past MAGI_SCORE_BOUND_MAX make the layer fall back to the online-softmax kernel (and the
    cross attention to its two-launch form); last_forward_kernels records the choice."""
    import math

    hidden, Hq, Hkv, D = 256, 6, 2, 128
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=21)
    premul = D ** -0.5 * math.log2(math.e)

    def expected(rotary_half=48):
        b = lambda qn, kn, r: 1.01 * premul * MOD.qk_score_bound(qn, kn, r)
        sc = (M.pow2_scale_for(premul * layer.q_layernorm.output_norm_bound()), M.pow2_scale_for(layer.k_layernorm.output_norm_bound()))
        for ln in (layer.q_layernorm, layer.k_layernorm, layer.q_layernorm_xattn, layer.k_layernorm_xattn):
            ln.invalidate_cached_parameters()  # (recomputed from the parameters as they are now)
        return (b(layer.q_layernorm, layer.k_layernorm, rotary_half), b(layer.q_layernorm_xattn, layer.k_layernorm_xattn, 0)), sc

    _cacheless_forward_vs_oracle(layer, dev, 1)
    b0, s0 = layer.score_bounds(), layer.fp8_operand_scales()
    assert max(b0) <= M.MAGI_SCORE_BOUND_MAX and "bounded" in layer.last_forward_kernels["core"]
    assert "bounded" in layer.last_forward_kernels["cross"]
    g = torch.Generator().manual_seed(5)
    # 1. in-place copy_ under no_grad (advances the version counter)
    with torch.no_grad():
        layer.q_layernorm.weight.copy_(torch.randn(D, generator=g) * 0.4)
    b1, s1 = layer.score_bounds(), layer.fp8_operand_scales()
    assert b1[0] != b0[0] and b1[1] == b0[1]
    _cacheless_forward_vs_oracle(layer, dev, 2)
    want_b, want_s = expected()
    assert b1 == pytest.approx(want_b) and s1 == want_s
    # 2. a write through .data is invisible to the version counter: the caller invalidates
    layer.k_layernorm.weight.data.copy_(torch.randn(D, generator=g) * 0.4)
    layer.k_layernorm.bias.data.copy_(torch.randn(D, generator=g) * 0.5)
    layer.invalidate_cached_parameters()
    b2, s2 = layer.score_bounds(), layer.fp8_operand_scales()
    want_b, want_s = expected()
    assert b2 == pytest.approx(want_b) and s2 == want_s and b2[0] != b1[0]
    _cacheless_forward_vs_oracle(layer, dev, 3)
    # 3. load_state_dict in place, then with assign=True (new Parameter objects): large gains, bound above the limit
    sd = {k_: v_.clone() for k_, v_ in layer.state_dict().items()}
    sd["q_layernorm.weight"] = torch.full((D,), 1.0, device=dev)         # gamma + 1 = 2: scores four times as large
    sd["k_layernorm.weight"] = torch.full((D,), 1.0, device=dev)
    layer.load_state_dict(sd)
    b3 = layer.score_bounds()
    assert b3[0] > M.MAGI_SCORE_BOUND_MAX and b3 == pytest.approx(expected()[0])
    # (the scores are four times as large, and with them the effect of q's and k's rounding to bf16, which the layer
    # and the oracle do at different points: q after / before the softmax scale; the softmax is sharp, so outputs
    # are close to single V rows of magnitude 2-4, where two bf16 ulps are 0.031)
    _cacheless_forward_vs_oracle(layer, dev, 4, tol=4e-2)
    assert "online" in layer.last_forward_kernels["core"] and "bounded" in layer.last_forward_kernels["cross"]
    sd = {k_: v_.clone() for k_, v_ in layer.state_dict().items()}
    sd["q_layernorm.weight"] = torch.randn(D, generator=g).to(dev) * 0.1
    sd["k_layernorm.weight"] = torch.randn(D, generator=g).to(dev) * 0.1
    sd["q_layernorm_xattn.weight"] = torch.full((D,), 1.0, device=dev, dtype=torch.bfloat16)
    sd["k_layernorm_xattn.weight"] = torch.full((D,), 1.0, device=dev, dtype=torch.bfloat16)
    layer.load_state_dict(sd, assign=True)
    b4 = layer.score_bounds()
    assert b4[0] <= M.MAGI_SCORE_BOUND_MAX < b4[1] and b4 == pytest.approx(expected()[0])
    assert layer.fp8_operand_scales() == expected()[1]
    _cacheless_forward_vs_oracle(layer, dev, 5, tol=4e-2)
    assert "bounded" in layer.last_forward_kernels["core"] and "online" in layer.last_forward_kernels["cross"]


def test_layer_measures_the_bound_when_the_parameter_bound_is_too_loose(dev):
    """Gains that vary across features: the bound that follows from the norm parameters takes the largest gain for
    every element (here 3 on one feature of q and of k: 148, far above MAGI_SCORE_BOUND_MAX), the rows themselves are
    hardly longer than with unit gains (measured bound about 30).  With measure_bound_above_limit the core attention measures max|q| max|k| and
    the bounded-score kernel runs after all: same launches as a call with a stated bound (2 passes + 2 kernels more
    than the plain launch), parity with the oracle.  With uniform gains of 2 the measured bound (66) is above the
    limit too and the online-softmax kernel runs behind the measurement: bit-identical to the forward without it."""
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=13)
    sd = {k_: v_.clone() for k_, v_ in layer.state_dict().items()}
    for nm in ("q_layernorm", "k_layernorm"):
        w = torch.zeros(D, device=dev)
        w[5] = 2.0
        sd[nm + ".weight"], sd[nm + ".bias"] = w, torch.zeros(D, device=dev)
    layer.load_state_dict(sd)
    assert layer.score_bounds()[0] > 2 * M.MAGI_SCORE_BOUND_MAX
    assert layer.measure_bound_above_limit is None     # (the passes do not pay on a launch this small: plain launch)
    _cacheless_forward_vs_oracle(layer, dev, 6, tol=4e-2)
    assert "online" in layer.last_forward_kernels["core"]
    layer.measure_bound_above_limit = True
    before = MOD.L.lib().magi_launch_count()
    _cacheless_forward_vs_oracle(layer, dev, 6, tol=4e-2)
    with_measurement = MOD.L.lib().magi_launch_count() - before
    assert "measured" in layer.last_forward_kernels["core"]
    layer.measure_bound_above_limit = False
    before = MOD.L.lib().magi_launch_count()
    _cacheless_forward_vs_oracle(layer, dev, 6, tol=4e-2)
    assert with_measurement == MOD.L.lib().magi_launch_count() - before + 4
    # uniform gains of 2: measured 66 > 64, so the measurement ends in the online-softmax kernel
    sd["q_layernorm.weight"] = torch.full((D,), 1.0, device=dev)
    sd["k_layernorm.weight"] = torch.full((D,), 1.0, device=dev)
    layer.load_state_dict(sd)
    outs = []
    for flag in (False, True):
        layer.measure_bound_above_limit = flag
        from magi_attn.rope import LearnableRotaryEmbeddingCat
        g = torch.Generator().manual_seed(2)
        fr, H, W, dn = 2, 3, 4, 2
        L_ = fr * H * W
        hs = torch.randn(dn * L_, 1, hidden, generator=g).bfloat16().to(dev)
        y = (torch.randn(8, hidden, generator=g) * 0.5).bfloat16().to(dev)
        mask = torch.tensor([[1.0] * 8, [0.0] * 8]).view(dn, 1, 1, 8)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=0, denoising_range_num=dn,
                               range_num=dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=False,
                               distill_nearly_clean_chunk=False, clip_token_nums=L_, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L_).to(dev),
                                                                         R.generate_kv_range_for_uncondition(dn, L_).to(dev), L_),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L_, 8))
        rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, 0, dn)
        with torch.no_grad():
            outs.append(layer(hs, y, None, rope, meta)[0])
    assert torch.equal(outs[0], outs[1])


def test_layer_batched_cacheless_pass(dev):
    """The unconditional pass of classifier-free guidance: chunks become batch rows, tokens are
    ordered (position, batch), every row attends to itself only, no cache."""
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W, B = 2, 3, 4, 3
    L = fr * H * W
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=2)
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(fr, H, W, 0, 1)
    g = torch.Generator().manual_seed(3)
    hs = torch.randn(L, B, hidden, generator=g).bfloat16()
    lens = torch.tensor([3, 0, 8])
    mask = (torch.arange(8)[None] < lens[:, None]).float().view(B, 1, 1, 8)
    y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16()
    k_range = R.generate_kv_range_for_uncondition(B, L)
    core_p = P.build_core_attn_params(k_range.to(dev), k_range.to(dev), L)
    cross_p = P.build_cross_attn_params(mask.to(dev), L, 8)
    meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=0, denoising_range_num=1,
                           range_num=1, extract_prefix_video_feature=False, fwd_extra_1st_chunk=False,
                           distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                           core_attn_params=core_p, cross_attn_params=cross_p)
    with torch.no_grad():
        core, xo = layer(hs.to(dev), y.to(dev), None, rope, meta)
    assert core.shape == (L, B, Hq * D)
    cu_k = cross_p.cu_seqlens_kv.cpu()
    for b in range(B):  # each batch row == a batch-1 forward of that row
        cache_ref = O.KVCacheModel(L, Hkv, D)
        yb = y[cu_k[b]:cu_k[b + 1]]
        c_ref, x_ref = _oracle_layer(layer, hs[:, b:b + 1], yb, O.rope_for_forward(fr, H, W, 0, 1), 0, L,
                                     np.array([[0, L]]), np.array([[0, L]]), cache_ref, False, False, False,
                                     torch.tensor([0, L]), torch.tensor([0, int(lens[b])]), has_ip=False)
        assert (core[:, b].float().cpu() - c_ref[:, 0].float()).abs().max() <= 3e-2
        assert (xo[:, b].float().cpu() - x_ref[:, 0].float()).abs().max() <= 3e-2
        assert _cosine(core[:, b], c_ref[:, 0]) >= 0.9999 and _cosine(xo[:, b], x_ref[:, 0]) >= 0.9999


def test_layer_output_in_linear_proj_layout(dev):
    """proj_layout=True: both attention launches write into the "(hn n hd)" buffer that linear_proj consumes
    (dit_module.py:1336-1339).  Same kernels, other store addresses: bit-identical to re-ordering the two
    separate outputs, with and without the KV cache, and through the torch fallback at batch > 1."""
    hidden, Hq, Hkv, D = 256, 16, 8, 128
    fr, H, W = 1, 3, 5
    L = fr * H * W
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=5)
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    g = torch.Generator().manual_seed(6)
    ip = P.InferenceParams(1, 4 * L)
    ip.update_kv_cache = True
    for sp, dn, has_ip in ((0, 2, True), (2, 2, True), (0, 2, False)):
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
        lens = torch.tensor([5, 0][:dn])
        mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
        y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16().to(dev)
        k_range = R.generate_default_kvrange(sp, dn, L) if has_ip else R.generate_kv_range_for_uncondition(dn, L)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=True,
                               distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                         k_range.to(dev), L),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        with torch.no_grad():
            core, xo = layer(hs, y, ip if has_ip else None, rope, meta)
            fused = layer(hs, y, ip if has_ip else None, rope, meta, proj_layout=True)
        assert fused.shape == (S, 1, 2 * Hq * D)
        assert torch.equal(fused.cpu(), O.attn_linear_proj_input(core.cpu(), xo.cpu()))
        assert torch.count_nonzero(xo[L:]).item() == 0  # the chunk without text
    # batch > 1: no single-stride destination exists, the module re-orders with torch
    B = 2
    hs = torch.randn(L, B, hidden, generator=g).bfloat16().to(dev)
    lens = torch.tensor([4, 8])
    mask = (torch.arange(8)[None] < lens[:, None]).float().view(B, 1, 1, 8)
    y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16().to(dev)
    kr = R.generate_kv_range_for_uncondition(B, L)
    meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=0, denoising_range_num=1,
                           range_num=1, extract_prefix_video_feature=False, fwd_extra_1st_chunk=False,
                           distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                           core_attn_params=P.build_core_attn_params(kr.to(dev), kr.to(dev), L),
                           cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
    rope = rope_mod.get_embed_for_forward(fr, H, W, 0, 1)
    with torch.no_grad():
        core, xo = layer(hs, y, None, rope, meta)
        fused = layer(hs, y, None, rope, meta, proj_layout=True)
    assert torch.equal(fused.cpu(), O.attn_linear_proj_input(core.cpu(), xo.cpu()))


def test_layer_with_arena_backed_cache(dev):
    """The same cached forward with the lazily allocated per-layer cache and with a view of the all-layer arena:
    identical outputs and identical cache rows."""
    from magi_attn.cache import KVCacheArena
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W = 1, 4, 4
    L = fr * H * W
    layer = _make_layer(dev, hidden, Hq, Hkv, seed=7)
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    outs = []
    for use_arena in (False, True):
        ip = P.InferenceParams(1, 4 * L)
        ip.update_kv_cache = True
        if use_arena:
            arena = KVCacheArena(5, 4 * L, Hkv, device=dev)
            arena.buffer.fill_(float("nan"))
            arena.attach(ip)  # the layer's number (3) selects arena row 3
        g = torch.Generator().manual_seed(8)
        res = []
        for sp, dn in ((0, 2), (2, 2)):
            S = dn * L
            hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
            mask = torch.ones(dn, 1, 1, 8)
            y = (torch.randn(dn * 8, hidden, generator=g) * 0.5).bfloat16().to(dev)
            meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp,
                                   denoising_range_num=dn, range_num=sp + dn, extract_prefix_video_feature=False,
                                   fwd_extra_1st_chunk=True, distill_nearly_clean_chunk=False, clip_token_nums=L,
                                   enable_cuda_graph=False,
                                   core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                             R.generate_default_kvrange(sp, dn, L).to(dev), L),
                                   cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
            with torch.no_grad():
                res.append(layer(hs, y, ip, rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn), meta))
        outs.append((res, ip.key_value_memory_dict[3].clone()))
    for (c0, x0), (c1, x1) in zip(outs[0][0], outs[1][0]):
        assert torch.equal(c0, c1) and torch.equal(x0, x1)
    assert torch.equal(outs[0][1][: 4 * L], outs[1][1][: 4 * L])
    assert torch.isnan(arena.layer(2)).all() and torch.isnan(arena.layer(4)).all()  # other layers untouched


@pytest.mark.parametrize("staging_buffers", [1, 2, 3])
def test_layers_with_offloaded_caches_match_resident_ones(dev, staging_buffers):
    """kv_offload as an option (dit_module.py:803-811, 915): three layers whose caches live in pinned host memory behind
    a ring of 1, 2 or 3 device staging buffers, run through a schedule that appends, re-reads without persisting
    (update_kv_cache False: side buffer), drops the last chunk (distill) and then starts a second generation on the
    same arena with different inputs (a copy made ahead for the next layer must not survive a rewrite of the host
    rows).  Every output and every persisted cache row is bit-identical to the same schedule on a resident arena."""
    from magi_attn.cache import KVCacheArena, OffloadedKVCache
    from magi_attn.rope import LearnableRotaryEmbeddingCat
    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W = 1, 4, 4
    L = fr * H * W
    n_chunks = 6
    layers = []
    for i in range(3):
        torch.manual_seed(40 + i)
        layer = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=i, device=dev)
        with torch.no_grad():
            for prm in layer.parameters():
                prm.copy_(torch.randn_like(prm.float()) * (0.1 if prm.dim() == 1 else hidden ** -0.5))
            layer.linear_qkv.layer_norm.weight.add_(1.0)
        layers.append(layer)
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    # (slice_point, denoising chunks, update_kv_cache, distill_nearly_clean_chunk)
    schedule = [(0, 2, True, False), (2, 2, False, False), (2, 2, True, True), (3, 3, True, False),
                (0, 2, True, False), (2, 3, True, False)]          # the last two: a new generation on the same arena
    results = []
    for offload in (False, True):
        arena = KVCacheArena(3, n_chunks * L, Hkv, device=dev, kv_offload=offload, staging_buffers=staging_buffers)
        ip = P.InferenceParams(1, n_chunks * L)
        arena.attach(ip)
        if offload:
            assert all(isinstance(ip.key_value_memory_dict[i], OffloadedKVCache) for i in range(3))
            assert arena.host.is_pinned() and len(arena.stages) == min(3, staging_buffers)
        g = torch.Generator().manual_seed(9)
        outs, rows = [], []
        for sp, dn, update, distill in schedule:
            ip.update_kv_cache = update
            S = dn * L
            hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
            y = (torch.randn(dn * 8, hidden, generator=g) * 0.5).bfloat16().to(dev)
            meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp,
                                   denoising_range_num=dn, range_num=sp + dn, extract_prefix_video_feature=False,
                                   fwd_extra_1st_chunk=True, distill_nearly_clean_chunk=distill, clip_token_nums=L,
                                   enable_cuda_graph=False,
                                   core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                             R.generate_default_kvrange(sp, dn, L).to(dev), L),
                                   cross_attn_params=P.build_cross_attn_params(torch.ones(dn, 1, 1, 8).to(dev), L, 8))
            rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
            x = hs
            with torch.no_grad():
                for layer in layers:       # each layer's self-attention output feeds the next (hidden = Hq * D / 3)
                    core, cross = layer(x, y, ip, rope, meta)
                    outs.append((core.clone(), cross.clone()))
                    x = (core.view(S, 1, 3, hidden).float().mean(2) + hs.float()).bfloat16()
            arena.synchronize()
            kept = (sp + (dn - 1 if distill else dn)) * L if update else None
            if kept is not None:
                src = arena.host if offload else arena.buffer
                rows.append(src[:, sp * L:kept].clone().cpu())
        results.append((outs, rows))
    for (c0, x0), (c1, x1) in zip(*[r[0] for r in results]):
        assert torch.equal(c0, c1) and torch.equal(x0, x1)
    assert len(results[0][1]) == len(results[1][1]) == 5
    for r0, r1 in zip(results[0][1], results[1][1]):
        assert torch.equal(r0, r1)


def test_copying_form_of_the_cache_update_with_offloaded_caches(dev):
    """adjust_key_and_value_for_inference (the reference-shaped method for a materialised key_and_value) on an
    offloaded cache: the prefix comes through the staging buffer and the appended rows reach the pinned host copy;
    keys, values and cache rows equal the oracle's model of the reference's tensor."""
    from magi_attn.cache import KVCacheArena
    Hkv, D, L_ = 2, 128, 40
    layer = MOD.FullyParallelAttention(256, 6, Hkv, layer_number=1, device=dev)
    arena = KVCacheArena(3, 6 * L_, Hkv, device=dev, kv_offload=True, staging_buffers=2)
    ip = P.InferenceParams(1, 6 * L_)
    arena.attach(ip)
    arena.host.zero_()
    model = O.KVCacheModel(6 * L_, Hkv, D)
    g = torch.Generator().manual_seed(4)
    for sp, dn, update, distill in ((0, 2, True, False), (2, 2, False, False), (2, 2, True, True), (3, 3, True, False)):
        kv = torch.randn(dn * L_, Hkv, 2 * D, generator=g).bfloat16()
        ip.update_kv_cache = update
        meta = P.ModelMetaArgs(H=1, W=L_, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=True,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L_, enable_cuda_graph=False,
                               core_attn_params=None, cross_attn_params=None)
        k, v = layer.adjust_key_and_value_for_inference(kv.to(dev), ip, meta)
        k_ref, v_ref = model.adjust(kv, has_inference_params=True, update_kv_cache=update, slice_point=sp,
                                    clip_token_nums=L_, fwd_extra_1st_chunk=True, distill_nearly_clean_chunk=distill)
        assert torch.equal(k.cpu(), k_ref) and torch.equal(v.cpu(), v_ref), (sp, dn)
        arena.synchronize()
        assert torch.equal(arena.host[1], model.mem)
    assert not arena.host[0].any() and not arena.host[2].any()


@pytest.mark.parametrize("fast_exp2", [True, False])
def test_layer_with_fp8_self_attention_and_fp8_cache(dev, fast_exp2):
    """attention_dtype="fp8": same schedule as above through two layers with identical weights, one bf16 and one
    fp8.  The reference has no fp8 attention (parity unpinned by it); the bf16 layer, itself checked against the
    oracle above, is the yardstick: per step cosine >= 0.998 and max-abs <= 2^-5 max|V| on the self-attention
    output, bit-identical cross-attention output, and a cache that dequantises to the bf16 cache within e4m3
    rounding (2^-4 relative, per-(chunk, head) scale)."""
    from magi_attn.cache import Fp8KVCache
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden, Hq, Hkv, D = 256, 6, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    n_chunks = 6
    ref_layer = _make_layer(dev, hidden, Hq, Hkv, seed=5)
    torch.manual_seed(5)
    fp8_layer = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=3, device=dev, attention_dtype="fp8",
                                           fp8_fast_exp2=fast_exp2)
    fp8_layer.load_state_dict(ref_layer.state_dict())
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip_ref, ip_fp8 = P.InferenceParams(1, n_chunks * L), P.InferenceParams(1, n_chunks * L)
    g = torch.Generator().manual_seed(6)
    #        sp dn update distill extra has_ip
    steps = [(0, 2, True, False, True, True),
             (0, 3, True, True, True, True),
             (2, 3, False, False, False, True),
             (2, 3, True, False, False, True),
             (1, 4, True, True, True, True),
             (3, 3, False, False, True, True),
             (0, 2, False, False, False, False)]
    for sp, dn, update, distill, extra, has_ip in steps:
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
        lens = torch.randint(0, 9, (dn,), generator=g)
        mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
        y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16().to(dev)
        k_range = R.generate_default_kvrange(sp, dn, L) if has_ip else R.generate_kv_range_for_uncondition(dn, L)
        q_range = R.q_ranges_from_chunks(dn, L)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=extra,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(q_range.to(dev), k_range.to(dev), L),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        ip_ref.update_kv_cache = ip_fp8.update_kv_cache = update
        with torch.no_grad():
            core_ref, xo_ref = ref_layer(hs, y, ip_ref if has_ip else None, rope, meta)
            core, xo = fp8_layer(hs, y, ip_fp8 if has_ip else None, rope, meta)
            vmax = ref_layer.linear_qkv.forward_v(ref_layer.linear_qkv.forward_ln(hs)).float().abs().max().item()
        assert torch.equal(xo, xo_ref)
        if not has_ip:  # (a pass that leaves the caches alone) the fp8 path writes the linear_proj layout too
            with torch.no_grad():
                fused = fp8_layer(hs, y, None, rope, meta, proj_layout=True)
            assert torch.equal(fused, MOD.attn_linear_proj_input(core, xo))
        a, b = core.double().flatten(), core_ref.double().flatten()
        cos = (a @ b / (a.norm() * b.norm())).item()
        err = (a - b).abs().max().item()
        if has_ip and ip_ref.key_value_memory_dict:
            vmax = max(vmax, ip_ref.key_value_memory_dict[3][..., D:].float().abs().max().item())
        assert cos >= 0.998 and err <= 2 ** -5 * vmax, ((sp, dn, update, distill, extra), cos, err, vmax)
        if has_ip and (extra or sp > 0) and update:
            keep = S - L if distill else S
            cache = ip_fp8.key_value_memory_dict[3]
            assert isinstance(cache, Fp8KVCache)
            rows = slice(sp * L, sp * L + keep)
            sc = lambda t: t[sp:sp + keep // L].repeat_interleave(L, dim=0)[:, :, None]
            want = ip_ref.key_value_memory_dict[3][rows].float()
            for got, ref_half in ((cache.k[rows].float() * sc(cache.k_scale), want[..., :D]),
                                  (cache.v[rows].float() * sc(cache.v_scale), want[..., D:])):
                assert ((got - ref_half).abs() <= ref_half.abs() * 2 ** -4 + 2 ** -9 * ref_half.abs().max()).all()


def test_fp8_layer_prepares_its_operands_in_two_launches(dev):
    """Between the GEMM of the projections and the fp8 attention kernel the layer issues exactly two kernels: the prologue
    with e4m3 outputs (q, and k into the cache rows) and the one-launch V quantiser; no absmax / conversion
    passes and no torch elementwise kernels.  The library's own launch counter gives the number of its launches per
    steady-state forward (six: input norm, prologue, V quantiser, fp8 attention, text-side k norm, cross attention);
    a kernel trace of the same forward, when the profiler records device activity, names what lies between them."""
    from torch.profiler import ProfilerActivity, profile
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden, Hq, Hkv, D = 256, 8, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    torch.manual_seed(11)
    layer = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=0, device=dev, attention_dtype="fp8")
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip = P.InferenceParams(1, 6 * L)
    g = torch.Generator().manual_seed(12)

    def step(sp, dn, update, distill):
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
        mask = torch.ones(dn, 1, 1, 8)
        y = (torch.randn(dn * 8, hidden, generator=g) * 0.5).bfloat16().to(dev)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=True,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(
                                   R.q_ranges_from_chunks(dn, L).to(dev), R.generate_default_kvrange(sp, dn, L).to(dev), L),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        ip.update_kv_cache = update
        with torch.no_grad():
            return layer(hs, y, ip, rope, meta, proj_layout=True)

    step(0, 2, True, False)  # warm-up: caches the fp32 norm parameters, the constant scale tables, the side buffers
    step(0, 3, True, True)
    torch.cuda.synchronize()
    for args in ((1, 3, True, True), (2, 3, True, False)):  # with and without rows that are not persisted
        n0 = M.lib().magi_launch_count()
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            step(*args)
            torch.cuda.synchronize()
        assert M.lib().magi_launch_count() - n0 == 6
        evs = sorted((e for e in prof.events() if e.device_type == torch.autograd.DeviceType.CUDA and "Memcpy" not in e.name
                      and "Memset" not in e.name), key=lambda e: e.time_range.start)
        names = [e.name for e in evs]
        if not names:  # (no device activity recorded: the launch count above is the check)
            continue
        attn = [i for i, n in enumerate(names) if "attn_fwd_fp8_kernel" in n]
        assert len(attn) == 1, names
        ln = max(i for i, n in enumerate(names[:attn[0]]) if "layer_norm_kernel" in n)
        between = names[ln + 1:attn[0]]  # the one GEMM of the four projections, then the two launches
        assert len(between) == 3 and "magi::" not in between[0], between
        assert "prologue_kernel" in between[1] and "quantize_groups_kernel" in between[2], between


def test_layer_with_the_projections_and_prologue_in_one_launch(dev):
    """fused_projection=True: the layer's four projections and the prologue run as magi_qkv_proj_prologue.  Same
    schedule through two layers with identical weights; the raw projections differ from the library GEMM's only
    where the accumulation order decides a bf16 rounding, so outputs and caches agree closely but not bit for bit:
    cosine >= 0.9999, max-abs <= 2e-2 on the attention outputs (the bar of the bf16 path against the oracle), cache
    rows within 2^-6 of the row's largest magnitude."""
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden, Hq, Hkv, D = 256, 8, 2, 128
    fr, H, W = 2, 3, 4
    L = fr * H * W
    ref_layer = _make_layer(dev, hidden, Hq, Hkv, seed=9)
    torch.manual_seed(9)
    one = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=3, device=dev, fused_projection=True)
    one.load_state_dict(ref_layer.state_dict())
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip_ref, ip_one = P.InferenceParams(1, 6 * L), P.InferenceParams(1, 6 * L)
    g = torch.Generator().manual_seed(10)
    #        sp dn update distill extra has_ip proj_layout
    steps = [(0, 2, True, False, True, True, False),
             (0, 3, True, True, True, True, True),
             (2, 3, False, False, False, True, False),
             (0, 2, False, False, False, False, True)]
    for sp, dn, update, distill, extra, has_ip, proj in steps:
        S = dn * L
        hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
        lens = torch.randint(1, 9, (dn,), generator=g)
        mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
        y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16().to(dev)
        k_range = R.generate_default_kvrange(sp, dn, L) if has_ip else R.generate_kv_range_for_uncondition(dn, L)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=extra,
                               distill_nearly_clean_chunk=distill, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                         k_range.to(dev), L),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        ip_ref.update_kv_cache = ip_one.update_kv_cache = update
        with torch.no_grad():
            want = ref_layer(hs, y, ip_ref if has_ip else None, rope, meta, proj_layout=proj)
            got = one(hs, y, ip_one if has_ip else None, rope, meta, proj_layout=proj)
        for a, b in zip(got if isinstance(got, tuple) else (got,), want if isinstance(want, tuple) else (want,)):
            assert a.shape == b.shape
            assert (a.float() - b.float()).abs().max().item() <= 2e-2 and _cosine(a, b) >= 0.9999
        if has_ip and update:
            ca, cb = ip_one.key_value_memory_dict[3].float(), ip_ref.key_value_memory_dict[3].float()
            keep = S - L if distill else S
            rows = slice(sp * L, sp * L + keep)
            for half in (slice(0, D), slice(D, 2 * D)):
                d = (ca[rows][..., half] - cb[rows][..., half]).abs()
                assert torch.all(d <= cb[rows][..., half].abs().amax(dim=-1, keepdim=True) * 2.0 ** -6)


# ----------------------------------------------------------------------------- layer input norm
@pytest.mark.parametrize("rows,cols,params", [
    (1000, 6144, "bf16"), (333, 3072, "bf16"), (77, 4096, "fp32"), (5, 8, "bf16"), (64, 8192, "bf16"),
    (100, 1000, "fp32"), (1, 520, "bf16"), (4099, 1536, "none"), (9000, 6144, "bf16"),
])
def test_layer_norm_matches_oracle(rows, cols, params):
    """Layer input LayerNorm (dit_module.py:401, 412-413): fp32 statistics, one rounding to bf16.  The oracle
    evaluates the definition in float64; bar as for the prologue (one bf16 ulp, < 1 in 1000 elements differ)."""
    g = torch.Generator().manual_seed(rows * 31 + cols)
    x = (torch.randn(rows, cols, generator=g) * 2.0 + 0.5).bfloat16()
    dt = {"bf16": torch.bfloat16, "fp32": torch.float32, "none": None}[params]
    w = None if dt is None else (1 + 0.3 * torch.randn(cols, generator=g)).to(dt)
    b = None if dt is None else (0.2 * torch.randn(cols, generator=g)).to(dt)
    dev = lambda t: None if t is None else t.cuda()
    y = M.layer_norm(x.cuda(), dev(w), dev(b), 1e-5)
    torch.cuda.synchronize()
    assert y.shape == x.shape and y.dtype == torch.bfloat16
    ref = O.input_layer_norm(x, w, b, 1e-5).float().bfloat16()
    _ulp_check(y, ref, f"layer_norm {rows}x{cols} {params}")


def test_layer_norm_strided_rows_leading_axes_and_offset_mean():
    g = torch.Generator().manual_seed(77)
    # rows that are column slices of a wider buffer, as a view of a fused activation would be
    wide = torch.randn(301, 2 * 3072, generator=g).bfloat16()
    w = (1 + 0.1 * torch.randn(3072, generator=g)).bfloat16()
    b = (0.1 * torch.randn(3072, generator=g)).bfloat16()
    y = M.layer_norm(wide.cuda()[:, 3072:], w.cuda(), b.cuda(), 1e-6)
    _ulp_check(y, O.input_layer_norm(wide[:, 3072:], w, b, 1e-6).float().bfloat16(), "strided rows")
    # [sq, b, h] input as the layer passes it, written into a caller's buffer
    x3 = torch.randn(50, 2, 1024, generator=g).bfloat16()
    out = torch.empty(50, 2, 1024, dtype=torch.bfloat16, device="cuda")
    y3 = M.layer_norm(x3.cuda(), w.cuda()[:1024].contiguous(), None, 1e-6, out=out)
    assert y3 is out
    _ulp_check(y3, O.input_layer_norm(x3, w[:1024], None, 1e-6).float().bfloat16(), "3-d input")
    # a mean far above the spread: the two-pass variance must not cancel
    xo = (torch.randn(40, 2048, generator=g) * 0.25 + 100.0).bfloat16()
    yo = M.layer_norm(xo.cuda(), None, None, 1e-5)
    _ulp_check(yo, O.input_layer_norm(xo, None, None, 1e-5).float().bfloat16(), "offset mean")
    # a constant row: zero variance, the result is the bias
    c = torch.full((3, 512), 1.5).bfloat16()
    yc = M.layer_norm(c.cuda(), w.cuda()[:512].contiguous(), b.cuda()[:512].contiguous(), 1e-5)
    assert torch.equal(yc.cpu(), b[:512].expand(3, -1))


def test_layer_norm_rejects_bad_arguments():
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(TypeError):
        M.layer_norm(x.float(), None, None)
    with pytest.raises(ValueError):
        M.layer_norm(x, torch.ones(32, dtype=torch.bfloat16, device="cuda"), None)
    with pytest.raises(TypeError):
        M.layer_norm(x, torch.ones(64, dtype=torch.bfloat16, device="cuda"), torch.ones(64, device="cuda"))
    with pytest.raises(M.MagiError):
        M.layer_norm(torch.zeros(4, 60, dtype=torch.bfloat16, device="cuda"), None, None)
    assert M.layer_norm(x[:0], None, None).shape == (0, 64)


def test_rope_table_built_on_the_device_matches_the_oracle(dev):
    """The table the layer (and the benchmark) builds with device sin / cos for the 720p window (72 latent frames of
    45 x 80, last 24 kept) against the CPU restatement of the reference's table: fp32 angles up to ~71 rad, where
    device and host sin / cos implementations may differ in the last bits of their argument reduction."""
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    fr, H, W, dn, sp = 6, 45, 80, 4, 8
    got = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, sp, dn)
    want = O.rope_for_forward(dn * fr, H, W, sp, dn)
    assert got.shape == want.shape == (dn * fr * H * W, 96) and got.dtype == torch.float32
    assert (got.cpu() - want).abs().max().item() <= 1e-5
    # and a small odd grid, where the centre row has all-zero spatial angles
    got = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(4, 5, 7, 1, 2)
    want = O.rope_for_forward(4, 5, 7, 1, 2)
    assert (got.cpu() - want).abs().max().item() <= 1e-6
