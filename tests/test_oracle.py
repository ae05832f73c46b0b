"""Pins of the CPU oracle: each restated function is checked against something other than
its own formula (closed forms, library routines, brute force, invariants, and the vectors the
reference keeps in comments)."""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import magi_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ----------------------------------------------------------------------------- rope table
def test_freq_bands_spot_values():
    b = O.freq_bands(16)
    assert b.shape == (16,)
    assert b[0].item() == 1.0
    assert abs(b[15].item() - 10000.0 ** (-15 / 16)) < 1e-9
    assert abs(b[8].item() - 0.01) < 1e-8  # 10000^-0.5


def test_rope_table_layout_and_separability():
    T, H, W = 3, 4, 6
    tab = O.rope_table(T, H, W)
    assert tab.shape == (T * H * W, 96)
    sin, cos = tab[:, :48].reshape(T, H, W, 48), tab[:, 48:].reshape(T, H, W, 48)
    # columns 0..15 depend on t only, 16..31 on h only, 32..47 on w only
    assert torch.equal(sin[:, :, :, :16], sin[:, :1, :1, :16].expand(T, H, W, 16))
    assert torch.equal(sin[:, :, :, 16:32], sin[:1, :, :1, 16:32].expand(T, H, W, 16))
    assert torch.equal(cos[:, :, :, 32:], cos[:1, :1, :, 32:].expand(T, H, W, 16))
    # sin^2 + cos^2 = 1
    assert torch.allclose(sin**2 + cos**2, torch.ones_like(sin), atol=1e-6)
    # h positions are symmetric about 0: sin odd, cos even under h -> H-1-h
    assert torch.allclose(sin[0, :, 0, 16:32], -sin[0, :, 0, 16:32].flip(0), atol=1e-6)
    assert torch.allclose(cos[0, :, 0, 16:32], cos[0, :, 0, 16:32].flip(0), atol=1e-6)
    # t = 0 row has zero temporal angle
    assert torch.all(sin[0, :, :, :16] == 0) and torch.all(cos[0, :, :, :16] == 1)


def test_rope_table_closed_form_spot():
    T, H, W = 5, 4, 6
    tab = O.rope_table(T, H, W)
    t, h, w = 3, 1, 5
    row = (t * H + h) * W + w
    for j in (0, 3, 15):
        band = 10000.0 ** (-j / 16)
        assert abs(tab[row, j].item() - math.sin(t * band)) < 1e-6
        assert abs(tab[row, 16 + j].item() - math.sin((h - 1.5) * band)) < 1e-6
        assert abs(tab[row, 48 + 32 + j].item() - math.cos((w - 2.5) * band)) < 1e-6


def test_rope_rescale_identity_for_256_positions_and_formula_otherwise():
    # H*W == 256 -> s = 1 -> ref shape == feat shape -> x/(f-1)*(f-1): identity up to rounding
    a = O.rope_for_forward(2, 16, 16, 0, 1)
    b = O.rope_table(2, 16, 16)
    assert torch.allclose(a, b, atol=1e-6)
    # otherwise h positions scale by (H/s - 1)/(H - 1)
    T, H, W = 2, 8, 13
    s = math.sqrt(H * W / 256)
    tab = O.rope_for_forward(T, H, W, 0, 1)
    h, j = 6, 2
    row = (1 * H + h) * W + 0
    pos = (h - (H - 1) / 2) / (H - 1) * (H / s - 1)
    assert abs(tab[row, 16 + j].item() - math.sin(pos * 10000.0 ** (-j / 16))) < 1e-6


def test_rope_slice_equals_offset_table():
    # the last dn chunks of the table built over prefix + new frames == absolute temporal positions
    H, W, fr = 4, 6, 2
    sp, dn = 3, 2
    sl = O.rope_for_forward(dn * fr, H, W, sp, dn)
    full = O.rope_for_forward((sp + dn) * fr, H, W, 0, sp + dn)
    assert sl.shape[0] == dn * fr * H * W
    assert torch.equal(sl, full[-sl.shape[0]:])
    # first kept row sits at t = sp*fr
    assert abs(sl[0, 0].item() - math.sin(sp * fr * 1.0)) < 1e-6


# ----------------------------------------------------------------------------- norms
def test_qk_layernorm_vs_fp64_definition():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 3, 128, generator=g)
    w = torch.randn(128, generator=g) * 0.1
    b = torch.randn(128, generator=g) * 0.1
    y = O.qk_layernorm(x, w, b, 1e-6)
    xd = x.double()
    mu = xd.mean(-1, keepdim=True)
    var = ((xd - mu) ** 2).mean(-1, keepdim=True)  # biased
    ref = (xd - mu) / torch.sqrt(var + 1e-6) * (w.double() + 1) + b.double()
    assert (y.double() - ref).abs().max() < 1e-5
    # zero-centred gamma = 0, beta = 0 gives unit variance rows
    y0 = O.qk_layernorm(x, torch.zeros(128), torch.zeros(128))
    assert torch.allclose(y0.var(-1, unbiased=False), torch.ones(7, 3), atol=1e-4)


def test_input_layer_norm_vs_torch_module_and_invariances():
    g = torch.Generator().manual_seed(11)
    x = torch.randn(9, 384, generator=g) * 3 + 0.7
    ln = torch.nn.LayerNorm(384, eps=1e-5)
    with torch.no_grad():
        ln.weight.copy_(torch.randn(384, generator=g))
        ln.bias.copy_(torch.randn(384, generator=g))
        ref = ln(x)
    y = O.input_layer_norm(x, ln.weight.detach(), ln.bias.detach(), 1e-5)
    assert (y - ref.double()).abs().max() < 2e-5
    # without affine parameters: zero mean, unit (biased) variance, invariant to a shift and a positive scale
    y0 = O.input_layer_norm(x, None, None, 0.0)
    assert y0.mean(-1).abs().max() < 1e-12 and (y0.var(-1, unbiased=False) - 1).abs().max() < 1e-12
    assert (O.input_layer_norm(4.0 * x + 2.5, None, None, 0.0) - y0).abs().max() < 1e-5
    # eps enters under the root: a constant row maps to the bias
    c = torch.full((2, 384), 3.25)
    assert torch.equal(O.input_layer_norm(c, ln.weight.detach(), ln.bias.detach(), 1e-5), ln.bias.detach().double().expand(2, -1))


def test_rmsnorm_unit_rms():
    x = torch.randn(5, 2, 128, generator=torch.Generator().manual_seed(1))
    y = O.rmsnorm(x)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(5, 2), atol=1e-4)


# ----------------------------------------------------------------------------- rotary
def test_rope_matches_transformers_rotate_half_convention():
    from transformers.models.llama.modeling_llama import rotate_half

    g = torch.Generator().manual_seed(2)
    S, Hh, D, R2 = 11, 3, 128, 48
    x = torch.randn(1, S, Hh, D, generator=g)
    ang = torch.randn(S, R2, generator=g)
    cos, sin = ang.cos(), ang.sin()
    y = O.apply_rope_neox_partial(x, cos, sin)
    xr = x[..., : 2 * R2]
    c2 = torch.cat([cos, cos], -1)[None, :, None, :]
    s2 = torch.cat([sin, sin], -1)[None, :, None, :]
    ref = xr * c2 + rotate_half(xr) * s2
    assert torch.allclose(y[..., : 2 * R2], ref, atol=1e-6)
    assert torch.equal(y[..., 2 * R2:], x[..., 2 * R2:])  # pass-through dims untouched


def test_rope_invariants():
    g = torch.Generator().manual_seed(3)
    S, D, R2 = 6, 128, 48
    x = torch.randn(S, 2, D, generator=g)
    ang = torch.randn(S, R2, generator=g)
    y = O.apply_rope_neox_partial(x, ang.cos(), ang.sin())
    # each (i, i+48) pair keeps its norm
    n0 = x[..., :R2] ** 2 + x[..., R2:2 * R2] ** 2
    n1 = y[..., :R2] ** 2 + y[..., R2:2 * R2] ** 2
    assert torch.allclose(n0, n1, atol=1e-5)
    # zero angle is the identity
    z = torch.zeros(S, R2)
    assert torch.equal(O.apply_rope_neox_partial(x, z.cos(), z.sin()), x)
    # <rope(q,p), rope(k,p')> depends on p - p' only (1-D positions, same bands)
    q, k = torch.randn(D, generator=g), torch.randn(D, generator=g)
    bands = torch.rand(R2, generator=g)

    def rot(v, p):
        a = (p * bands)[None]
        return O.apply_rope_neox_partial(v[None, None], a.cos(), a.sin())[0, 0]

    d1 = torch.dot(rot(q, 5.0), rot(k, 2.0))
    d2 = torch.dot(rot(q, 13.0), rot(k, 10.0))
    assert abs(d1 - d2) < 1e-4


def test_prologue_composition_order_and_dtypes():
    g = torch.Generator().manual_seed(4)
    S, Hq, Hkv, D = 24, 3, 1, 128
    qr = torch.randn(S, Hq, D, generator=g).bfloat16()
    kr = torch.randn(S, Hkv, D, generator=g).bfloat16()
    vr = torch.randn(S, Hkv, D, generator=g).bfloat16()
    rope = O.rope_table(1, 4, 6)
    z = torch.zeros(D)
    q, kv = O.prologue(qr, kr, vr, rope, z, z, z, z)
    assert q.dtype == torch.bfloat16 and kv.shape == (S, Hkv, 2 * D)
    assert torch.equal(kv[..., D:], vr)  # V untouched
    # sin is the FIRST half of the table: swapping halves must change the result
    q_sw, _ = O.prologue(qr, kr, vr, torch.cat([rope[:, 48:], rope[:, :48]], -1), z, z, z, z)
    assert not torch.equal(q, q_sw)
    ref = O.apply_rope_neox_partial(F.layer_norm(qr.float(), (D,), eps=1e-6), rope[:, 48:], rope[:, :48]).bfloat16()
    assert torch.equal(q, ref)


# ----------------------------------------------------------------------------- attention
def _small_case(seed, L, dn, sp, Hq, Hkv, D=128):
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, D, seed, dtype=torch.float32)
    return q, k, v, O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)


@pytest.mark.parametrize("L,dn,sp,Hq,Hkv", [(16, 3, 0, 2, 1), (37, 2, 2, 6, 2), (50, 4, 1, 3, 3), (9, 1, 0, 6, 1)])
def test_range_attention_vs_fp64_brute_force(L, dn, sp, Hq, Hkv):
    q, k, v, qr, kr = _small_case(10 + L, L, dn, sp, Hq, Hkv, D=32)
    o = O.range_attention(q, k, v, qr, kr)
    ref = O.brute_attention_fp64(q, k, v, qr, kr)
    assert (o.double() - ref).abs().max() < 2e-6
    lse = O.range_attention_lse(q, k, v, qr, kr)
    g = Hq // Hkv
    s = torch.einsum("qhd,khd->hqk", q[:L].double(), k[: kr[0, 1]].double().repeat_interleave(g, 1)) * 32 ** -0.5
    assert (lse[:, :L].double() - torch.logsumexp(s, -1)).abs().max() < 1e-5


def test_range_attention_equals_block_mask_sdpa_on_c1_shape_subsample():
    # the benchmark's CPU configuration, shrunk in L only
    q, k, v, qr, kr = _small_case(1234, 192, 3, 0, 24, 8)
    a = O.range_attention(q, k, v, qr, kr)
    b = O.block_mask_attention(q, k, v, qr, kr)
    assert (a - b).abs().max() < 2e-6


def test_attention_invariants():
    q, k, v, qr, kr = _small_case(7, 24, 3, 1, 4, 2, D=64)
    # V = 1 -> O = 1
    o1 = O.range_attention(q, k, torch.ones_like(v), qr, kr)
    assert torch.allclose(o1, torch.ones_like(o1), atol=1e-6)
    # permuting keys inside a range leaves O unchanged
    o = O.range_attention(q, k, v, qr[:1], kr[:1])
    perm = torch.randperm(int(kr[0, 1]), generator=torch.Generator().manual_seed(0))
    k2, v2 = k.clone(), v.clone()
    k2[: kr[0, 1]] = k[: kr[0, 1]][perm]
    v2[: kr[0, 1]] = v[: kr[0, 1]][perm]
    assert (O.range_attention(q, k2, v2, qr[:1], kr[:1]) - o).abs().max() < 1e-5
    # a range's output does not depend on the other ranges
    full = O.range_attention(q, k, v, qr, kr)
    assert torch.equal(full[qr[1, 0]:qr[1, 1]], O.range_attention(q, k, v, qr[1:2], kr[1:2])[qr[1, 0]:qr[1, 1]])
    # own-chunk-only ranges == independent attention per chunk
    L = 24
    own = np.array([[(1 + i) * L, (2 + i) * L] for i in range(3)])
    oo = O.range_attention(q, k, v, qr, own)
    for i in range(3):
        ref = O.brute_attention_fp64(q[i * L:(i + 1) * L], k[(1 + i) * L:(2 + i) * L], v[(1 + i) * L:(2 + i) * L],
                                     [[0, L]], [[0, L]])
        assert (oo[i * L:(i + 1) * L].double() - ref).abs().max() < 1e-5
    # GQA == MHA on repeat_interleaved K/V
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    assert (O.range_attention(q, kk, vv, qr, kr) - full).abs().max() < 1e-6
    # default kv range == block lower-triangular mask; dn=1, sp=0 == plain attention
    p = O.range_attention(q[:L], k[:L], v[:L], [[0, L]], [[0, L]])
    ref = F.scaled_dot_product_attention(q[:L].transpose(0, 1)[None], k[:L].repeat_interleave(2, 1).transpose(0, 1)[None],
                                         v[:L].repeat_interleave(2, 1).transpose(0, 1)[None])[0].transpose(0, 1)
    assert (p - ref).abs().max() < 1e-6


def test_varlen_cross_attention_segments_and_empty():
    g = torch.Generator().manual_seed(5)
    Hq, Hkv, D, L = 4, 2, 32, 10
    lens = [7, 0, 3]
    q = torch.randn(3 * L, Hq, D, generator=g)
    k = torch.randn(sum(lens), Hkv, D, generator=g)
    v = torch.randn(sum(lens), Hkv, D, generator=g)
    cu_q = [0, L, 2 * L, 3 * L]
    cu_k = np.cumsum([0] + lens)
    o = O.varlen_cross_attention(q, k, v, cu_q, cu_k)
    assert torch.all(o[L:2 * L] == 0)  # segment without keys -> zero rows
    for s in (0, 2):
        ref = O.brute_attention_fp64(q[cu_q[s]:cu_q[s + 1]], k[cu_k[s]:cu_k[s + 1]], v[cu_k[s]:cu_k[s + 1]],
                                     [[0, L]], [[0, lens[s]]])
        assert (o[cu_q[s]:cu_q[s + 1]].double() - ref).abs().max() < 1e-5
    mask = torch.zeros(3, 16)
    for i, n in enumerate(lens):
        mask[i, :n] = 1
    cq, ck, qr, kr = O.cross_attn_params_from_mask(mask, L)
    assert cq.tolist() == cu_q and ck.tolist() == cu_k.tolist()
    assert qr.tolist() == [[0, 10], [10, 20], [20, 30]] and kr.tolist() == [[0, 7], [7, 7], [7, 10]]


# ----------------------------------------------------------------------------- KV cache model
def test_kv_cache_model_against_list_of_chunks():
    rng = np.random.default_rng(0)
    L, Hkv, D, n_chunks = 5, 2, 4, 6
    cache = O.KVCacheModel(n_chunks * L, Hkv, D, dtype=torch.float32)
    chunks = [None] * n_chunks  # what a reader of chunk c must see
    counter = [0]

    def new_kv(n):
        counter[0] += 1
        return torch.full((n * L, Hkv, 2 * D), float(counter[0])) + torch.arange(n * L)[:, None, None] * 1e-3

    for _ in range(60):
        sp = int(rng.integers(0, n_chunks - 1))
        dn = int(rng.integers(1, min(4, n_chunks - sp) + 1))
        upd = bool(rng.integers(0, 2))
        distill = bool(rng.integers(0, 2)) and dn > 1
        extra = bool(rng.integers(0, 2))
        has_ip = bool(rng.integers(0, 4))
        if any(chunks[c] is None for c in range(sp)):
            continue  # the pipeline never reads a chunk it has not written
        kv = new_kv(dn)
        k, v = cache.adjust(kv, has_inference_params=has_ip, update_kv_cache=upd, slice_point=sp, clip_token_nums=L,
                            fwd_extra_1st_chunk=extra, distill_nearly_clean_chunk=distill)
        if not has_ip or not (extra or sp > 0):
            assert torch.equal(k, kv[..., :D]) and torch.equal(v, kv[..., D:])
            continue
        expect = torch.cat([chunks[c] for c in range(sp)] + [kv], 0) if sp else kv
        assert torch.equal(torch.cat([k, v], -1), expect)
        if upd:
            keep = dn - 1 if distill else dn
            for j in range(keep):
                chunks[sp + j] = kv[j * L:(j + 1) * L].clone()
        for c in range(n_chunks):
            if chunks[c] is not None:
                assert torch.equal(cache.mem[c * L:(c + 1) * L], chunks[c])


def test_attn_linear_proj_input_index_by_index():
    # (n hn hd) -> (hn n hd) with n = 2, hn = 8, checked element by element against the index formula
    sq, b, Hq, D = 3, 2, 16, 4
    core = torch.arange(sq * b * Hq * D, dtype=torch.float32).view(sq, b, Hq * D)
    cross = -core - 1
    got = O.attn_linear_proj_input(core, cross)
    assert got.shape == (sq, b, 2 * Hq * D)
    hd = Hq * D // 8
    for s_ in range(sq):
        for b_ in range(b):
            for hn in range(8):
                for n, src in ((0, core), (1, cross)):
                    for d in range(hd):
                        assert got[s_, b_, hn * 2 * hd + n * hd + d] == src[s_, b_, hn * hd + d]


# ----------------------------------------------------------------------------- chunk-window arithmetic
def test_generate_sequences_reference_comment_examples():
    # the four worked examples kept next to the function in the reference (video_generate.py:139-161),
    # held as data in tests/golden/generate_sequences_examples.json
    with open(os.path.join(GOLDEN, "generate_sequences_examples.json")) as f:
        examples = json.load(f)
    assert len(examples) == 4
    for e in examples:
        got = O.generate_sequences(e["chunk_num"], e["window_size"], e["chunk_offset"])
        assert got == (e["clip_start"], e["clip_end"], e["t_start"], e["t_end"]), e


def test_layer_small_fixture_matches_oracle():
    # the frozen small layer pass: the oracle must still produce it from the stored inputs
    z = np.load(os.path.join(GOLDEN, "layer_small.npz"))
    bf = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    T, H, W, prefix, dn, Hq, Hkv, D = (int(x) for x in z["dims"])
    L = T * H * W
    assert np.array_equal(z["rope"], O.rope_for_forward(dn * T, H, W, prefix, dn).numpy())
    assert np.array_equal(z["q_ranges"], O.q_ranges_for(dn, L)) and np.array_equal(z["k_ranges"], O.default_kvrange(prefix, dn, L))
    q, kv = O.prologue(bf(z["q_raw"]), bf(z["k_raw"]), bf(z["v_raw"]), torch.from_numpy(z["rope"]),
                       *(torch.from_numpy(z[n]) for n in ("gq", "bq", "gk", "bk")))
    assert torch.equal(q, bf(z["q"])) and torch.equal(kv, bf(z["kv"]))
    cache = torch.cat([bf(z["prefix_kv"]), kv], 0)
    out = O.range_attention(q, cache[..., :D], cache[..., D:], z["q_ranges"], z["k_ranges"])
    assert torch.allclose(out.float(), torch.from_numpy(z["out"]), atol=1e-5, rtol=0)
    # independent check of the frozen output: fp64 brute force over the same stored tensors
    ref = O.brute_attention_fp64(q, cache[..., :D], cache[..., D:], z["q_ranges"], z["k_ranges"])
    assert torch.allclose(torch.from_numpy(z["out"]).double(), ref, atol=2e-5, rtol=0)
    xout = O.varlen_cross_attention(q, bf(z["xk"]), bf(z["xv"]), z["cu_q"], z["cu_k"])
    assert torch.allclose(xout.float(), torch.from_numpy(z["xout"]), atol=1e-5, rtol=0)
    assert torch.count_nonzero(torch.from_numpy(z["xout"])[L:]) == 0  # empty text segment -> zeros


def test_kvrange_tables_hand_derived():
    L = 100
    assert O.default_kvrange(2, 3, L).tolist() == [[0, 300], [0, 400], [0, 500]]
    # shipped configs: noise2clean [5,4,3,2], clean 1, 32 steps -> 8 steps per stage
    r = O.noise2clean_kvrange(8, 4, L, [5, 4, 3, 2], 1, [32, 20, 9, 0], 32)
    #  chunk ends 9,10,11,12; widths: clean->1, 20//8=2 ->3, 9//8=1 ->4, 0 ->5
    assert r.tolist() == [[800, 900], [700, 1000], [700, 1100], [700, 1200]]
    r = O.noise2clean_kvrange(0, 2, L, [5, 4, 3, 2], -1, [32, 31], 32)  # clean -> last entry (2); clamp at 0
    assert r.tolist() == [[0, 100], [0, 200]]
    assert O.prefix_video_kvrange(3, L, clean_chunk_kvrange=1).tolist() == [[0, 100], [100, 200], [200, 300]]
    assert O.prefix_video_kvrange(3, L, noise2clean=[5, 2]).tolist() == [[0, 100], [0, 200], [100, 300]]
    assert O.prefix_video_kvrange(2, L).tolist() == [[0, 100], [0, 200]]  # default window 8
    assert O.uncondition_kvrange(3, L).tolist() == [[0, 100], [100, 200], [200, 300]]
    assert O.q_ranges_for(2, L).tolist() == [[0, 100], [100, 200]]


def test_attention_flops_published_figures():
    # the per-config figures of the benchmark definition
    assert O.attention_flops(O.q_ranges_for(3, 1536), O.default_kvrange(0, 3, 1536), 24, 128) == pytest.approx(1.739e11, rel=1e-3)
    assert O.attention_flops(O.q_ranges_for(4, 9360), O.default_kvrange(4, 4, 9360), 24, 128) == pytest.approx(2.799e13, rel=1e-3)
    assert O.attention_flops(O.q_ranges_for(4, 21600), O.default_kvrange(8, 4, 21600), 48, 128) == pytest.approx(4.816e14, rel=1e-3)


# ----------------------------------------------------------------------------- fp8 quantiser
def test_fp8_quantiser_properties():
    x = torch.tensor([0.0, 1.0, -1.0, 447.0, 448.0, 449.0, 1e6, -1e6, 0.0625, 3.1])
    q = O.quantize_e4m3(x, torch.tensor(1.0)).float()
    assert q[4] == 448 and q[5] == 448 and q[6] == 448 and q[7] == -448  # saturates, never NaN/inf
    assert q[0] == 0 and q[1] == 1 and q[2] == -1 and q[8] == 0.0625
    xs = torch.linspace(-500, 500, 4001)
    qs = O.quantize_e4m3(xs, torch.tensor(1.0)).float()
    assert torch.all(qs[1:] >= qs[:-1])  # monotone
    g = torch.Generator().manual_seed(0)
    t = torch.randn(40, 3, 128, generator=g) * torch.tensor([0.1, 1.0, 30.0])[None, :, None]
    t8, sc = O.quantize_per_head_chunk(t, 16)
    assert sc.shape == (3, 3)
    for c in range(3):
        blk = t[c * 16:(c + 1) * 16]
        assert torch.allclose(sc[c], blk.abs().amax(dim=(0, 2)) / 448)
    back = O.dequantize_per_head_chunk(t8, sc, 16)
    rel = (back - t).abs() / t.abs().clamp_min(1e-3 * t.abs().amax())
    assert (back - t).abs().max() <= 0.0625 * t.abs().max() + 1e-6  # e4m3: 3 mantissa bits
    assert t8.float().abs().max() == 448  # absmax maps onto the top code


def test_div_clamp_double_rounding_through_bf16_hand_computed():
    """The reference's linear-layer quantiser rounds x / scale to bf16 before e4m3 (dit_module.py:376-381).  e4m3 has
    a grid of 1/8 in [1, 2) and bf16 one of 1/128, so a value just beside an e4m3 midpoint first lands ON the midpoint
    and then goes to the even code: worked out by hand, and different from the single rounding in both directions."""
    up = 1.0625 + 2.0 ** -10     # above the midpoint of 1.0 and 1.125: one rounding gives 1.125
    down = 1.1875 - 2.0 ** -10   # below the midpoint of 1.125 and 1.25: one rounding gives 1.125
    x = torch.tensor([up, down, -up, -down, 3.0 * up, 1e9, -1e9])
    one = O.quantize_e4m3(x, torch.tensor(1.0)).float()
    two = O.quantize_e4m3(x, torch.tensor(1.0), via_bf16=True).float()
    assert one.tolist() == [1.125, 1.125, -1.125, -1.125, 3.25, 448.0, -448.0]
    # bf16 first: 1.0625 exactly (tie -> even mantissa 000 = 1.0), 1.1875 exactly (tie -> even mantissa 010 = 1.25);
    # 3 x up = 3.189 is nearer 3.25 than 3.0 (grid 1/4 in [2, 4)) with either rounding
    assert two.tolist() == [1.0, 1.25, -1.0, -1.25, 3.25, 448.0, -448.0]
    # the scale divides first: the same codes from 4 x the values with scale 4, and per-column scales broadcast
    assert O.quantize_e4m3(4.0 * x, torch.tensor(4.0), via_bf16=True).float().tolist() == two.tolist()
    cols = O.quantize_e4m3(torch.tensor([[up, 2.0 * up]]), torch.tensor([1.0, 2.0]), via_bf16=True).float()
    assert cols.tolist() == [[1.0, 1.0]]


def test_prologue_premul_is_the_softmax_scale_moved_into_q():
    """prologue(q_premul=c) has no counterpart in the reference.  Pin: with c = softmax_scale * log2(e) the
    pre-scaled q through attention with softmax_scale = ln 2 equals (up to q's bf16 rounding) the reference-shaped
    unscaled prologue followed by default-scale attention; K, V are untouched; c = 1 is the plain prologue; and in
    fp32 (no rounding) the factor commutes exactly: prologue(x, c) == c * prologue(x)."""
    g = torch.Generator().manual_seed(3)
    T, H, W, Hq, Hkv, D = 2, 3, 4, 4, 2, 128
    S = T * H * W
    rope = O.rope_for_forward(T, H, W, 0, 1)
    mk = lambda *s: torch.randn(*s, generator=g)
    gq, bq, gk, bk = (mk(D) * 0.1 for _ in range(4))
    q_raw, k_raw, v_raw = mk(S, Hq, D).bfloat16(), mk(S, Hkv, D).bfloat16(), mk(S, Hkv, D).bfloat16()
    c = D ** -0.5 * math.log2(math.e)
    q0, kv0 = O.prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk)
    q1, kv1 = O.prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk, q_premul=c)
    qa, kva = O.prologue(q_raw, k_raw, v_raw, rope, gq, bq, gk, bk, q_premul=1.0)
    assert torch.equal(kv0, kv1) and torch.equal(q0, qa) and torch.equal(kv0, kva)
    qf0, _ = O.prologue(q_raw.float(), k_raw.float(), v_raw.float(), rope, gq, bq, gk, bk)
    qf1, _ = O.prologue(q_raw.float(), k_raw.float(), v_raw.float(), rope, gq, bq, gk, bk, q_premul=c)
    assert torch.allclose(qf1, qf0 * c, rtol=1e-6, atol=0)
    # one rounding to bf16 on each side: half an ulp (2^-8 relative) each
    assert (q1.float() - q0.float() * c).abs().max() <= 2 * 2 ** -8 * (q0.float().abs().max() * c)
    r = [[0, S]]
    a = O.range_attention(q0, kv0[..., :D], kv0[..., D:], r, r)
    b = O.range_attention(q1, kv1[..., :D], kv1[..., D:], r, r, softmax_scale=math.log(2.0))
    assert (a - b).abs().max() < 5e-3
