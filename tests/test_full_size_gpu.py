"""Benchmark-size parity of the kernels the layer and the benchmark actually launch.

Every shipped bf16 instantiation runs the 480p and the 720p layer shapes and the ragged four-video batch: the
online-softmax kernel (32 rows per wavefront; what a caller without a score bound gets), the bounded-score kernels
(64 rows per wavefront, no running maximum): the 16x16x32-MFMA form with 256-row workgroups that
FullyParallelAttention.forward and bench.py launch, the 32x32x16-MFMA form with 256- and 512-row workgroups, and the
default form with the softmax scale applied while q is loaded (what the four reference-shaped callables select when
given score_bound=).  The fused prologue runs at S = 86400 x 56 head rows into
a 259200-row cache, and one FullyParallelAttention.forward runs at hidden 6144 / 48 / 8 heads over a resident arena.

Outputs of this size are checked on row subsamples.  Query rows are independent of each other, so fp32 attention of
a sample of rows against the full key range is exact for those rows: many rows per chunk with plain fp32 matmuls on
the GPU, a few of them through the CPU oracle as well (which also pins the GPU-side reference).  Size-independent
properties on the whole tensor: V = 1 gives O = 1, and K / V read in place from the interleaved cache give the same
bits as contiguous copies.

Bars (bf16 path, from the benchmark definition): max-abs <= 2e-2 and cosine >= 0.9999 against fp32 attention of the
same bf16 inputs; prologue within one bf16 ulp of the oracle with fewer than 1 in 1000 elements different, V bit
exact."""
import math

import numpy as np
import pytest
import torch

import magi_attn as M
from magi_attn import module as MOD
from magi_attn import params as P
from magi_attn import ranges as R
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MIN_COS = 0.9999
D = 128
PREMUL = D ** -0.5 * math.log2(math.e)
LN2 = math.log(2.0)
# per-head RMS-normalised q and k have length sqrt(D): |q . k| <= D, times the pre-scale factor, plus 1 % for the
# roundings to bf16 (what FullyParallelAttention.score_bounds() derives from unit-gain norm parameters)
UNIT_GAIN_BOUND = 1.01 * D * PREMUL

# kernel variants: name -> (q carries the scale, keyword arguments of range_attention)
VARIANTS = {
    "online": (False, {}),
    "online-prescaled": (True, dict(q_prescaled=True)),
    "bounded-256": (True, dict(q_prescaled=True, score_bound=UNIT_GAIN_BOUND, q_tile_rows=0)),
    "bounded-512": (True, dict(q_prescaled=True, score_bound=UNIT_GAIN_BOUND, q_tile_rows=512)),
    "bounded-mfma32": (True, dict(q_prescaled=True, score_bound=UNIT_GAIN_BOUND, bounded_mfma32=True)),
    "bounded-scale-on-load": (False, dict(score_bound=UNIT_GAIN_BOUND)),
}


def _cmp(out, ref, what=""):
    o = out.detach().double().flatten()
    r = ref.detach().double().flatten().to(o.device)
    err = (o - r).abs().max().item()
    cos = (torch.dot(o, r) / (o.norm() * r.norm()).clamp_min(1e-30)).item()
    assert err <= MAX_ABS, f"{what}: max-abs {err}"
    assert cos >= MIN_COS, f"{what}: cosine {cos}"
    return err, cos


def _ranges(dev, *arrs):
    return [torch.tensor(np.asarray(a), dtype=torch.int32, device=dev) for a in arrs]


def _rms_normed(x):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)


def _fp32_rows(q_rows, k, v, scale):
    """softmax(q k^T * scale) v in fp32 for q_rows [r, Hq, D] against all of k / v [T, Hkv, D] (strided views of the
    cache are fine), one KV head at a time."""
    r, Hq, _ = q_rows.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    ref = torch.empty(r, Hq, D, device=q_rows.device)
    qs = q_rows.float()
    for hk in range(Hkv):
        kk, vv = k[:, hk].float(), v[:, hk].float()
        s = torch.einsum("rgd,kd->rgk", qs[:, hk * G:(hk + 1) * G], kk) * scale
        ref[:, hk * G:(hk + 1) * G] = torch.einsum("rgk,kd->rgd", torch.softmax(s, -1), vv)
    return ref


SHAPES = {
    # name: (L, dn, sp, Hq, Hkv, seed, sampled rows per chunk, of which through the CPU oracle)
    "480p": (9360, 4, 4, 24, 8, 2234, 256, 8),
    "720p": (21600, 4, 8, 48, 8, 3234, 128, 4),
}


@pytest.fixture(scope="module", params=sorted(SHAPES))
def layer_case(request, dev):
    """Inputs of one benchmark shape and the fp32 reference of its sampled rows, built once for all kernel variants:
    q both unscaled and carrying softmax_scale * log2(e) (each rounded to bf16 once from the same fp32 values), the
    interleaved cache, the ranges, the sampled rows and their fp32 attention for both forms of q.  The reference rows
    are themselves checked against the CPU oracle here."""
    L, dn, sp, Hq, Hkv, seed, n_rows, cpu_rows = SHAPES[request.param]
    g = torch.Generator(device=dev).manual_seed(seed)
    qf = _rms_normed(torch.randn(dn * L, Hq, D, device=dev, generator=g))
    q, qp = qf.bfloat16(), (qf * PREMUL).bfloat16()
    del qf
    cache = torch.randn((sp + dn) * L, Hkv, 2 * D, device=dev, generator=g)
    cache[..., :D] = _rms_normed(cache[..., :D])
    cache = cache.bfloat16()
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    k, v = cache[..., :D], cache[..., D:]
    # the promise the bounded variants make must hold for these tensors
    assert (qp.float().norm(dim=-1).max() * k.float().norm(dim=-1).max()).item() <= UNIT_GAIN_BOUND
    rs = np.random.default_rng(seed)
    rows, ref, refp = [], [], []
    for i in range(dn):
        idx = torch.tensor(np.sort(rs.choice(L, n_rows, replace=False)) + i * L, device=dev)
        ke = int(kr[i, 1])
        rows.append(idx)
        ref.append(_fp32_rows(q[idx], k[:ke], v[:ke], D ** -0.5))
        refp.append(_fp32_rows(qp[idx], k[:ke], v[:ke], LN2))
        sub = idx[:cpu_rows].cpu()
        kc, vc = k[:ke].cpu(), v[:ke].cpu()
        o_cpu = O.range_attention(q[sub].cpu(), kc, vc, [[0, cpu_rows]], [[0, ke]])
        assert (ref[-1][:cpu_rows].cpu() - o_cpu).abs().max() < 1e-4, "GPU-side fp32 reference vs CPU oracle"
        o_cpu = O.range_attention(qp[sub].cpu(), kc, vc, [[0, cpu_rows]], [[0, ke]], softmax_scale=LN2)
        assert (refp[-1][:cpu_rows].cpu() - o_cpu).abs().max() < 1e-4, "GPU-side fp32 reference vs CPU oracle (pre-scaled q)"
        del kc, vc
    tq, tk = _ranges(dev, qr, kr)
    return dict(name=request.param, L=L, dn=dn, q=q, qp=qp, cache=cache, tq=tq, tk=tk, rows=rows, ref=ref, refp=refp)


@pytest.mark.parametrize("variant", sorted(VARIANTS))
def test_core_attention_full_size(layer_case, variant):
    c = layer_case
    prescaled, kw = VARIANTS[variant]
    q = c["qp"] if prescaled else c["q"]
    refs = c["refp"] if prescaled else c["ref"]
    k, v = c["cache"][..., :D], c["cache"][..., D:]
    out, lse = M.range_attention(q, k, v, c["tq"], c["tk"], c["L"], **kw)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()
    for i, (idx, ref) in enumerate(zip(c["rows"], refs)):
        _cmp(out[idx], ref, f"{c['name']} {variant} chunk {i}")
    # K / V in place from the interleaved cache == contiguous copies, bit for bit
    out2, _ = M.range_attention(q, k.contiguous(), v.contiguous(), c["tq"], c["tk"], c["L"], return_lse=False, **kw)
    assert torch.equal(out, out2), "strided cache views vs contiguous K / V"
    del out2
    # values all ones -> output all ones (every row, every head)
    ones = c["cache"].clone()
    ones[..., D:] = 1
    o1, _ = M.range_attention(q, ones[..., :D], ones[..., D:], c["tq"], c["tk"], c["L"], return_lse=False, **kw)
    assert (o1.float() - 1).abs().max().item() <= 2 ** -7


@pytest.mark.parametrize("variant", ["online", "bounded-256", "bounded-512", "bounded-mfma32", "bounded-scale-on-load"])
def test_full_size_ragged_batch_with_cross_attention(dev, variant):
    """Four videos packed on one token axis with 1, 2, 3 and 4 active 9360-token chunks and 0-6 cached prefix chunks
    each (seeded), chunk-causal inside each video (24 / 8 heads), then cross attention from every video token to that
    video's T5 tokens (valid lengths uniform 20-800, K / V on 24 heads)."""
    prescaled, kw = VARIANTS[variant]
    L, Hq, Hkv = 9360, 24, 8
    rs = np.random.default_rng(5234)
    active = [1, 2, 3, 4]
    prefix = [int(x) for x in rs.integers(0, 7, size=4)]
    lens = [int(x) for x in rs.integers(20, 801, size=4)]
    qr, kr, seg_len = [], [], []
    qpos = kbase = 0
    for a, p, n in zip(active, prefix, lens):
        for j in range(a):
            qr.append([qpos, qpos + L])
            kr.append([kbase, kbase + (p + j + 1) * L])
            seg_len.append(n)  # every chunk of a video attends to that video's caption
            qpos += L
        kbase += (p + a) * L
    Tq, Tk = qpos, kbase
    g = torch.Generator(device=dev).manual_seed(5234)
    qf = _rms_normed(torch.randn(Tq, Hq, D, device=dev, generator=g))
    q = (qf * PREMUL).bfloat16() if prescaled else qf.bfloat16()
    scale = LN2 if prescaled else D ** -0.5
    del qf
    cache = torch.randn(Tk, Hkv, 2 * D, device=dev, generator=g)
    cache[..., :D] = _rms_normed(cache[..., :D])
    cache = cache.bfloat16()
    tq, tk = _ranges(dev, qr, kr)
    out, _ = M.range_attention(q, cache[..., :D], cache[..., D:], tq, tk, L, return_lse=False, **kw)
    for i, ((q0, _), (k0, k1)) in enumerate(zip(qr, kr)):
        rows = torch.tensor(np.sort(rs.choice(L, 64, replace=False)) + q0, device=dev)
        ref = _fp32_rows(q[rows], cache[k0:k1, :, :D], cache[k0:k1, :, D:], scale)
        _cmp(out[rows], ref, f"{variant} self range {i} GPU fp32 subsample")
        sub = rows[:4].cpu()
        o_cpu = O.range_attention(q[sub].cpu(), cache[k0:k1, :, :D].cpu(), cache[k0:k1, :, D:].cpu(), [[0, 4]],
                                  [[0, k1 - k0]], softmax_scale=scale)
        _cmp(out[sub], o_cpu, f"{variant} self range {i} CPU oracle subsample")
    ones = cache.clone()
    ones[..., D:] = 1
    o1, _ = M.range_attention(q, ones[..., :D], ones[..., D:], tq, tk, L, return_lse=False, **kw)
    assert (o1.float() - 1).abs().max() <= 2 ** -7
    # cross attention: one segment per chunk, L queries against its video's caption (K normalised like the layer's)
    cu_q = torch.arange(0, Tq + 1, L, dtype=torch.int32, device=dev)
    cu_k = torch.tensor(np.concatenate([[0], np.cumsum(seg_len)]), dtype=torch.int32, device=dev)
    kvx = torch.randn(int(cu_k[-1]), Hq, 2 * D, device=dev, generator=g)
    kvx[..., :D] = _rms_normed(kvx[..., :D])
    kvx = kvx.bfloat16()
    xo, _ = M.range_attention(q, kvx[..., :D], kvx[..., D:], cu_q, cu_k, L, 800, ranges_mode=M.MAGI_RANGES_CU,
                              return_lse=False, **kw)
    for i, n in enumerate(seg_len):
        rows = torch.tensor(np.sort(rs.choice(L, 64, replace=False)) + i * L, device=dev)
        k0 = int(cu_k[i])
        ref = _fp32_rows(q[rows], kvx[k0:k0 + n, :, :D], kvx[k0:k0 + n, :, D:], scale)
        _cmp(xo[rows], ref, f"{variant} cross segment {i} GPU fp32 subsample")
        sub = rows[:4].cpu()
        o_cpu = O.range_attention(q[sub].cpu(), kvx[k0:k0 + n, :, :D].cpu(), kvx[k0:k0 + n, :, D:].cpu(), [[0, 4]],
                                  [[0, n]], softmax_scale=scale)
        _cmp(xo[sub], o_cpu, f"{variant} cross segment {i} CPU oracle subsample")


# ----------------------------------------------------------------------------- prologue at the 720p shape
def _ulp_check(a, ref, what=""):
    a, ref = a.cpu(), ref.cpu()
    af, rf = a.float(), ref.float()
    ulp = torch.clamp(rf.abs() * 2.0 ** -7, min=1e-5)
    assert torch.all((af - rf).abs() <= ulp), f"{what}: more than one bf16 ulp off"
    frac = (a != ref).float().mean().item()
    assert frac < 1e-3, f"{what}: {frac:.2e} of the elements differ"


def _e4m3_check(got, ref, what=""):
    gb, rb = got.cpu().view(torch.uint8).int(), ref.cpu().view(torch.uint8).int()
    diff = gb != rb
    assert diff.float().mean().item() < 2e-3, f"{what}: {diff.float().mean().item():.2e} of the elements differ"
    mag_g, mag_r = gb & 0x7f, rb & 0x7f
    near = ((gb & 0x80) == (rb & 0x80)) & ((mag_g - mag_r).abs() <= 1) | ((mag_g + mag_r) <= 1)
    assert torch.all(near | ~diff), f"{what}: more than one e4m3 code off"


def test_prologue_full_size_720p(dev):
    """S = 86400 tokens x (48 + 8) head rows with the rotary table of the 720p window (72 latent frames of 45 x 80,
    the last 24 are this forward's), written into a 259200-row cache at row 172800.  512 sampled tokens against the
    oracle's prologue (one bf16 ulp; V bit exact), the rows of the cache outside the destination untouched; then the
    same pass with e4m3 outputs (neighbouring code at most)."""
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    fr, H, W, dn, sp, Hq, Hkv = 6, 45, 80, 4, 8, 48, 8
    L = fr * H * W
    S, start = dn * L, sp * L
    g = torch.Generator(device=dev).manual_seed(720)
    q_raw = torch.randn(S, Hq * D, device=dev, generator=g).bfloat16()
    k_raw = torch.randn(S, Hkv * D, device=dev, generator=g).bfloat16()
    v_raw = torch.randn(S, Hkv * D, device=dev, generator=g).bfloat16()
    gc = torch.Generator().manual_seed(721)
    gq, bq, gk, bk = (torch.randn(D, generator=gc) * 0.2 for _ in range(4))
    rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, sp, dn)
    rope_ref = O.rope_for_forward(dn * fr, H, W, sp, dn)
    assert rope.shape == (S, 96)
    cache = torch.full(((sp + dn) * L, Hkv, 2 * D), 7.0, dtype=torch.bfloat16, device=dev)
    to = lambda t: t.to(dev)
    q, _, _ = M.qk_prologue(q_raw, k_raw, v_raw, rope, to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv,
                            kv_out=cache[start:], n_cache_rows=S, q_premul=PREMUL)
    torch.cuda.synchronize()
    assert torch.all(cache[:start] == 7.0), "rows ahead of the write position were touched"
    rs = np.random.default_rng(722)
    idx = np.sort(np.concatenate([[0, 1, L - 1, L, S - 1], rs.choice(S, 507, replace=False)]))
    ti = torch.tensor(idx, device=dev)
    q_ref, kv_ref = O.prologue(q_raw[ti].cpu().view(-1, Hq, D), k_raw[ti].cpu().view(-1, Hkv, D),
                               v_raw[ti].cpu().view(-1, Hkv, D), rope_ref[idx], gq, bq, gk, bk, q_premul=PREMUL)
    _ulp_check(q[ti], q_ref, "q")
    _ulp_check(cache[start + ti, :, :D], kv_ref[..., :D], "k (cache rows)")
    assert torch.equal(cache[start + ti, :, D:].cpu(), kv_ref[..., D:]), "v (cache rows)"
    # every V row is a copy of its raw row: checked on the whole tensor
    assert torch.equal(cache[start:, :, D:].reshape(S, Hkv * D), v_raw)
    # e4m3 outputs: q and k quantised with constant power-of-two scales from the norm-parameter bound
    bound = lambda g_, b_: math.sqrt(D) * (g_ + 1).abs().max().item() + b_.norm().item()
    qs, ks = M.pow2_scale_for(PREMUL * bound(gq, bq)), M.pow2_scale_for(bound(gk, bk))
    k8 = torch.zeros((sp + dn) * L, Hkv, D, device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn)
    q8, _, _ = M.qk_prologue_fp8(q_raw, k_raw, rope, to(gq), to(bq), to(gk), to(bk), Hq=Hq, Hkv=Hkv, q_scale=qs,
                                 k_scale=ks, q_premul=PREMUL, k_out=k8[start:], n_cache_rows=S)
    torch.cuda.synchronize()
    q_f, k_f = O.prologue(q_raw[ti].cpu().view(-1, Hq, D), k_raw[ti].cpu().view(-1, Hkv, D),
                          v_raw[ti].cpu().view(-1, Hkv, D), rope_ref[idx], gq, bq, gk, bk, q_premul=PREMUL, downcast=False)
    _e4m3_check(q8[ti], O.quantize_e4m3(q_f, torch.tensor(qs)), "q e4m3")
    _e4m3_check(k8[start + ti], O.quantize_e4m3(k_f, torch.tensor(ks)), "k e4m3 (cache rows)")
    assert torch.count_nonzero(k8[:start].view(torch.uint8)).item() == 0


# ----------------------------------------------------------------------------- the layer at the 720p shape
def test_layer_forward_full_size_720p(dev):
    """FullyParallelAttention.forward at hidden 6144, 48 / 8 heads, chunks of 21600 tokens, over one layer's view of
    a resident KVCacheArena: two forwards of four clean chunks fill the prefix (slice_point 0 and 4), then the
    forward under test runs four denoising chunks at slice_point 8 (Q 86400 tokens over K / V 259200), output in the
    linear_proj layout.  Checked on 32 sampled tokens per chunk against the reference's forward restated with the
    oracle's pieces: LayerNorm and projections in fp32 matmuls on those rows, the oracle's prologue, fp32 attention
    over the cache rows (which are themselves checked on the sampled tokens against the oracle's prologue)."""
    from magi_attn.cache import KVCacheArena
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden, Hq, Hkv = 6144, 48, 8
    fr, H, W = 6, 45, 80
    L = fr * H * W
    n_chunks, dn = 12, 4
    torch.manual_seed(77)
    layer = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=1, device=dev)
    with torch.no_grad():
        for p in layer.parameters():
            if p.dim() == 1:
                p.copy_(torch.randn_like(p.float()) * 0.1)
            else:
                p.copy_(torch.randn_like(p.float()) * hidden ** -0.5)
        layer.linear_qkv.layer_norm.weight.add_(1.0)
    assert 0.0 < layer.score_bounds()[0] <= M.MAGI_SCORE_BOUND_MAX  # the bounded kernel is the one that runs
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    ip = P.InferenceParams(1, n_chunks * L)
    ip.update_kv_cache = True
    arena = KVCacheArena(3, n_chunks * L, Hkv, device=dev)
    arena.buffer.fill_(float("nan"))
    arena.attach(ip)
    g = torch.Generator(device=dev).manual_seed(78)
    rs = np.random.default_rng(79)
    lens_all = [[800, 20, 413, 0], [0, 33, 0, 800], [655, 0, 800, 64]]  # text tokens per chunk; 0 = a chunk without text
    hs = y = meta = rope = None
    for step, sp in enumerate((0, 4, 8)):
        S = dn * L
        hs = (torch.randn(S, 1, hidden, device=dev, generator=g) * 1.5 + 0.1).bfloat16()
        lens = torch.tensor(lens_all[step])
        mask = (torch.arange(800)[None] < lens[:, None]).float().view(dn, 1, 1, 800)
        y = (torch.randn(int(lens.sum()), hidden, device=dev, generator=g) * 0.5).bfloat16()
        k_range = R.generate_default_kvrange(sp, dn, L)
        meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                               range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=True,
                               distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                               core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev),
                                                                         k_range.to(dev), L),
                               cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 800))
        rope = rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn)
        with torch.no_grad():
            fused = layer(hs, y, ip, rope, meta, proj_layout=True)
        torch.cuda.synchronize()
    sp = 8
    S = dn * L
    assert fused.shape == (S, 1, 2 * Hq * D) and torch.isfinite(fused).all()
    cache = ip.key_value_memory_dict[1]
    assert cache.data_ptr() == arena.layer(1).data_ptr()
    assert torch.isnan(arena.layer(0)).all() and torch.isnan(arena.layer(2)).all()  # the other layers' rows untouched
    assert torch.isfinite(cache.float()).all()
    # un-group the linear_proj layout: [S, 8 groups, (core, cross), Hq / 8, D]
    grouped = fused.view(S, MOD.PROJ_GROUPS, 2, Hq // MOD.PROJ_GROUPS, D)
    core = grouped[:, :, 0].reshape(S, Hq, D)
    cross = grouped[:, :, 1].reshape(S, Hq, D)
    # --- reference on sampled tokens ---
    idx = np.sort(np.concatenate([rs.choice(L, 32, replace=False) + i * L for i in range(dn)]))
    ti = torch.tensor(idx, device=dev)
    lq = layer.linear_qkv
    x = hs[ti, 0].float()
    mixed = torch.nn.functional.layer_norm(x, (hidden,), lq.layer_norm.weight.float(), lq.layer_norm.bias.float(),
                                           lq.layer_norm.eps).bfloat16()
    got_mixed = lq.forward_ln(hs[ti])[:, 0]
    _ulp_check(got_mixed, mixed, "layer input norm")
    lin = lambda m: (got_mixed.float() @ m.weight.float().t()).bfloat16()  # (fp32 matmul of the bf16 operands)
    q_raw, k_raw, v_raw, qx_raw = lin(lq.q), lin(lq.k), lin(lq.v), lin(lq.qx)
    cpu = lambda t: t.detach().float().cpu()
    rope_ref = O.rope_for_forward(dn * fr, H, W, sp, dn)
    q_ref, kv_ref = O.prologue(q_raw.cpu().view(-1, Hq, D), k_raw.cpu().view(-1, Hkv, D), v_raw.cpu().view(-1, Hkv, D),
                               rope_ref[idx], cpu(layer.q_layernorm.weight), cpu(layer.q_layernorm.bias),
                               cpu(layer.k_layernorm.weight), cpu(layer.k_layernorm.bias))
    # the layer's projections come from the library's bf16 GEMM, whose accumulation order may round a raw value the
    # other way: cache rows within 2^-6 of the row's largest magnitude (the bar of the fused-projection test)
    got_kv = cache[sp * L + ti].float().cpu()
    for half, nm in ((slice(0, D), "k"), (slice(D, 2 * D), "v")):
        want = kv_ref[..., half].float()
        assert torch.all((got_kv[..., half] - want).abs() <= want.abs().amax(dim=-1, keepdim=True) * 2.0 ** -6), nm
    # core attention of the sampled rows over the cache the layer wrote (prefix included)
    qd = q_ref.to(dev)
    kr = R.generate_default_kvrange(sp, dn, L).numpy()
    for i in range(dn):
        sel = torch.tensor(np.nonzero((idx >= i * L) & (idx < (i + 1) * L))[0], device=dev)
        ke = int(kr[i, 1])
        ref = _fp32_rows(qd[sel], cache[:ke, :, :D], cache[:ke, :, D:], D ** -0.5)
        _cmp(core[ti[sel]], ref, f"core, chunk {i}")
    # cross attention: bf16 norms of q and k (the reference keeps the cross-attention norms in bf16), fp32 attention
    ln_bf16 = lambda t, ln: torch.nn.functional.layer_norm(t, (D,), ln.weight.detach() + 1, ln.bias.detach(), ln.eps)
    qx = ln_bf16(qx_raw.view(-1, Hq, D), layer.q_layernorm_xattn)
    kvx = torch.nn.functional.linear(y, layer.linear_kv_xattn.weight).view(y.shape[0], Hkv, 2 * D)
    kx = ln_bf16(kvx[..., :D], layer.k_layernorm_xattn)
    cu_k = meta.cross_attn_params.cu_seqlens_kv.cpu().numpy()
    for i in range(dn):
        sel = torch.tensor(np.nonzero((idx >= i * L) & (idx < (i + 1) * L))[0], device=dev)
        k0, k1 = int(cu_k[i]), int(cu_k[i + 1])
        if k1 == k0:  # a chunk without text: zero rows, all of them
            assert torch.count_nonzero(cross[i * L:(i + 1) * L]).item() == 0
            continue
        ref = _fp32_rows(qx[sel], kx[k0:k1], kvx[k0:k1, :, D:], D ** -0.5)
        _cmp(cross[ti[sel]], ref, f"cross, chunk {i}")
