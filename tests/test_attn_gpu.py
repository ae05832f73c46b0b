"""GPU parity of the range-attention kernel (through the C-ABI) against the CPU oracle.

Tolerance (bf16 path, from the benchmark definition): max-abs <= 2e-2 and cosine >= 0.9999
against the fp32 reference on identical seeded inputs."""
import math
import os

import numpy as np
import pytest
import torch

import magi_attn as M
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu

MAX_ABS = 2e-2
MIN_COS = 0.9999


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


CASES = [
    # L, dn, sp, Hq, Hkv
    (128, 1, 0, 1, 1),      # exactly one q tile, two key tiles
    (64, 2, 0, 2, 1),       # half-filled q tile
    (200, 3, 1, 6, 2),      # ragged everywhere, GQA 3
    (77, 2, 2, 3, 1),       # L below one tile
    (1, 3, 2, 6, 1),        # single-token chunks, GQA 6
    (333, 4, 3, 12, 4),
    (1536, 3, 0, 24, 8),    # the CPU-runnable benchmark configuration
]


@pytest.mark.parametrize("L,dn,sp,Hq,Hkv", CASES)
def test_chunk_causal_parity(dev, L, dn, sp, Hq, Hkv):
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=1234 + L)
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    ref = O.range_attention(q, k, v, qr, kr)
    lse_ref = O.range_attention_lse(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr, kr)
    out, lse = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, int(kr.max() - kr.min()))
    assert out.dtype == torch.bfloat16 and out.shape == q.shape and lse.shape == (Hq, dn * L)
    _cmp(out, ref, f"L={L}")
    # the kernel's row sum runs over the probabilities as rounded to bf16 (what the PV product uses): ~1e-3
    assert (lse.cpu() - lse_ref).abs().max() < 5e-3


def test_sliding_window_ranges_and_unsorted_order(dev):
    L, sp, dn, Hq, Hkv = 150, 8, 4, 6, 2
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=5)
    qr = O.q_ranges_for(dn, L)
    kr = O.noise2clean_kvrange(sp, dn, L, [5, 4, 3, 2], 1, [32, 20, 9, 0], 32)
    perm = [2, 0, 3, 1]  # the order of the ranges must not matter
    ref = O.range_attention(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr[perm], kr[perm])
    out, _ = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, 5 * L)
    _cmp(out, ref)


def test_empty_key_range_uncovered_rows_and_clamping(dev):
    L, Hq, Hkv = 100, 4, 2
    q, k, v = O.synthetic_qkv(4 * L, 3 * L, Hq, Hkv, 128, seed=6)
    # range 0: no keys -> zeros; rows [L, 2L) in no range -> zeros (fresh output); range 2 k end past total_k -> clamped
    qr = np.array([[0, L], [2 * L, 3 * L], [3 * L, 4 * L + 50]])
    kr = np.array([[40, 40], [0, 2 * L], [L, 3 * L + 999]])
    ref = O.range_attention(q, k, v, np.clip(qr, 0, 4 * L), np.clip(kr, 0, 3 * L))
    tq, tk = _ranges(dev, qr, kr)
    out, lse = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, L + 50, 3 * L)
    assert torch.all(out[: 2 * L] == 0)
    assert torch.all(torch.isinf(lse[:, :L])) and torch.all(lse[:, :L] < 0)
    _cmp(out, ref)


def test_many_ranges_and_q_tile_bound(dev):
    # 40 ranges of uneven length; max_seqlen_q is only an upper bound
    rng = np.random.default_rng(0)
    lens = rng.integers(1, 300, size=40)
    cu = np.concatenate([[0], np.cumsum(lens)])
    Tq = int(cu[-1])
    Hq, Hkv = 3, 1
    q, k, v = O.synthetic_qkv(Tq, 700, Hq, Hkv, 128, seed=7)
    qr = np.stack([cu[:-1], cu[1:]], 1)
    ks = rng.integers(0, 400, size=40)
    kr = np.stack([ks, ks + rng.integers(1, 300, size=40)], 1)
    ref = O.range_attention(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr, kr)
    out, _ = M.flex_flash_attn_func(q.to(dev), k.to(dev), v.to(dev), tq, tk, 512, 300)
    _cmp(out, ref)


def test_kv_cache_views_and_two_segment_keys(dev):
    """K / V read in place from an interleaved [T, Hkv, 2D] cache, and the key axis split into
    [cache prefix | side buffer] must both equal attention over contiguous concatenated K / V."""
    L, sp, dn, Hq, Hkv, D = 90, 2, 3, 6, 2, 128
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, D, seed=8)
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    ref = O.range_attention(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr, kr)
    cache = torch.cat([k, v], -1).to(dev)  # [T, Hkv, 2D]
    out, _ = M.range_attention(q.to(dev), cache[..., :D], cache[..., D:], tq, tk, L)
    _cmp(out, ref, "in-place cache")
    base = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L)[0]
    assert torch.equal(out, base)  # same arithmetic whatever the strides
    for split in (0, sp * L, sp * L + 37, (sp + dn) * L):  # split inside a tile, at the ends
        big = torch.full((split + 5, Hkv, 2 * D), float("nan"), dtype=torch.bfloat16, device=dev)
        big[:split] = cache[:split]
        tail = cache[split:].clone()
        o2, _ = M.range_attention(q.to(dev), big[:split, :, :D], big[:split, :, D:], tq, tk, L,
                                  k2=tail[..., :D], v2=tail[..., D:], k_split=split)
        assert torch.equal(o2, base), f"split={split}"


def test_flash_attn_func_batched_and_varlen_with_empty_segment(dev):
    g = torch.Generator().manual_seed(9)
    B, Sq, Sk, Hq, Hkv, D = 3, 70, 150, 4, 2, 128
    q = torch.randn(B, Sq, Hq, D, generator=g).bfloat16()
    k = torch.randn(B, Sk, Hkv, D, generator=g).bfloat16()
    v = torch.randn(B, Sk, Hkv, D, generator=g).bfloat16()
    out = M.flash_attn_func(q.to(dev), k.to(dev), v.to(dev))
    assert out.shape == (B, Sq, Hq, D)
    for b in range(B):
        _cmp(out[b], O.range_attention(q[b], k[b], v[b], [[0, Sq]], [[0, Sk]]), f"batch {b}")
    # varlen cross attention: text lengths 20..800, one empty
    Lq = 130
    lens = [800, 0, 20, 413]
    qx = torch.randn(len(lens) * Lq, Hq, D, generator=g).bfloat16()
    kx = torch.randn(sum(lens), Hkv, D, generator=g).bfloat16()
    vx = torch.randn(sum(lens), Hkv, D, generator=g).bfloat16()
    cu_q = torch.arange(0, (len(lens) + 1) * Lq, Lq, dtype=torch.int32)
    cu_k = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32)
    ox = M.flash_attn_varlen_func(qx.to(dev), kx.to(dev), vx.to(dev), cu_q.to(dev), cu_k.to(dev), Lq, 800)
    refx = O.varlen_cross_attention(qx, kx, vx, cu_q, cu_k)
    assert torch.all(ox[Lq:2 * Lq] == 0)
    _cmp(ox, refx)
    with pytest.raises(NotImplementedError):
        M.flash_attn_func(q.to(dev), k.to(dev), v.to(dev), causal=True)


def test_softmax_scale_and_large_scores(dev):
    # unnormalised inputs: scores of magnitude ~50 must not overflow the online softmax
    g = torch.Generator().manual_seed(10)
    q = (torch.randn(256, 2, 128, generator=g) * 4).bfloat16()
    k = (torch.randn(512, 1, 128, generator=g) * 4).bfloat16()
    v = torch.randn(512, 1, 128, generator=g).bfloat16()
    tq, tk = _ranges(dev, [[0, 256]], [[0, 512]])
    for scale in (None, 0.03):
        out, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, 256, softmax_scale=scale)
        assert torch.isfinite(out).all()
        _cmp(out, O.range_attention(q, k, v, [[0, 256]], [[0, 512]], softmax_scale=scale))


def test_apply_rotary_emb_matches_oracle(dev):
    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 37, 3, 128, generator=g)
    ang = torch.randn(37, 48, generator=g)
    cos, sin = ang.cos(), ang.sin()
    y = M.apply_rotary_emb(x.to(dev), cos.to(dev), sin.to(dev))
    ref = O.apply_rope_neox_partial(x, cos, sin)
    assert (y.cpu() - ref).abs().max() < 1e-6
    yb = M.apply_rotary_emb(x.bfloat16().to(dev), cos.to(dev), sin.to(dev))
    assert (yb.float().cpu() - O.apply_rope_neox_partial(x.bfloat16().float(), cos, sin)).abs().max() < 2e-2
    assert torch.equal(yb[..., 96:].cpu(), x.bfloat16()[..., 96:])
    # in place: the tensor itself is rotated; a strided view cannot be (a copy would be rotated instead)
    xi = x.to(dev).clone()
    assert M.apply_rotary_emb(xi, cos.to(dev), sin.to(dev), inplace=True).data_ptr() == xi.data_ptr()
    assert torch.equal(xi, y)
    with pytest.raises(ValueError):
        M.apply_rotary_emb(x.to(dev).transpose(1, 2).contiguous().transpose(1, 2), cos.to(dev), sin.to(dev), inplace=True)


def test_rejects_bad_arguments(dev):
    q = torch.zeros(8, 2, 64, dtype=torch.bfloat16, device=dev)
    r = torch.zeros(1, 2, dtype=torch.int32, device=dev)
    with pytest.raises(M.MagiError) as e:
        M.range_attention(q, q, q, r, r, 8)
    assert e.value.code == -38
    q = torch.zeros(8, 3, 128, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(8, 2, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(M.MagiError):
        M.range_attention(q, k, k, r, r, 8)
    with pytest.raises(TypeError):
        M.range_attention(q.float(), k, k, r, r, 8)


# (the benchmark-size shapes are in tests/test_full_size_gpu.py, for every shipped kernel instantiation)


def test_grouped_output_layout(dev):
    # out as [Tq, groups, heads per group, D] inside a wider buffer: same values as the plain layout, bit for bit,
    # and nothing written outside the destination
    L, sp, dn, Hq, Hkv = 77, 1, 2, 12, 4
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=21)
    qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
    tq, tk = _ranges(dev, qr, kr)
    plain, _ = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L)
    for groups in (4, 2, 12):
        buf = torch.full((dn * L, groups, 2, Hq // groups, 128), 7.0, dtype=torch.bfloat16, device=dev)
        M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, out=buf[:, :, 1], return_lse=False)
        assert torch.equal(buf[:, :, 1].reshape(dn * L, Hq, 128), plain)
        assert torch.all(buf[:, :, 0] == 7.0)
    with pytest.raises(ValueError):
        M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L,
                          out=torch.empty(dn * L, 5, 2, 128, dtype=torch.bfloat16, device=dev))


def test_more_ranges_than_the_in_kernel_ranking_handles(dev):
    # above 256 ranges the kernel skips the longest-first ranking and maps range slots in reverse index order;
    # results must not depend on it (cu_seqlens form: 300 segments, some of them without keys)
    rng = np.random.default_rng(3)
    n = 300
    ql = rng.integers(1, 40, size=n)
    kl = rng.integers(0, 70, size=n)
    kl[::17] = 0
    cu_q = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(kl)]).astype(np.int32)
    Hq, Hkv = 4, 2
    q, k, v = O.synthetic_qkv(int(cu_q[-1]), int(cu_k[-1]), Hq, Hkv, 128, seed=31)
    ref = O.varlen_cross_attention(q, k, v, cu_q, cu_k)
    empty_rows = np.concatenate([np.arange(cu_q[i], cu_q[i + 1]) for i in range(n) if kl[i] == 0])
    # the online-softmax kernel, then the bounded-score kernel behind a stated and behind a measured bound
    for choice in ({}, {"score_bound": 17.0}, {"auto_bound": True}):
        out = M.flash_attn_varlen_func(q.to(dev), k.to(dev), v.to(dev), torch.tensor(cu_q, device=dev),
                                       torch.tensor(cu_k, device=dev), int(ql.max()), int(kl.max()), **choice)
        _cmp(out, ref, f"300 segments {choice}")
        assert torch.count_nonzero(out[torch.tensor(empty_rows, device=dev)]).item() == 0


def test_randomised_shapes_ranges_strides_and_splits(dev):
    """Seeded sweep over head counts, range geometry (arbitrary starts, overlaps between K ranges, gaps between
    Q ranges), strided / interleaved K-V storage and key-axis splits, each compared with the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(int(os.environ.get("MAGI_TEST_SWEEP_CASES", 24))):  # more cases on demand
        Hkv = int(rng.choice([1, 2, 3, 4]))
        G = int(rng.choice([1, 2, 3, 6]))
        Hq = Hkv * G
        n = int(rng.integers(1, 6))
        ql = rng.integers(1, 260, size=n)
        gaps = rng.integers(0, 20, size=n)
        q_start = np.cumsum(gaps + np.concatenate([[0], ql[:-1]]))
        qr = np.stack([q_start, q_start + ql], 1)
        Tq = int(qr[-1, 1] + rng.integers(0, 10))
        Tk = int(rng.integers(1, 700))
        ks = rng.integers(0, Tk, size=n)
        kr = np.stack([ks, np.minimum(Tk, ks + rng.integers(0, 400, size=n))], 1)
        q, k, v = O.synthetic_qkv(Tq, Tk, Hq, Hkv, 128, seed=5000 + case)
        prescaled = case % 5 in (1, 3)  # q carries softmax_scale * log2(e): the oracle then runs with scale ln 2
        if prescaled:
            q = (q.float() * (128 ** -0.5 * math.log2(math.e))).bfloat16()
        ref = O.range_attention(q, k, v, qr, kr, softmax_scale=math.log(2.0) if prescaled else None)
        covered = np.zeros(Tq, bool)
        for a, b in qr:
            covered[a:b] = True
        tq, tk = _ranges(dev, qr, kr)
        layout = case % 3
        if layout == 0:  # separate contiguous K and V
            kd, vd = k.to(dev), v.to(dev)
        elif layout == 1:  # interleaved cache [T, Hkv, 2D]
            cache = torch.cat([k, v], -1).to(dev)
            kd, vd = cache[..., :128], cache[..., 128:]
        else:  # padded rows: token stride larger than Hkv * D
            pad = torch.zeros(Tk, Hkv + 1, 128, dtype=torch.bfloat16, device=dev)
            pad2 = torch.zeros_like(pad)
            pad[:, :Hkv] = k.to(dev)
            pad2[:, :Hkv] = v.to(dev)
            kd, vd = pad[:, :Hkv], pad2[:, :Hkv]
        kw = {}
        if case % 4 == 3:  # key axis = [first split rows | side buffer]
            split = int(rng.integers(0, Tk + 1))
            kw = dict(k2=kd[split:], v2=vd[split:], k_split=split)  # same strides as the first segment
            kd, vd = kd[:split], vd[:split]
        cov = torch.tensor(covered, device=dev)
        # every kernel that can serve the call: the online softmax, the bounded-score kernel behind a stated bound
        # (Cauchy-Schwarz on the tensors themselves) and behind the bound the library measures, and its 32x32x16 form
        factor = 1.0 if prescaled else 128 ** -0.5 * math.log2(math.e)
        bound = 1.01 * factor * q.float().norm(dim=-1).max().item() * k.float().norm(dim=-1).max().item()
        kernels = [("online", {}), ("bounded", {"score_bound": bound}), ("measured", {"auto_bound": True})]
        if prescaled:
            kernels.append(("bounded-mfma32", {"score_bound": bound, "bounded_mfma32": True}))
        for name, choice in kernels:
            out, lse = M.range_attention(q.to(dev), kd, vd, tq, tk, int(ql.max()), q_prescaled=prescaled, **kw, **choice)
            if torch.count_nonzero(ref).item() == 0:  # every range of this case is empty
                assert torch.count_nonzero(out).item() == 0
            else:
                _cmp(out[cov], ref[torch.tensor(covered)], f"case {case} {name}")
            assert torch.count_nonzero(out[~cov]).item() == 0, f"case {case} {name}: uncovered rows written"
            assert torch.isfinite(out).all()


def test_repeated_launches_are_bit_identical(dev):
    """The reference passes deterministic=torch.are_deterministic_algorithms_enabled() to its attention calls
    (dit_module.py:1040, 1062, 1131).  This kernel has one writer per output row and no atomics, so every launch
    gives the same bits, bf16 and fp8 alike, also when other work shares the GPU between the launches."""
    L, dn, sp, Hq, Hkv = 700, 3, 2, 12, 4
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=99)
    tq, tk = _ranges(dev, O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L))
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    first, lse0 = M.range_attention(qd, kd, vd, tq, tk, L)
    bound = 1.01 * (qd.float().norm(dim=-1).max() * kd.float().norm(dim=-1).max()).item() / math.sqrt(128) * math.log2(math.e)
    assert bound <= M.MAGI_SCORE_BOUND_MAX
    first_b, lse0_b = M.range_attention(qd, kd, vd, tq, tk, L, score_bound=bound)  # the bounded-score kernel
    q8, qs = M.quantize_fp8(qd, L)
    k8, ks = M.quantize_fp8(kd, L)
    v8, vs = M.quantize_fp8(vd, L)
    first8, _ = M.range_attention(q8, k8, v8, tq, tk, L, q_scale=qs, k_scale=ks, v_scale=vs, scale_chunk_tokens=L)
    for _ in range(3):
        noise = torch.randn(1 << 20, device=dev).sum()  # unrelated work in between
        again, lse = M.range_attention(qd, kd, vd, tq, tk, L)
        again_b, lse_b = M.range_attention(qd, kd, vd, tq, tk, L, score_bound=bound)
        assert torch.equal(again_b, first_b) and torch.equal(lse_b, lse0_b)
        again8, _ = M.range_attention(q8, k8, v8, tq, tk, L, q_scale=qs, k_scale=ks, v_scale=vs, scale_chunk_tokens=L)
        assert torch.equal(again, first) and torch.equal(lse, lse0) and torch.equal(again8, first8)
        del noise


def test_graph_capture_and_replay(dev):
    """The library allocates nothing, never synchronises and launches on the caller's stream, so an input norm +
    prologue + attention sequence can be captured into a HIP graph (the reference's enable_cuda_graph case).  Every replay, with
    new inputs copied into the static buffers and eager work in between, must equal the eager result bit for bit."""
    S, Hq, Hkv, D, L = 3 * 96, 6, 2, 128, 96
    g = torch.Generator().manual_seed(11)
    mk = lambda *shape: torch.randn(*shape, generator=g).bfloat16().to(dev)
    q_raw, k_raw, v_raw = mk(S, Hq * D), mk(S, Hkv * D), mk(S, Hkv * D)
    rope = torch.randn(S, 96, generator=g).to(dev)
    z = torch.zeros(D, device=dev)
    q = torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev)
    kv = torch.empty(S, Hkv, 2 * D, dtype=torch.bfloat16, device=dev)
    out = torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev)
    tq, tk = _ranges(dev, O.q_ranges_for(3, L), O.default_kvrange(0, 3, L))
    hid = mk(S, Hq * D)  # stands for the layer input; its norm feeds the q side here
    w_ln, b_ln = mk(Hq * D), mk(Hq * D)

    def step(dst):
        M.layer_norm(hid, w_ln, b_ln, 1e-6, out=q_raw)
        M.qk_prologue(q_raw, k_raw, v_raw, rope, z, z, z, z, Hq=Hq, Hkv=Hkv, kv_out=kv, n_cache_rows=S, q_out=q)
        M.range_attention(q, kv[..., :D], kv[..., D:], tq, tk, L, out=dst, return_lse=False)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(out)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(out)
    for rep in range(4):
        for t in (hid, k_raw, v_raw):
            t.copy_(torch.randn(t.shape, generator=g).bfloat16())
        eager = torch.empty_like(out)
        step(eager)
        torch.cuda.synchronize()
        out.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep}"


def test_token_strides_beyond_32_bit_tile_offsets_are_refused(dev):
    """The kernels address a 64-key tile with 32-bit byte offsets from its first row: K / V rows more than 2^23
    elements apart are reported as not implemented (no allocation that large is needed to ask)."""
    Tq, Tk, Hq, Hkv, D = 100, 150, 4, 2, 128
    q, k, v = O.synthetic_qkv(Tq, Tk, Hq, Hkv, D, seed=321)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    tq, tk = _ranges(dev, [[0, 60], [60, 100]], [[0, 150], [17, 90]])
    far_k = kd.as_strided((1, Hkv, D), ((1 << 23) + 8, D, 1))  # (one row: the stride is never followed)
    with pytest.raises(M.MagiError) as e:
        M.range_attention(qd, far_k, far_k, tq, tk, 60, return_lse=False)
    assert e.value.code == -38
    ok_k = kd.as_strided((1, Hkv, D), (1 << 23, D, 1))
    M.range_attention(qd, ok_k, ok_k, tq, _ranges(dev, [[0, 1], [0, 1]])[0], 60, return_lse=False)


@pytest.mark.parametrize("block_m", [384, 128])
def test_every_workgroup_shape_on_the_small_cases(dev, block_m):
    """The library picks 384-row (12-wave) workgroups for grids of many rounds and 128-row ones otherwise, so the
    small parity cases would only ever meet the latter: force each shape (magi_attn_args.q_tile_rows) through
    the chunk-causal cases, a sliding window in shuffled order, the two-segment key axis and a strided cache."""
    for L, dn, sp, Hq, Hkv in CASES:
        q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=4321 + L)
        qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
        tq, tk = _ranges(dev, qr, kr)
        out, lse = M.range_attention(q.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_tile_rows=block_m)
        _cmp(out, O.range_attention(q, k, v, qr, kr), f"block_m={block_m} L={L}")
        assert (lse.cpu() - O.range_attention_lse(q, k, v, qr, kr)).abs().max() < 5e-3
    L, dn, sp, Hq, Hkv = 500, 4, 3, 6, 2
    q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=77)
    qr = O.q_ranges_for(dn, L)[[2, 0, 3, 1]]
    kr = O.noise2clean_kvrange(sp, dn, L, [5, 4, 3, 2], 1, [32, 20, 9, 0], 32)[[2, 0, 3, 1]]
    ref = O.range_attention(q, k, v, qr, kr)
    tq, tk = _ranges(dev, qr, kr)
    cache = torch.cat([k, v], dim=-1).to(dev)  # interleaved [T, Hkv, 2D]: strided K and V views
    out, _ = M.range_attention(q.to(dev), cache[..., :128], cache[..., 128:], tq, tk, L, return_lse=False,
                               q_tile_rows=block_m)
    _cmp(out, ref, f"block_m={block_m} window, strided cache")
    split = 3 * L + 123
    out2, _ = M.range_attention(q.to(dev), cache[:split, :, :128], cache[:split, :, 128:], tq, tk, L,
                                k2=cache[split:, :, :128], v2=cache[split:, :, 128:], k_split=split, return_lse=False,
                                q_tile_rows=block_m)
    _cmp(out2, ref, f"block_m={block_m} two segments")


@pytest.mark.parametrize("block_m", [384, 128])
def test_prescaled_q_flag(dev, block_m):
    """q_prescaled: q carries softmax_scale * log2(e), so q . k is the exp2 exponent.  The 12-wave kernel has an
    instantiation that then accumulates the score MFMAs onto the negated running maximum; every other one runs with
    a unit score scale.  Oracle on the same pre-scaled bf16 q with softmax_scale = ln 2 (2^x = e^(x ln 2)); lse
    likewise.  Includes large scores (no multiply in fp32 is there to absorb them) and a first tile far below 0."""
    import math

    cs = 128 ** -0.5 * math.log2(math.e)
    for L, dn, sp, Hq, Hkv, gain in [(200, 3, 1, 6, 2, 1.0), (77, 2, 2, 3, 1, 1.0), (1536, 3, 0, 24, 8, 1.0),
                                     (300, 2, 1, 4, 4, 12.0), (130, 1, 0, 2, 1, -9.0)]:
        q, k, v = O.synthetic_qkv(dn * L, (sp + dn) * L, Hq, Hkv, 128, seed=515 + L)
        if gain < 0:  # q anti-parallel to every key: all exponents far below the initial maximum 0
            k = (k.float().abs() * 0 + k.float()[:1, :1].sign() * 2).bfloat16().expand_as(k).contiguous()
            q = (-k[:1, :1].float() * abs(gain)).bfloat16().expand(dn * L, Hq, 128).contiguous()
            v = torch.randn(v.shape, generator=torch.Generator().manual_seed(5)).bfloat16()
        qp = (q.float() * (cs * (gain if gain > 0 else 1.0))).bfloat16()
        qr, kr = O.q_ranges_for(dn, L), O.default_kvrange(sp, dn, L)
        tq, tk = _ranges(dev, qr, kr)
        out, lse = M.range_attention(qp.to(dev), k.to(dev), v.to(dev), tq, tk, L, q_prescaled=True, softmax_scale=123.0,
                                     q_tile_rows=block_m)
        ref = O.range_attention(qp, k, v, qr, kr, softmax_scale=math.log(2.0))
        assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
        _cmp(out, ref, f"block_m={block_m} L={L} gain={gain}")
        lse_ref = O.range_attention_lse(qp, k, v, qr, kr, softmax_scale=math.log(2.0))
        assert (lse.cpu() - lse_ref).abs().max() < 5e-3 * max(1.0, lse_ref.abs().max().item() / 50)
