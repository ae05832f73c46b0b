#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one layer-forward of the path on the 720p 24B-style shape: fused prologue
(QK-LayerNorm + 3-D RoPE + bf16 cast + in-place KV-cache append) -> chunk-causal range
attention over [8 cached prefix chunks | 4 denoising chunks] -> T5 cross-attention (two head
norms + varlen attention).  Inputs are synthetic, seeded, and resident in HBM before the
timed region.  One JSON line is printed; `value` is the masked-corrected attention TFLOP/s of
the whole step (core + cross attention FLOPs over the step's wall time), `roofline` prices the
dominant kernel (core attention) against the MI355X dense bf16 MFMA peak from HIP-event
timings of that kernel alone (with the shader clock sampled during the run beside it), and
`cpu_baseline` times the CPU oracle (torch SDPA fp32, same ranges) on a bounded sample of the
same workload on this machine's host cores.
"""
import argparse
import math
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "magi-1_amd"))

import numpy as np
import torch

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA (the vendor figure: 256 CUs x 4 SIMDs x 1024 FLOP/clk at 2.4 GHz)
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0
MFMA_BF16_FLOP_PER_CLK = 256 * 4 * 1024  # whole chip, per shader clock
Q_PREMUL = 128 ** -0.5 * math.log2(math.e)  # softmax_scale * log2(e) at head_dim 128
# Inputs are per-head normalised with unit gain: |q . k| <= 128 * Q_PREMUL (Cauchy-Schwarz), plus 1 % for the
# roundings to bf16, exactly what FullyParallelAttention.score_bounds() derives from the norm parameters.
SCORE_BOUND = 1.01 * 128 * Q_PREMUL
# HBM-side bytes per launch on the 720p workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a
# plain copy of known size in the same run (both counters read 1.00 x the bytes of the copy).  NOT measured in this run:
# the figures and the commands that produced them are in profiles/bench_720p_hbm_traffic_pmc.txt
# (core: the latest of two counter runs; the other read 105.5 GB for the same launch, the fetch side varies that much from
# run to run at the same launch time)
MEASURED_TRAFFIC = {"720p-24B": {"core": 70.87e9 + 1.0617e9, "prologue": 0.7245e9 + 1.4373e9,
                                 "layer_norm": 0.531e9 + 1.0617e9, "cross": 0.5629e9 + 1.0617e9}}
TRAFFIC_SOURCE = "profiles/bench_720p_hbm_traffic_pmc.txt (counter run of this command, not this run)"


class ClockSampler:
    """Samples the shader clock and the socket power through amdsmi from a host thread while kernels run; the
    median of the samples taken inside the timed region is reported.  Absent library or permissions: no figure."""

    def __init__(self, period=0.05):
        import threading

        self.period, self.samples, self._stop, self._thread = period, [], threading.Event(), None
        try:
            import amdsmi

            amdsmi.amdsmi_init()
            self.smi, self.h = amdsmi, amdsmi.amdsmi_get_processor_handles()[0]
            self._read()
        except Exception:  # noqa: BLE001 - any failure means "no clock figure"
            self.smi = None

    def _read(self):
        m = self.smi.amdsmi_get_gpu_metrics_info(self.h)
        clk = m.get("current_gfxclks") or [m.get("current_gfxclk")]
        clk = [c for c in clk if isinstance(c, (int, float)) and 0 < c < 10000]
        pw = m.get("current_socket_power") or m.get("average_socket_power")
        return (float(np.mean(clk)) if clk else None, float(pw) if isinstance(pw, (int, float)) and pw < 1e5 else None)

    def _run(self):
        while not self._stop.is_set():
            try:
                self.samples.append(self._read())
            except Exception:  # noqa: BLE001
                pass
            self._stop.wait(self.period)

    def __enter__(self):
        if self.smi is not None:
            import threading

            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self._thread is not None:
            self._thread.join()

    def result(self, last_fraction=1.0):
        """Medians over the samples (last_fraction < 1: over the last part of them only; the driver's metrics lag the
        load by a few hundred milliseconds)."""
        keep = self.samples[int(len(self.samples) * (1.0 - last_fraction)):]
        clk = [c for c, _ in keep if c]
        pw = [p for _, p in keep if p]
        return (float(np.median(clk)) if clk else None, float(np.median(pw)) if pw else None, len(self.samples))

WORKLOADS = {
    # name: (T_lat frames per chunk, H, W, denoise chunks, prefix chunks, Hq, Hkv)
    "720p-24B": (6, 45, 80, 4, 8, 48, 8),
    "480p-4.5B": (6, 30, 52, 4, 4, 24, 8),
    # one rank's share of the 720p layer under an 8-way head split (one KV head with its 6 query heads, all tokens)
    "720p-24B-head-share": (6, 45, 80, 4, 8, 6, 1),
}


def build_inputs(name, dev, seed=1234, kv_window="default"):
    import magi_attn as M
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    fr, H, W, dn, sp, Hq, Hkv = WORKLOADS[name]
    D = 128
    L = fr * H * W
    S = dn * L
    g = torch.Generator(device=dev).manual_seed(seed + 2000)
    rn = lambda *shape: torch.randn(*shape, device=dev, generator=g).bfloat16()
    rope_mod = LearnableRotaryEmbeddingCat(128, device=dev)
    zeros = torch.zeros(D, device=dev)
    # KV cache for the whole window, prefix filled by the same prologue (clean chunks, same distribution)
    cache = torch.empty((sp + dn) * L, Hkv, 2 * D, dtype=torch.bfloat16, device=dev)
    for c0 in range(0, sp, 4):
        n = min(4, sp - c0)
        rope_p = rope_mod.get_embed_for_forward(n * fr, H, W, c0, n)
        k_raw, v_raw = rn(n * L, Hkv * D), rn(n * L, Hkv * D)
        M.qk_prologue(k_raw[:, :0], k_raw, v_raw, rope_p, None, None, zeros, zeros, Hq=0, Hkv=Hkv,
                      kv_out=cache[c0 * L:], n_cache_rows=n * L)
    inp = dict(
        name=name, L=L, S=S, dn=dn, sp=sp, Hq=Hq, Hkv=Hkv, D=D, cache=cache, zeros=zeros,
        q_raw=rn(S, Hq * D), k_raw=rn(S, Hkv * D), v_raw=rn(S, Hkv * D), qx_raw=rn(S, Hq, D),
        rope=rope_mod.get_embed_for_forward(dn * fr, H, W, sp, dn),
        q=torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev),
        out=torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev),
        xout=torch.empty(S, Hq, D, dtype=torch.bfloat16, device=dev),
    )
    from magi_attn import ranges as R

    inp["q_ranges"] = R.q_ranges_from_chunks(dn, L, device=dev)
    if kv_window == "default":  # every chunk attends to all chunks up to itself (the configuration the metric is quoted on)
        kr = R.generate_default_kvrange(sp, dn, L)
    else:  # the shipped sliding window: noise2clean_kvrange [5, 4, 3, 2] over 32 steps, chunks 8 steps apart
        kr = R.generate_noise2clean_kvrange(sp, dn, L, [5, 4, 3, 2], 1, [8 * (dn - 1 - j) for j in range(dn)][:dn], 32)
    inp["k_ranges_host"] = kr.numpy()
    inp["k_ranges"] = kr.to(dev)
    # T5 side: valid lengths uniform in [20, 800] per chunk, K | V interleaved per head as the projection emits them
    rs = np.random.default_rng(seed)
    lens = rs.integers(20, 801, size=dn)
    inp["t5_lens"] = lens
    inp["cu_q"] = torch.arange(0, (dn + 1) * L, L, dtype=torch.int32, device=dev)
    inp["cu_k"] = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=dev)
    inp["kvx"] = rn(int(lens.sum()), Hkv, 2 * D)
    return inp


def flops_of(inp):
    L, dn, sp, Hq, D = inp["L"], inp["dn"], inp["sp"], inp["Hq"], inp["D"]
    core = 4.0 * D * Hq * sum(L * float(e - b) for b, e in inp["k_ranges_host"])
    cross = 4.0 * D * Hq * float(sum(L * int(n) for n in inp["t5_lens"]))
    return core, cross


def prologue_bytes(inp):
    S, Hq, Hkv, D = inp["S"], inp["Hq"], inp["Hkv"], inp["D"]
    return 2 * (S * Hq * D * 2) + 2 * (S * Hkv * 2 * D * 2) + S * 96 * 4


CORE_BOUND = {"value": SCORE_BOUND}  # (--core-kernel online sets it to 0: no promise, online softmax)


def run_step(inp, ev=None):
    """One layer-forward of the hot path, as FullyParallelAttention.forward issues it.
    ev: optional dict of event pairs to record around kernels."""
    import magi_attn as M

    L, sp, D = inp["L"], inp["sp"], inp["D"]
    cache = inp["cache"]
    z = inp["zeros"]

    def rec(key, which):
        if ev is not None:
            ev[key][which].record()

    # the prologue folds softmax_scale * log2(e) into q ahead of q's rounding to bf16; QK-normed scores are bounded
    # (score_bound, from the norm parameters), so the attention kernel runs without a running maximum
    rec("prologue", 0)
    M.qk_prologue(inp["q_raw"], inp["k_raw"], inp["v_raw"], inp["rope"], z, z, z, z, Hq=inp["Hq"], Hkv=inp["Hkv"],
                  kv_out=cache[sp * L:], n_cache_rows=inp["S"], q_out=inp["q"], q_premul=Q_PREMUL)
    rec("prologue", 1)
    rec("core", 0)
    M.range_attention(inp["q"], cache[..., :D], cache[..., D:], inp["q_ranges"], inp["k_ranges"], L,
                      out=inp["out"], return_lse=False, q_prescaled=True, score_bound=CORE_BOUND["value"])
    rec("core", 1)
    # cross attention: k norm (a few thousand text tokens), then the attention kernel on the RAW qx projection with
    # the q norm applied while q is loaded
    rec("cross", 0)
    kx = M.head_norm(inp["kvx"][..., :D], z, z)
    rec("cross_attn", 0)
    M.range_attention(inp["qx_raw"], kx, inp["kvx"][..., D:], inp["cu_q"], inp["cu_k"], L, 800,
                      ranges_mode=M.MAGI_RANGES_CU, out=inp["xout"], return_lse=False, score_bound=SCORE_BOUND,
                      q_norm=(z, z, 1e-6))
    rec("cross_attn", 1)
    rec("cross", 1)


def fp32_rows_reference(q, k, v, k_ranges, L, rows_per_chunk, scale, seed=0):
    """fp32 attention of a random sample of query rows per chunk (all heads, full key ranges), on the GPU with
    plain matmuls; rows are independent, so this is exact for the sampled rows.  q [S, Hq, D] (any float dtype),
    k / v [T, Hkv, D] -> (row indices [n], reference [n, Hq, D] fp32)."""
    S, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    rs = np.random.default_rng(seed)
    idx, refs = [], []
    for i, (kb, ke) in enumerate(k_ranges):
        rows = torch.tensor(np.sort(rs.choice(L, rows_per_chunk, replace=False)) + i * L, device=q.device)
        ref = torch.empty(rows_per_chunk, Hq, D, device=q.device)
        for hk in range(Hkv):
            sc = torch.einsum("rgd,kd->rgk", q[rows, hk * G:(hk + 1) * G].float(), k[kb:ke, hk].float()) * scale
            ref[:, hk * G:(hk + 1) * G] = torch.einsum("rgk,kd->rgd", torch.softmax(sc, -1), v[kb:ke, hk].float())
        idx.append(rows)
        refs.append(ref)
    return torch.cat(idx), torch.cat(refs)


def deviation(out, ref):
    a, b = out.double().flatten(), ref.double().flatten()
    return {"cosine": round((torch.dot(a, b) / (a.norm() * b.norm())).item(), 6),
            "max_abs": round((a - b).abs().max().item(), 6), "ref_abs_max": round(b.abs().max().item(), 5)}


def fp8_leg(inp, core_fl, bf16_tflops, steps, ref_rows, ref):
    """The same core attention with Q / K / V quantised to e4m3 (per-(chunk, head) absmax scales), in both scale
    modes of the kernel: kernel-only HIP-event timing, throughput against the fp8 dense peak and against the bf16
    kernel, and the deviation from fp32 attention of the ORIGINAL bf16 tensors on a sample of query rows."""
    import magi_attn as M

    L, D = inp["L"], inp["D"]
    cache = inp["cache"]
    res = {"kernel": "attn_fwd_fp8_kernel", "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
           "accuracy_reference": f"fp32 attention of {ref.shape[0]} sampled query rows x all heads on the bf16 tensors"}
    out8 = torch.empty_like(inp["out"])
    S, sp, Hq, Hkv = inp["S"], inp["sp"], inp["Hq"], inp["Hkv"]
    z = inp["zeros"]
    for mode in ("pow2_prescaled", "generic"):
        pow2 = mode == "pow2_prescaled"
        # pow2_prescaled (what the layer module runs): power-of-two scales on the MFMA's block-scale operands,
        # softmax_scale * log2(e) already in q; generic: any positive scales, q scaled back so that the kernel's own
        # softmax scale applies.  Cached prefix: quantised from the bf16 cache (absmax scales per chunk and head).
        k8, ks = M.quantize_fp8(cache[..., :D], L, pow2_scales=pow2)
        v8, vs = M.quantize_fp8(cache[..., D:], L, pow2_scales=pow2)
        if pow2:
            # this step's rows as FullyParallelAttention(attention_dtype="fp8") prepares them, two launches from the
            # raw projections on: the prologue writes q and k as e4m3 with constant scales from the norm-parameter
            # bound (gamma = 1, beta = 0 here: no element of a normed row exceeds sqrt(D)), k into the cache rows;
            # one launch takes v's absmax scales and quantises it
            q_sc, k_sc = M.pow2_scale_for(Q_PREMUL * math.sqrt(D)), M.pow2_scale_for(math.sqrt(D))
            q8 = torch.empty(S, Hq, D, dtype=torch.float8_e4m3fn, device=k8.device)
            qs = torch.full((S // L, Hq), q_sc, device=k8.device)
            ks[sp:] = k_sc

            def prepare():
                M.qk_prologue_fp8(inp["q_raw"], inp["k_raw"], inp["rope"], z, z, z, z, Hq=Hq, Hkv=Hkv, q_scale=q_sc,
                                  k_scale=k_sc, q_premul=Q_PREMUL, q_out=q8, k_out=k8[sp * L:], n_cache_rows=S)
                M.quantize_fp8_split(inp["v_raw"].view(S, Hkv, D), L, S, v8[sp * L:], vs[sp:], None, None, pow2_scales=True)

            prepare()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                prepare()
            e1.record()
            torch.cuda.synchronize()
            prep_ms = e0.elapsed_time(e1) / steps
            prep_bytes = S * Hq * D * 3 + S * Hkv * D * 3 * 2 + S * 96 * 4  # raw bf16 in, e4m3 out, rotary table
            res["operand_preparation"] = {
                "launches": 2, "kernels": "prologue_kernel<., e4m3> + quantize_groups_kernel", "ms": round(prep_ms, 4),
                "bytes": prep_bytes, "achieved": round(prep_bytes / (prep_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                "frac": round(prep_bytes / (prep_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        else:
            q8, qs = M.quantize_fp8(inp["q"], L, premul=1.0 / Q_PREMUL)
        for fast in ((False, True) if pow2 else (False,)):  # the fast exp2 variant runs on the same operands
            kw = dict(q_scale=qs, k_scale=ks, v_scale=vs, scale_chunk_tokens=L, out=out8, return_lse=False,
                      fp8_pow2_prescaled=pow2, fp8_fast_exp2=fast)
            M.range_attention(q8, k8, v8, inp["q_ranges"], inp["k_ranges"], L, **kw)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                M.range_attention(q8, k8, v8, inp["q_ranges"], inp["k_ranges"], L, **kw)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / steps
            tf = core_fl / (ms * 1e-3) / 1e12
            res[mode + ("_fast_exp2" if fast else "")] = {
                "achieved": round(tf, 2), "frac": round(tf / PEAK_FP8_TFLOPS, 4), "ms": round(ms, 3),
                "speedup_vs_bf16": round(tf / bf16_tflops, 3), "vs_fp32": deviation(out8[ref_rows], ref)}
        del q8, k8, v8
    # headline: the exact exponential in fp32 (what the layer module runs by default); the piecewise-linear exp2 is
    # an opt-in approximation and stays a separate, labelled entry
    res["mode_of_the_layer_module"] = "pow2_prescaled"
    res["achieved"], res["frac"], res["ms"], res["speedup_vs_bf16"] = (res["pow2_prescaled"][k_] for k_ in
                                                                       ("achieved", "frac", "ms", "speedup_vs_bf16"))
    res["opt_in_approximation"] = "pow2_prescaled_fast_exp2"
    return res


def cpu_baseline(inp, rows_per_chunk=1536):
    """CPU oracle (torch SDPA fp32, one call per range) on a bounded sample of the workload:
    the first rows_per_chunk queries of every denoising chunk, the 6 (= Hq/Hkv) q heads of KV
    head 0, full key ranges.  Heads and rows are independent, so this is a slice of the real job.
    One warm-up run, then the best of three."""
    from oracle import magi_oracle as O

    L, dn, sp, Hq, Hkv, D = inp["L"], inp["dn"], inp["sp"], inp["Hq"], inp["Hkv"], inp["D"]
    G = Hq // Hkv
    rows = min(rows_per_chunk, L)
    idx = torch.cat([torch.arange(j * L, j * L + rows) for j in range(dn)])
    q = inp["q"][idx.to(inp["q"].device), :G].float().cpu()
    k = inp["cache"][:, :1, :D].float().cpu()
    v = inp["cache"][:, :1, D:].float().cpu()
    qr = np.array([[j * rows, (j + 1) * rows] for j in range(dn)])
    kr = inp["k_ranges_host"]
    fl = O.attention_flops(qr, kr, G, D)
    torch.set_num_threads(os.cpu_count() if os.cpu_count() and os.cpu_count() <= 64 else torch.get_num_threads())
    times = []
    for _ in range(4):  # (the first is the warm-up)
        t0 = time.perf_counter()
        o = O.range_attention(q, k, v, qr, kr, softmax_scale=math.log(2.0))  # q carries softmax_scale * log2(e)
        times.append(time.perf_counter() - t0)
    dt = min(times[1:])
    return dict(value=fl / dt / 1e12, unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"first {rows} q rows of each of the {dn} chunks x {G} q heads of kv head 0, full key ranges, "
                       f"{fl:.3e} FLOP; warm-up + best of 3: {dt:.2f} s (runs {', '.join(f'{t:.2f}' for t in times)}; "
                       f"torch {torch.__version__} CPU SDPA fp32)"), o, idx


def layer_norm_leg(inp, steps, traffic=None):
    """The LayerNorm of the layer input (the step ahead of the projections that feed the prologue), kernel-only:
    reported beside the headline, not part of `value`.  Re-uses the raw-q buffer as the hidden states and the
    cross-attention output buffer for the result (nothing reads that buffer afterwards)."""
    import magi_attn as M

    S, hidden = inp["S"], inp["Hq"] * inp["D"]
    x, y = inp["q_raw"], inp["xout"].view(S, hidden)
    w = torch.ones(hidden, dtype=torch.bfloat16, device=x.device)
    b = torch.zeros(hidden, dtype=torch.bfloat16, device=x.device)
    for _ in range(2):
        M.layer_norm(x, w, b, 1e-6, out=y)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        M.layer_norm(x, w, b, 1e-6, out=y)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    gbs = 2 * S * hidden * 2 / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "kernel": "layer_norm_kernel", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS,
            "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": traffic, "ms": round(ms, 4)}


def projection_leg(inp, steps):
    """The four projections that feed the prologue (q, k, v and the cross-attention q: [S, hidden] x
    [2 (Hq + Hkv) 128, hidden]^T), kernel-only and beside the headline: the library GEMM followed by the prologue
    kernel (what the layer module runs) against the hand-written GEMM whose epilogue is the prologue
    (magi_qkv_proj_prologue, the module's fused_projection option).  Same inputs, destinations of the step."""
    import magi_attn as M

    S, Hq, Hkv, D = inp["S"], inp["Hq"], inp["Hkv"], inp["D"]
    hidden = Hq * D
    dev = inp["q"].device
    g = torch.Generator(device=dev).manual_seed(77)
    x = inp["q_raw"]  # [S, hidden] bf16 N(0, 1): stands for the normalised hidden states
    w = (torch.randn((2 * Hq + 2 * Hkv) * D, hidden, device=dev, generator=g) * hidden ** -0.5).bfloat16()
    raw = torch.empty(S, w.shape[0], dtype=torch.bfloat16, device=dev)
    z = inp["zeros"]
    # destinations of their own (the step's q and cache rows still serve the CPU baseline's comparison)
    q_dst = torch.empty_like(inp["q"])
    kv_dst = torch.empty(S, Hkv, 2 * D, dtype=torch.bfloat16, device=dev)
    nq, nk = Hq * D, Hkv * D
    flop = 2.0 * S * hidden * w.shape[0]

    def two_step():
        torch.mm(x, w.t(), out=raw)
        M.qk_prologue(raw[:, :nq], raw[:, nq:nq + nk], raw[:, nq + nk:nq + 2 * nk], inp["rope"], z, z, z, z, Hq=Hq, Hkv=Hkv,
                      kv_out=kv_dst, n_cache_rows=S, q_out=q_dst, q_premul=Q_PREMUL)

    def one_launch():
        M.qkv_proj_prologue(x, w, inp["rope"], z, z, z, z, Hq=Hq, Hkv=Hkv, Hqx=Hq, kv_out=kv_dst, n_cache_rows=S,
                            q_out=q_dst, qx_out=inp["xout"], q_premul=Q_PREMUL)

    # the reference's fp8_quant layers: per linear (q, k, v, qx) its own input quantiser (div_clamp_to, one pass over x)
    # and the library's fp8 GEMM, then the prologue on the four results
    from magi_attn.module import PerTensorQuantizedFp8Linear
    lins = []
    row = 0
    for n_out in (nq, nk, nk, nq):
        lin = torch.nn.Linear(hidden, n_out, bias=False, dtype=torch.bfloat16, device=dev)
        lin.weight.data = w[row:row + n_out]
        lins.append(PerTensorQuantizedFp8Linear.from_linear(lin, 6.0))
        row += n_out

    def fp8_linears():
        qr_, kr_, vr_, _ = (l_(x) for l_ in lins)
        M.qk_prologue(qr_, kr_, vr_, inp["rope"], z, z, z, z, Hq=Hq, Hkv=Hkv, kv_out=kv_dst, n_cache_rows=S, q_out=q_dst,
                      q_premul=Q_PREMUL)

    res = {"flop": flop, "unit": "TFLOP/s", "peak": PEAK_BF16_TFLOPS}
    for name, fn in (("library_gemm", lambda: torch.mm(x, w.t(), out=raw)), ("library_gemm_then_prologue", two_step),
                     ("gemm_with_prologue_epilogue", one_launch),
                     ("fp8_quant_linears_then_prologue", fp8_linears)):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        tf = flop / (ms * 1e-3) / 1e12
        res[name] = {"ms": round(ms, 3), "achieved": round(tf, 1), "frac": round(tf / PEAK_BF16_TFLOPS, 4)}
    res["what_the_layer_module_runs"] = "library_gemm_then_prologue"
    return res


def timed(fn, steps, warmup=1):
    """Average milliseconds of fn() over `steps` calls on the current stream (HIP events)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def mfma_ceiling_leg(dev):
    """What a loop of nothing but MFMAs sustains on THIS box, in this process, after the timed region: the three MFMA
    shapes (bf16 16x16x32 = the bounded-score attention kernel's instruction, bf16 32x32x16, fp8 32x32x64 = the fp8
    kernel's, fp8 16x16x128) on all-zero operands and
    on operands drawn from N(0, 1) activations (bf16) / their e4m3 quantisation (fp8), one wave per SIMD, ~30 ms
    launches, with the shader clock and the socket power sampled while each runs.  The part is power limited: the
    random-operand rate, not the 2.4 GHz figure, is what a kernel made of these MFMAs can reach here.
    Measurement-only helper library (libmagi_probe.so, built by the same Makefile; the product path never loads it)."""
    import ctypes as C

    path = os.path.join(ROOT, "magi-1_amd", "magi_attn", "libmagi_probe.so")
    if not os.path.exists(path):
        return {"error": "libmagi_probe.so is not built (make -C magi-1_amd/csrc)"}
    lib = C.CDLL(path)
    lib.magi_probe_mfma_only.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                         C.POINTER(C.c_float), C.POINTER(C.c_double)]
    lib.magi_probe_mfma_only.restype = C.c_int
    g = torch.Generator(device=dev).manual_seed(4242)
    x = torch.randn(1 << 22, device=dev, generator=g)
    words_bf16 = x[: 1 << 21].bfloat16().view(torch.int32)                          # 2^20 words of two bf16 values
    words_fp8 = (x * (448.0 / x.abs().max())).to(torch.float8_e4m3fn).view(torch.int32)  # 2^20 words of four e4m3 values
    sink = torch.empty(256 * 256, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"what": "MFMA-only loop, one wave per SIMD, operands in registers, 100 launches of 20-30 ms back to back after a "
                   "warm-up (2-3 s per entry: the socket power the driver reports is an average over about a second; clock "
                   "and power: median of the last 30 % of the samples); "
                   "random = N(0,1) activations as bf16 / as e4m3 scaled to absmax 448",
           "unit": "TFLOP/s"}
    for name, kind, words in (("bf16_32x32x16", 0, words_bf16), ("bf16_16x16x32", 1, words_bf16), ("fp8_32x32x64", 2, words_fp8),
                              ("fp8_16x16x128", 3, words_fp8)):
        entry = {}
        for label, ptr in (("zero_operands", None), ("random_operands", words.data_ptr())):
            ms, fl = C.c_float(0), C.c_double(0)
            # (2-3 s per entry so that the sampled clock and power are this loop's, not its predecessor's)
            with ClockSampler(period=0.02) as smp:
                rc = lib.magi_probe_mfma_only(kind, ptr, sink.data_ptr(), 24000, 100, stream,
                                              C.byref(ms), C.byref(fl))
            if rc != 0:
                entry[label] = {"error": rc}
                continue
            clk, pw, _ = smp.result(last_fraction=0.3)
            entry[label] = {"tflops": round(fl.value / (ms.value * 1e-3) / 1e12, 1), "ms_per_launch": round(ms.value, 2),
                            "shader_clock_mhz": None if clk is None else round(clk), "socket_power_w": None if pw is None else round(pw)}
        out[name] = entry
    return out


def hbm_ceiling_leg(inp, dev):
    """What kernels of nothing but 16-byte loads and stores sustain on THIS box's memory, in this process, after the
    timed region: a copy, a read-only and a write-only pass over ~1 GB (the size of the layer's tensors), 20 launches
    each.  The streaming kernels of the path (prologue, layer norm, fp8 operand preparation) are reported against the
    copy rate beside the nominal 8 TB/s.  Same measurement-only helper library as the MFMA ceiling."""
    import ctypes as C

    path = os.path.join(ROOT, "magi-1_amd", "magi_attn", "libmagi_probe.so")
    if not os.path.exists(path):
        return {"error": "libmagi_probe.so is not built (make -C magi-1_amd/csrc)"}
    lib = C.CDLL(path)
    if not hasattr(lib, "magi_probe_stream"):
        return {"error": "libmagi_probe.so predates magi_probe_stream (make -C magi-1_amd/csrc)"}
    lib.magi_probe_stream.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    lib.magi_probe_stream.restype = C.c_int
    src, dst = inp["cache"], inp["xout"]  # (xout is scratch by now: nothing reads the cross-attention output afterwards)
    nbytes = min(src.numel() * src.element_size(), dst.numel() * dst.element_size()) // 16 * 16
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {"what": "16 bytes per lane, one contiguous piece per workgroup; GB/s counts every byte read and every byte written",
           "unit": "GB/s", "bytes": nbytes}
    for name, kind, moved in (("copy", 0, 2 * nbytes), ("read_only", 1, nbytes), ("write_only", 2, nbytes)):
        ms = C.c_float(0)
        rc = lib.magi_probe_stream(kind, src.data_ptr(), dst.data_ptr(), nbytes, 20, stream, C.byref(ms))
        out[name] = {"error": rc} if rc != 0 else {"gbs": round(moved / (ms.value * 1e-3) / 1e9, 1), "ms": round(ms.value, 4)}
    return out


def secondary_legs(inp, dev, steps):
    """Core-attention launches the headline does not time, kernel only, a few steps each: the online-softmax kernel a
    caller gets who neither states a score bound nor lets the library measure one (unscaled q), the bounded kernel
    fed with unscaled q and a bound (it scales q while loading it), the reference's unchanged call with the bound
    measured by the library, the shipped sliding window on the same layer, and the 480p 4.5B-style layer."""
    import magi_attn as M
    from magi_attn import ranges as R

    L, sp, dn, D, S, Hq, Hkv = inp["L"], inp["sp"], inp["dn"], inp["D"], inp["S"], inp["Hq"], inp["Hkv"]
    cache, z = inp["cache"], inp["zeros"]
    core_fl, _ = flops_of(inp)
    k, v = cache[..., :D], cache[..., D:]
    q_unscaled = torch.empty_like(inp["q"])
    M.qk_prologue(inp["q_raw"], inp["k_raw"], inp["v_raw"], inp["rope"], z, z, z, z, Hq=Hq, Hkv=Hkv,
                  kv_out=cache[sp * L:], n_cache_rows=S, q_out=q_unscaled)  # (k, v rows rewritten with the same values)
    res = {}

    def entry(ms, fl, kernel):
        tf = fl / (ms * 1e-3) / 1e12
        return {"kernel": kernel, "ms": round(ms, 3), "achieved": round(tf, 2), "unit": "TFLOP/s",
                "frac": round(tf / PEAK_BF16_TFLOPS, 4), "flops": fl}

    ms = timed(lambda: M.range_attention(q_unscaled, k, v, inp["q_ranges"], inp["k_ranges"], L, out=inp["out"],
                                         return_lse=False), steps)
    res["online_softmax_unscaled_q"] = entry(ms, core_fl, "attn_fwd_bf16_kernel (32 rows per wavefront, running maximum)")
    ms = timed(lambda: M.range_attention(q_unscaled, k, v, inp["q_ranges"], inp["k_ranges"], L, out=inp["out"],
                                         return_lse=False, score_bound=SCORE_BOUND), steps)
    res["bounded_unscaled_q_scale_on_load"] = entry(ms, core_fl, "attn_fwd_bf16_x16_kernel (q scaled while loaded)")
    # the reference's own call, nothing added: unscaled q, no bound.  The library measures max|q| max|k| in two passes and
    # both kernels are launched behind them (MAGI_ATTN_AUTO_BOUND); the time is that of all five launches.
    assert M.functional._measuring_a_bound_pays(q_unscaled, k, dn, L, (sp + dn) * L)
    ms = timed(lambda: M.range_attention(q_unscaled, k, v, inp["q_ranges"], inp["k_ranges"], L, (sp + dn) * L, out=inp["out"],
                                         return_lse=False, auto_bound=True), steps)
    res["reference_call_unchanged_measured_bound"] = entry(
        ms, core_fl, "row_norm_max_kernel x 2 + attn_fwd_bf16_x16_kernel (selected on the device) + attn_fwd_bf16_kernel (returns at once)")
    del q_unscaled
    # the bounded kernel's 32x32x16-MFMA form (MAGI_ATTN_BOUNDED_MFMA32) on the headline's inputs: same box, same run
    ms = timed(lambda: M.range_attention(inp["q"], k, v, inp["q_ranges"], inp["k_ranges"], L, out=inp["out"],
                                         return_lse=False, q_prescaled=True, score_bound=SCORE_BOUND, bounded_mfma32=True), steps)
    res["bounded_mfma_32x32x16_form"] = entry(ms, core_fl, "attn_fwd_bf16_w64_kernel (64 rows per wavefront on v_mfma_f32_32x32x16)")
    # restore the headline's output (the accuracy legs compare inp["out"])
    M.range_attention(inp["q"], k, v, inp["q_ranges"], inp["k_ranges"], L, out=inp["out"], return_lse=False,
                      q_prescaled=True, score_bound=SCORE_BOUND)
    if inp["name"] == "720p-24B":
        kr = R.generate_noise2clean_kvrange(sp, dn, L, [5, 4, 3, 2], 1, [8 * (dn - 1 - j) for j in range(dn)][:dn], 32)
        fl = 4.0 * D * Hq * sum(L * float(e - b) for b, e in kr.numpy())
        krd = kr.to(dev)
        scratch = torch.empty_like(inp["out"])
        ms = timed(lambda: M.range_attention(inp["q"], k, v, inp["q_ranges"], krd, L, out=scratch, return_lse=False,
                                             q_prescaled=True, score_bound=SCORE_BOUND), steps)
        res["sliding_window_noise2clean_5_4_3_2"] = entry(ms, fl, "attn_fwd_bf16_x16_kernel")
        res["sliding_window_noise2clean_5_4_3_2"]["k_ranges"] = kr.numpy().tolist()
        del scratch
        small = build_inputs("480p-4.5B", dev)
        fl, _ = flops_of(small)
        run_step(small)
        ev = [{k_: (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
               for k_ in ("prologue", "core", "cross", "cross_attn")} for _ in range(steps)]
        torch.cuda.synchronize()
        for s_ in range(steps):
            run_step(small, ev[s_])
        torch.cuda.synchronize()
        ms = float(np.mean([e["core"][0].elapsed_time(e["core"][1]) for e in ev]))
        res["layer_480p_4.5B"] = entry(ms, fl, "attn_fwd_bf16_x16_kernel")
        res["layer_480p_4.5B"]["workload"] = (f"Q {small['S']} tok x {small['Hq']} heads over K/V "
                                              f"{(small['sp'] + small['dn']) * small['L']} tok x {small['Hkv']} heads")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="720p-24B", choices=sorted(WORKLOADS))
    ap.add_argument("--kv-window", default="default", choices=["default", "noise2clean"],
                    help="key ranges: all chunks up to the query's own (default) or the shipped sliding window")
    ap.add_argument("--core-kernel", default="bounded", choices=["bounded", "online"],
                    help="core attention: the bounded-score 64-row kernel the layer module uses (default) or, by "
                         "withholding the score bound, the online-softmax 32-row kernel that generic callers get")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the MFMA-only ceiling measurement")
    ap.add_argument("--no-secondary", action="store_true", help="skip the secondary core-attention timings")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fp8", action="store_true")
    ap.add_argument("--no-projection", action="store_true", help="skip the projection GEMM leg")
    ap.add_argument("--no-accuracy", action="store_true", help="skip the fp32 sampled-row check of the bf16 output")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run one plain device copy of known size (for scaling FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.core_kernel == "online":
        CORE_BOUND["value"] = 0.0
    inp = build_inputs(args.workload, dev, kv_window=args.kv_window)
    core_fl, cross_fl = flops_of(inp)

    for _ in range(args.warmup):
        run_step(inp)
    torch.cuda.synchronize()
    keys = ("prologue", "core", "cross", "cross_attn")
    evs = [{k: (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for k in keys}
           for _ in range(args.steps)]
    torch.cuda.synchronize()
    with ClockSampler() as sampler:
        t0 = time.perf_counter()
        for s in range(args.steps):
            run_step(inp, evs[s])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    clock_mhz, power_w, n_samples = sampler.result()
    ms_per_step = dt / args.steps * 1e3
    kern_ms = {k: float(np.mean([e[k][0].elapsed_time(e[k][1]) for e in evs])) for k in keys}

    value = (core_fl + cross_fl) / (ms_per_step * 1e-3) / 1e12
    core_tflops = core_fl / (kern_ms["core"] * 1e-3) / 1e12
    pro_gbs = prologue_bytes(inp) / (kern_ms["prologue"] * 1e-3) / 1e9
    cross_tflops = cross_fl / (kern_ms["cross_attn"] * 1e-3) / 1e12
    cross_bytes = 2 * inp["S"] * inp["Hq"] * inp["D"] * 2 + 2 * int(inp["t5_lens"].sum()) * inp["Hkv"] * inp["D"] * 2
    cross_gbs = cross_bytes / (kern_ms["cross_attn"] * 1e-3) / 1e9
    traffic = MEASURED_TRAFFIC.get(args.workload, {})
    result = {
        "metric": "attention TFLOP/s (masked-corrected), chunk-causal layer, 1 GPU",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{args.workload} layer-forward: prologue + chunk-causal attention "
                               f"(Q {inp['S']} tok x {inp['Hq']} heads over K/V {(inp['sp'] + inp['dn']) * inp['L']} tok x "
                               f"{inp['Hkv']} heads, d=128, {inp['sp']} cached + {inp['dn']} denoising chunks of {inp['L']}) "
                               f"+ T5 cross-attention (lens {inp['t5_lens'].tolist()})"
                               + ("" if args.kv_window == "default" else f", sliding-window key ranges {inp['k_ranges_host'].tolist()}"),
                   "core_flops": core_fl, "cross_flops": cross_fl},
        "roofline": {"bound": "mfma", "kernel": "attn_fwd_bf16_x16_kernel" if args.core_kernel == "bounded" else "attn_fwd_bf16_kernel", "achieved": round(core_tflops, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(core_tflops / PEAK_BF16_TFLOPS, 4),
                     "traffic": traffic.get("core") if args.kv_window == "default" else None,
                     "traffic_source": TRAFFIC_SOURCE, "ms": round(kern_ms["core"], 3),
                     "score_bound": round(CORE_BOUND["value"], 3),
                     # the step is >= 99 % core launch, so the clock sampled over the timed region is its clock
                     "shader_clock_mhz": None if clock_mhz is None else round(clock_mhz, 0),
                     "socket_power_w": None if power_w is None else round(power_w, 0), "clock_samples": n_samples,
                     "peak_at_measured_clock": None if clock_mhz is None else round(MFMA_BF16_FLOP_PER_CLK * clock_mhz * 1e6 / 1e12, 1),
                     "frac_of_peak_at_measured_clock": None if clock_mhz is None else
                     round(core_tflops / (MFMA_BF16_FLOP_PER_CLK * clock_mhz * 1e6 / 1e12), 4)},
        "roofline_prologue": {"bound": "hbm", "kernel": "prologue_kernel", "achieved": round(pro_gbs, 1),
                              "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(pro_gbs / PEAK_HBM_GBS, 4),
                              "traffic": traffic.get("prologue"), "traffic_source": TRAFFIC_SOURCE,
                              "ms": round(kern_ms["prologue"], 4)},
        # the T5 cross attention launch (q norm inside the kernel): ~13 key tiles per query tile, so Q / O streaming
        # and the per-workgroup ramp weigh as much as the MFMAs; priced against both roofs
        "roofline_cross": {"bound": "mfma", "kernel": "attn_fwd_bf16_x16_kernel (q_norm)", "achieved": round(cross_tflops, 2),
                           "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(cross_tflops / PEAK_BF16_TFLOPS, 4),
                           "hbm_gbs": round(cross_gbs, 1), "hbm_frac": round(cross_gbs / PEAK_HBM_GBS, 4),
                           "traffic": traffic.get("cross"), "traffic_source": TRAFFIC_SOURCE,
                           "ms": round(kern_ms["cross_attn"], 4), "ms_with_k_norm": round(kern_ms["cross"], 4)},
    }
    ref_rows = ref = None
    if not (args.no_fp8 and args.no_accuracy):
        # fp32 attention of 64 sampled rows per chunk on the tensors the kernels read (q as pre-scaled: scale ln 2)
        D_ = inp["D"]
        ref_rows, ref = fp32_rows_reference(inp["q"], inp["cache"][..., :D_], inp["cache"][..., D_:],
                                            inp["k_ranges_host"], inp["L"], 64, math.log(2.0))
        result["accuracy"] = {"what": "bf16 core attention output vs fp32 attention of 64 sampled query rows per chunk "
                                      "x all heads, full key ranges, same tensors", **deviation(inp["out"][ref_rows], ref)}
    if not args.no_fp8:
        result["fp8"] = fp8_leg(inp, core_fl, core_tflops, args.steps, ref_rows, ref)
    if not args.no_secondary:
        result["secondary"] = secondary_legs(inp, dev, max(3, args.steps // 4))
    if not args.no_ceiling:
        ceil = mfma_ceiling_leg(dev)
        result["mfma_ceiling"] = ceil
        try:
            top = ceil["bf16_16x16x32"]["random_operands"]["tflops"]  # (the MFMA shape the core kernel is made of)
            result["roofline"]["measured_ceiling"] = top
            result["roofline"]["frac_of_measured_ceiling"] = round(core_tflops / top, 4)
            if "fp8" in result:
                top8 = ceil["fp8_32x32x64"]["random_operands"]["tflops"]
                for m_ in ("pow2_prescaled", "pow2_prescaled_fast_exp2", "generic"):
                    result["fp8"][m_]["frac_of_measured_ceiling"] = round(result["fp8"][m_]["achieved"] / top8, 4)
                result["fp8"]["measured_ceiling"] = top8
        except (KeyError, TypeError):
            pass
    result["roofline_layer_norm"] = layer_norm_leg(inp, args.steps, traffic.get("layer_norm"))
    result["roofline_layer_norm"]["traffic_source"] = TRAFFIC_SOURCE
    if not args.no_ceiling:
        hc = hbm_ceiling_leg(inp, dev)
        result["hbm_ceiling"] = hc
        top = hc.get("copy", {}).get("gbs")
        if top:
            for key in ("roofline_prologue", "roofline_layer_norm"):
                result[key]["frac_of_measured_copy"] = round(result[key]["achieved"] / top, 4)
            prep = result.get("fp8", {}).get("operand_preparation")
            if prep and "achieved" in prep:
                prep["frac_of_measured_copy"] = round(prep["achieved"] / top, 4)
    if not args.no_projection:
        result["projection"] = projection_leg(inp, args.steps)
    if args.copy_calibration:
        inp["q"].copy_(inp["out"])  # reads and writes out.numel() * 2 bytes each
        torch.cuda.synchronize()
        result["copy_calibration_bytes_each_way"] = inp["out"].numel() * 2
    if not args.no_cpu_baseline:
        cb, o_cpu, idx = cpu_baseline(inp)
        got = inp["out"][idx.to(dev), : inp["Hq"] // inp["Hkv"]].float().cpu()
        cb["gpu_vs_cpu"] = deviation(got, o_cpu)
        result["cpu_baseline"] = cb
    print(json.dumps(result))


if __name__ == "__main__":
    main()
