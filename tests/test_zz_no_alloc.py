"""magi_attn_fwd_static_scratch: the entry point for callers that can neither pass a workspace nor allocate one.  Its
scratch memory (the measured score bound of MAGI_ATTN_AUTO_BOUND) is an array in the library's device image.  Through
the C-ABI, against magi_attn_fwd with a caller-provided workspace: bit-identical outputs, on two calls in a row of
which the second is smaller (the array keeps the first call's contents; the call has to clear what it needs), for
inputs on either side of the bound."""
import numpy as np
import pytest
import torch

import magi_attn as M
from magi_attn import _lib as L
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu


def _call(entry, dev, q, k, v, qr, kr, max_q, workspace):
    """One call through ctypes with every buffer made here, outside the library."""
    out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((q.shape[1], q.shape[0]), float("nan"), dtype=torch.float32, device=dev)
    tq = torch.tensor(np.asarray(qr), dtype=torch.int32, device=dev)
    tk = torch.tensor(np.asarray(kr), dtype=torch.int32, device=dev)
    a = L.AttnArgs()
    a.q, a.k, a.v, a.out, a.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
    a.q_ranges, a.k_ranges = tq.data_ptr(), tk.data_ptr()
    a.q_stride_t, a.q_stride_h = q.stride(0), q.stride(1)
    a.k_stride_t, a.k_stride_h = k.stride(0), k.stride(1)
    a.v_stride_t, a.v_stride_h = v.stride(0), v.stride(1)
    a.o_stride_t, a.o_stride_h = out.stride(0), out.stride(1)
    a.total_q, a.total_k, a.k_split = q.shape[0], k.shape[0], k.shape[0]
    a.n_ranges, a.ranges_mode, a.max_seqlen_q = len(qr), L.MAGI_RANGES_PAIRS, max_q
    a.Hq, a.Hkv, a.D, a.dtype = q.shape[1], k.shape[1], 128, L.MAGI_DTYPE_BF16
    a.flags = L.MAGI_ATTN_AUTO_BOUND
    a.workspace = None if workspace is None else workspace.data_ptr()
    L.check(entry(a, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return out, lse


def test_static_scratch_entry_matches_the_workspace_entry(dev):
    lib = L.lib()
    cases = []
    # first a large-gain input (bound above the limit: online softmax), then a smaller normed one (bounded kernel),
    # then the large one again: the array must not remember
    for L_, dn, sp, Hq, Hkv, gain, seed in ((333, 4, 2, 12, 4, 3.0, 1), (77, 2, 1, 6, 2, 1.0, 2), (200, 3, 1, 6, 2, 2.5, 3),
                                            (64, 1, 0, 2, 1, 1.0, 4)):
        q, k, v = O.synthetic_qkv(dn * L_, (sp + dn) * L_, Hq, Hkv, 128, seed=seed)
        q, k = (q.float() * gain).bfloat16(), (k.float() * gain).bfloat16()
        cases.append((q.to(dev), k.to(dev), v.to(dev), O.q_ranges_for(dn, L_), O.default_kvrange(sp, dn, L_), L_, (q, k, v)))
    ws = torch.empty(4, dtype=torch.float32, device=dev)
    want = [_call(lib.magi_attn_fwd, dev, q, k, v, qr, kr, mq, ws) for q, k, v, qr, kr, mq, _ in cases]
    got = []
    for q, k, v, qr, kr, mq, _ in cases:  # back to back, nothing else in between
        got.append(_call(lib.magi_attn_fwd_static_scratch, dev, q, k, v, qr, kr, mq, None))
    for (o0, l0), (o1, l1), case in zip(want, got, cases):
        assert not torch.isnan(o1).any() and torch.equal(o0, o1) and torch.equal(l0, l1)
        ref = O.range_attention(*case[6], case[3], case[4])
        assert (o1.float().cpu() - ref).abs().max().item() <= 2e-2
    # without the flag the entry point is magi_attn_fwd
    q, k, v, qr, kr, mq, _ = cases[1]
    plain = M.range_attention(q, k, v, torch.tensor(qr, dtype=torch.int32, device=dev),
                              torch.tensor(kr, dtype=torch.int32, device=dev), mq)[0]
    via = M.range_attention(q, k, v, torch.tensor(qr, dtype=torch.int32, device=dev),
                            torch.tensor(kr, dtype=torch.int32, device=dev), mq, static_scratch=True)[0]
    assert torch.equal(plain, via)


def test_static_scratch_entry_under_graph_capture(dev):
    """What the entry point is for: a call that measures its bound, captured into a HIP graph with no allocation in the
    captured region (out given, no lse).  Replays on inputs that alternate between the two sides of the bound, with
    eager calls in between, equal the eager results bit for bit."""
    L_, dn, sp, Hq, Hkv = 160, 2, 1, 6, 2
    q, k, v = [t.to(dev) for t in O.synthetic_qkv(dn * L_, (sp + dn) * L_, Hq, Hkv, 128, seed=31)]
    tq = torch.tensor(O.q_ranges_for(dn, L_), dtype=torch.int32, device=dev)
    tk = torch.tensor(O.default_kvrange(sp, dn, L_), dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    call = lambda dst: M.range_attention(q, k, v, tq, tk, L_, out=dst, return_lse=False, auto_bound=True, static_scratch=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(out)
    base_q, base_k = q.clone(), k.clone()
    for rep, gain in enumerate((1.0, 3.0, 1.0, 2.5)):
        q.copy_((base_q.float() * gain).bfloat16())
        k.copy_((base_k.float() * gain).bfloat16())
        eager = torch.empty_like(out)
        M.range_attention(q, k, v, tq, tk, L_, out=eager, return_lse=False, **({"score_bound": 17.0} if gain == 1.0 else {}))
        torch.cuda.synchronize()
        out.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} (gain {gain})"
