"""CPU tests of the host side: range generators and rope table of the product against the
oracle and the reference's worked examples, the metadata builders, and the C-ABI library
(loads, exports every declared symbol, rejects bad arguments before touching a GPU)."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

import magi_attn
from magi_attn import _lib as L
from magi_attn import params as P
from magi_attn import ranges as R
from magi_attn import rope as RP
from oracle import magi_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = magi_attn.lib()
    assert lib.magi_version() >= 100
    header = open(os.path.join(ROOT, "include", "magi_attn.h")).read()
    declared = set(re.findall(r"\b(magi_[a-z0-9_]+)\s*\(", header))
    assert declared == set(L.EXPORTS), declared ^ set(L.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name


def test_measurement_library_exports_what_its_header_declares():
    """libmagi_probe.so (MFMA-only and streaming loops that bench.py reports its ceilings from) is built by the same
    Makefile; nothing in the package loads it.  No compute call without a GPU: argument checks only."""
    path = os.path.join(ROOT, "magi-1_amd", "magi_attn", "libmagi_probe.so")
    assert os.path.exists(path), "build it with `make -C magi-1_amd/csrc`"
    lib = C.CDLL(path)
    header = open(os.path.join(ROOT, "magi-1_amd", "csrc", "probe", "magi_probe.h")).read()
    declared = re.findall(r"\b(magi_probe_\w+)\s*\(", header)
    assert sorted(set(declared)) == ["magi_probe_mfma_only", "magi_probe_stream"]
    for name in declared:
        assert hasattr(lib, name), name
    lib.magi_probe_stream.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    lib.magi_probe_stream.restype = C.c_int
    ms = C.c_float(0)
    assert lib.magi_probe_stream(7, None, None, 1024, 1, None, C.byref(ms)) == -22      # unknown kind
    assert lib.magi_probe_stream(0, None, None, 1024, 1, None, C.byref(ms)) == -22      # no buffers
    assert lib.magi_probe_stream(2, None, C.c_void_p(256), 1000, 1, None, C.byref(ms)) == -22  # not a multiple of 16
    for pkg_file in os.listdir(os.path.join(ROOT, "magi-1_amd", "magi_attn")):
        if pkg_file.endswith(".py"):
            assert "magi_probe" not in open(os.path.join(ROOT, "magi-1_amd", "magi_attn", pkg_file)).read(), pkg_file


def test_missing_library_is_an_error_not_a_fallback(tmp_path):
    """The library beside the package is the only compute path: when it is not there the first call raises (checked
    in a child process on a copy of the package without its .so; no environment variable redirects the loader)."""
    import shutil
    import subprocess
    import sys

    pkg = tmp_path / "magi_attn"
    shutil.copytree(os.path.join(ROOT, "magi-1_amd", "magi_attn"), pkg,
                    ignore=shutil.ignore_patterns("*.so", "__pycache__"))
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "import magi_attn._lib as L\n"
        "assert L.LIB_PATH.startswith(%r), L.LIB_PATH\n"
        "try:\n"
        "    L.lib()\n"
        "except RuntimeError as e:\n"
        "    assert 'no fallback' in str(e), e; print('raised')\n"
    ) % (str(tmp_path), str(pkg))
    env = dict(os.environ, MAGI_ATTN_LIBRARY=os.path.join(ROOT, "magi-1_amd", "magi_attn", "libmagi_attn.so"))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert r.returncode == 0 and r.stdout.strip() == "raised", (r.stdout, r.stderr[-2000:])


def test_struct_layouts_match_header(tmp_path):
    """ctypes mirrors vs the C compiler's view of include/magi_attn.h (sizes and field offsets)."""
    import subprocess

    pairs = (("magi_attn_args", L.AttnArgs), ("magi_prologue_args", L.PrologueArgs),
             ("magi_qkv_proj_args", L.QkvProjArgs), ("magi_quantize_args", L.QuantizeArgs))
    src = ['#include <stdio.h>', '#include <stddef.h>', '#include "magi_attn.h"', 'int main(void){']
    for cname, mirror in pairs:
        src += ['printf("%%zu\\n", sizeof(%s));' % cname]
        src += ['printf("%%zu\\n", offsetof(%s, %s));' % (cname, f[0]) for f in mirror._fields_]
    src += ['return 0;}']
    c = tmp_path / "layout.c"
    c.write_text("\n".join(src))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(c), "-o", str(exe)], check=True)
    out = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    pos = 0
    for cname, mirror in pairs:
        names = [f[0] for f in mirror._fields_]
        assert names[0] == "struct_size" and getattr(mirror, "struct_size").offset == 0
        assert out[pos] == C.sizeof(mirror), cname
        assert out[pos + 1:pos + 1 + len(names)] == [getattr(mirror, f).offset for f in names], cname
        assert mirror().struct_size == C.sizeof(mirror)  # filled in by the mirror's constructor
        pos += 1 + len(names)
    assert pos == len(out)


def test_a_struct_of_another_size_is_refused():
    """Every argument struct starts with its size as the caller compiled it; a caller built against another
    version of the header (a shorter or longer struct) gets MAGI_EINVAL instead of having fields read that it
    never wrote.  The Python mirrors are bound to one library version and refuse to load another."""
    lib = magi_attn.lib()
    assert lib.magi_version() == L.ABI_VERSION
    for mk, fn in ((L.AttnArgs, lib.magi_attn_fwd), (L.PrologueArgs, lib.magi_qk_prologue),
                   (L.QkvProjArgs, lib.magi_qkv_proj_prologue), (L.QuantizeArgs, lib.magi_quantize_fp8_split)):
        a = mk()
        for wrong in (0, a.struct_size - 8, a.struct_size + 8):
            a.struct_size = wrong
            assert fn(C.byref(a), None) == -22 and b"struct_size" in lib.magi_last_error(), mk.__name__
    assert isinstance(lib.magi_launch_count(), int)


def test_attn_argument_validation_without_gpu():
    lib = magi_attn.lib()
    a = L.AttnArgs()
    a.D, a.Hq, a.Hkv = 64, 4, 2
    assert lib.magi_attn_fwd(C.byref(a), None) == -38  # head_dim not implemented
    assert b"head_dim" in lib.magi_last_error()
    a.D, a.Hq, a.Hkv = 128, 5, 2
    assert lib.magi_attn_fwd(C.byref(a), None) == -22
    a.Hq = 4
    a.dtype = 7
    assert lib.magi_attn_fwd(C.byref(a), None) == -22
    a.dtype = 0
    a.n_ranges = 0
    assert lib.magi_attn_fwd(C.byref(a), None) == 0  # nothing to do
    a.n_ranges, a.total_q, a.max_seqlen_q = 1, 8, 8
    assert lib.magi_attn_fwd(C.byref(a), None) == -22  # NULL q
    assert b"NULL" in lib.magi_last_error()
    a.q = a.out = a.q_ranges = a.k_ranges = 4096
    a.q_stride_t = a.o_stride_t = 512
    a.q_stride_h = a.o_stride_h = 128
    a.k_stride_t, a.k_stride_h, a.v_stride_t, a.v_stride_h = 256, 128, 256, 100
    assert lib.magi_attn_fwd(C.byref(a), None) == -22  # misaligned stride
    a.v_stride_h = 128
    a.k = a.v = 4096
    a.total_k = 8
    a.out_group_heads = 3  # does not divide Hq = 4
    assert lib.magi_attn_fwd(C.byref(a), None) == -22 and b"out_group_heads" in lib.magi_last_error()
    assert lib.magi_attn_fwd(None, None) == -22


def test_prologue_argument_validation_without_gpu():
    lib = magi_attn.lib()
    p = L.PrologueArgs()
    p.D = 64
    assert lib.magi_qk_prologue(C.byref(p), None) == -38
    p.D, p.S = 128, 0
    assert lib.magi_qk_prologue(C.byref(p), None) == 0
    p.S, p.Hq, p.Hkv, p.R2 = 4, 2, 1, 44
    assert lib.magi_qk_prologue(C.byref(p), None) == -22 and b"R2" in lib.magi_last_error()
    p.R2 = 48
    assert lib.magi_qk_prologue(C.byref(p), None) == -22  # NULL buffers
    assert lib.magi_head_norm(None, 0, 0, None, None, None, 4, 2, 128, 0, 1e-6, None) == -22
    # layer norm: validation happens before any device work
    buf = (C.c_char * 64)()
    p16 = (C.addressof(buf) + 15) & ~15
    assert lib.magi_layer_norm(None, 64, None, None, 0, None, 64, 0, 64, 1e-5, None) == 0  # no rows: nothing to do
    assert lib.magi_layer_norm(None, 64, None, None, 0, None, 64, 4, 64, 1e-5, None) == -22
    assert lib.magi_layer_norm(p16, 64, None, None, 0, p16, 64, 4, 60, 1e-5, None) == -38  # cols % 8
    assert lib.magi_layer_norm(p16, 64, None, None, 0, p16, 64, 4, 8200, 1e-5, None) == -38
    assert lib.magi_layer_norm(p16, 32, None, None, 0, p16, 64, 4, 64, 1e-5, None) == -22  # stride < cols
    assert lib.magi_layer_norm(p16 + 2, 64, None, None, 0, p16, 64, 4, 64, 1e-5, None) == -22  # alignment
    assert b"magi_layer_norm" in lib.magi_last_error()
    assert lib.magi_apply_rotary(None, None, None, None, 1, 4, 2, 128, 80, 0, None) == -22


def test_generate_sequences_reference_examples_and_oracle():
    assert R.generate_sequences(8, 4, 2) == ([2, 2, 2, 2, 3, 4, 5, 6, 7], [3, 4, 5, 6, 7, 8, 8, 8, 8],
                                             [0, 0, 0, 0, 0, 0, 1, 2, 3], [1, 2, 3, 4, 4, 4, 4, 4, 4])
    for args in [(8, 8, 0), (8, 4, 0), (8, 1, 0), (12, 4, 3), (5, 7, 1), (1, 1, 0)]:
        assert R.generate_sequences(*args) == O.generate_sequences(*args)


def test_kvrange_generators_match_oracle():
    L_ = 9360
    for sp, dn in [(0, 1), (0, 4), (4, 4), (8, 4), (3, 2)]:
        assert np.array_equal(R.generate_default_kvrange(sp, dn, L_).numpy(), O.default_kvrange(sp, dn, L_))
        steps = [32, 17, 8, 0][:dn]
        a = R.generate_noise2clean_kvrange(sp, dn, L_, [5, 4, 3, 2], 1, steps, 32).numpy()
        assert np.array_equal(a, O.noise2clean_kvrange(sp, dn, L_, [5, 4, 3, 2], 1, steps, 32))
        assert a.dtype == np.int32
        b = R.generate_kvrange_for_denoising_video(sp, dn, L_, [], -1, steps, 32).numpy()
        assert np.array_equal(b, O.default_kvrange(sp, dn, L_))
    assert np.array_equal(R.generate_kvrange_for_prefix_video(5, L_, 1).numpy(), O.prefix_video_kvrange(5, L_, 1))
    assert np.array_equal(R.generate_kvrange_for_prefix_video(5, L_, -1, [5, 4, 3, 2]).numpy(),
                          O.prefix_video_kvrange(5, L_, -1, [5, 4, 3, 2]))
    assert np.array_equal(R.generate_kv_range_for_uncondition(4, L_).numpy(), O.uncondition_kvrange(4, L_))
    assert np.array_equal(R.q_ranges_from_chunks(4, L_).numpy(), O.q_ranges_for(4, L_))
    # batch > 1 offsets every row by b * range_num chunks (video_generate.py:461-463)
    two = R.generate_default_kvrange(1, 2, 10, batch_size=2).tolist()
    assert two == [[0, 20], [0, 30], [30, 50], [30, 60]]
    with pytest.raises(ValueError):
        R.generate_noise2clean_kvrange(0, 2, 10, [5, 4, 3], 1, [0, 0], 32)


def test_rope_module_matches_oracle():
    m = RP.LearnableRotaryEmbeddingCat(128)
    assert torch.equal(m.bands.detach(), O.freq_bands(16))
    for T, H, W, sp, dn in [(6, 4, 6, 2, 3), (2, 16, 16, 0, 1), (4, 8, 13, 5, 2)]:
        a = m.get_embed_for_forward(T, H, W, sp, dn)
        b = O.rope_for_forward(T, H, W, sp, dn)
        assert a.shape == (T * H * W, 96) and torch.equal(a, b)
    assert torch.equal(m.get_embed([3, 4, 6]), O.rope_table(3, 4, 6))
    # the reference's two builder functions by name: (sin, cos) halves of the same table, and their per-axis form
    sin, cos = RP.build_rotary_pos_embed([3, 4, 6], bands=m.bands.detach(), dim=128)
    assert sin.shape == cos.shape == (72, 48) and torch.equal(torch.cat([sin, cos], -1), O.rope_table(3, 4, 6))
    f_sin, f_cos = RP.build_fourier_pos_embed([3, 4, 6], num_bands=16)
    assert f_sin.shape == (3, 4, 6, 3, 16) and torch.equal(f_sin.reshape(72, 48), sin) and torch.equal(f_cos.reshape(72, 48), cos)
    assert torch.equal(f_sin[2, 1, 5, 0], torch.sin(2.0 * RP.freq_bands(16)))            # axis 0 is time: position 2
    with pytest.raises(NotImplementedError):
        RP.build_rotary_pos_embed([3, 4, 6], in_pixels=True)
    assert RP.LearnableRotaryEmbeddingCat(128, in_pixels=False).bands.shape == (16,)


def test_param_builders():
    qr = torch.tensor([[0, 10], [10, 20]], dtype=torch.int32)
    kr = torch.tensor([[20, 50], [10, 60]], dtype=torch.int32)
    p = P.build_core_attn_params(qr, kr, 10)
    assert p.max_seqlen_k == 50 and p.max_seqlen_q == 10 and p.np_k_range.tolist() == kr.tolist()
    mask = torch.zeros(3, 1, 1, 16)
    mask[0, ..., :7] = 1
    mask[2, ..., :3] = 1
    x = P.build_cross_attn_params(mask, 10, 800)
    cq, ck, qr2, kr2 = O.cross_attn_params_from_mask(mask.reshape(3, 16), 10)
    assert torch.equal(x.cu_seqlens_q, cq) and torch.equal(x.cu_seqlens_kv, ck)
    assert torch.equal(x.q_ranges, qr2) and torch.equal(x.kv_ranges, kr2)
    assert x.cu_seqlens_q.dtype == torch.int32 and x.max_seqlen_kv == 800
    ip = P.InferenceParams(1, 100)
    assert ip.key_value_memory_dict == {} and ip.update_kv_cache is False


def test_functional_rejects_cpu_tensors():
    q = torch.zeros(4, 2, 128, dtype=torch.bfloat16)
    r = torch.zeros(1, 2, dtype=torch.int32)
    with pytest.raises(ValueError):
        magi_attn.range_attention(q, q, q, r, r, 4)


def test_kv_cache_arena_views_accounting_and_errors():
    from magi_attn.cache import KVCacheArena
    # the 24B 720p figure of the design notes: 48 layers x 259200 tokens x 8 heads x 256 x 2 B = 51 GB
    assert KVCacheArena.bytes_needed(48, 259200, 8) == 48 * 259200 * 8 * 256 * 2
    arena = KVCacheArena(3, 40, 2, device="cpu")
    ip = P.InferenceParams(1, 40)
    d = arena.attach(ip, layer_numbers=[5, 6, 7])
    assert sorted(d) == [5, 6, 7] and d[6].shape == (40, 2, 256)
    d[6][3, 1, 200] = 2.5  # a view: writes land in the arena, layers do not overlap
    assert arena.layer(1)[3, 1, 200] == 2.5 and arena.buffer.data_ptr() == d[5].data_ptr()
    assert d[7].data_ptr() - d[6].data_ptr() == 40 * 2 * 256 * 2
    with pytest.raises(ValueError):
        arena.attach(P.InferenceParams(1, 41))
    with pytest.raises(ValueError):
        arena.attach(ip, layer_numbers=[1, 1, 2])
    with pytest.raises(MemoryError):
        KVCacheArena(48, 259200, 8, device="cpu", memory_budget_bytes=1 << 30)
    with pytest.raises(ValueError):
        KVCacheArena(1, 8, 1, device="cpu", kv_offload=True)   # the staging buffers need a GPU
    with pytest.raises(ValueError):
        KVCacheArena(1, 8, 1, device="cuda", kv_offload=True, max_batch_size=2)
    with pytest.raises(MemoryError):                              # with kv_offload the budget counts the staging ring
        KVCacheArena(48, 259200, 8, device="cuda", kv_offload=True, memory_budget_bytes=1 << 30)


def test_projection_weights_share_one_buffer():
    """q / k / v / qx keep the reference's parameter names but are rows of one buffer, so one GEMM serves all four;
    the sharing survives load_state_dict and is re-established after a dtype / device move."""
    from magi_attn.module import CustomLayerNormLinear

    torch.manual_seed(0)
    m = CustomLayerNormLinear(64, 48, 16, dtype=torch.float32)
    assert sorted(n for n, _ in m.named_parameters()) == ["k.weight", "layer_norm.bias", "layer_norm.weight", "q.weight",
                                                          "qx.weight", "v.weight"]
    w = m.fused_weight()
    assert w.shape == (128, 64) and w.data_ptr() == m.q.weight.data_ptr()
    x = torch.randn(5, 1, 64)
    q, k, v, qx = m.forward_qkvx(x)
    for got, lin in ((q, m.forward_q), (k, m.forward_k), (v, m.forward_v), (qx, m.forward_qx)):
        assert torch.allclose(got, lin(x), atol=1e-6)
    sd = {n: torch.randn_like(t) for n, t in m.state_dict().items()}
    m.load_state_dict(sd)
    w2 = m.fused_weight()
    assert w2.data_ptr() == w.data_ptr()  # copied in place, still shared
    assert torch.equal(w2, torch.cat([sd["q.weight"], sd["k.weight"], sd["v.weight"], sd["qx.weight"]]))
    m = m.to(torch.bfloat16)  # re-allocates every parameter: the buffer is rebuilt on the next call
    w3 = m.fused_weight()
    assert w3.dtype == torch.bfloat16 and w3.data_ptr() == m.q.weight.data_ptr()
    assert m.k.weight.data_ptr() == w3.data_ptr() + 48 * 64 * 2
    assert torch.equal(w3[80:], sd["qx.weight"].bfloat16())


def test_fp8_kv_cache_shapes_and_layer_option():
    from magi_attn.cache import Fp8KVCache
    from magi_attn.module import FullyParallelAttention

    c = Fp8KVCache(10 * 24, 2, 24)
    assert c.k.shape == c.v.shape == (240, 2, 128) and c.k.dtype == torch.float8_e4m3fn
    assert c.k_scale.shape == c.v_scale.shape == (10, 2) and c.max_sequence_length == 240
    assert Fp8KVCache(25, 1, 24).k_scale.shape == (2, 1)  # a partial last chunk has a scale row too
    with pytest.raises(ValueError):
        Fp8KVCache(0, 2, 24)
    with pytest.raises(ValueError):
        FullyParallelAttention(64, 2, 1, attention_dtype="fp4")
    assert FullyParallelAttention(64, 2, 1, attention_dtype="fp8").attention_dtype == "fp8"


def test_attention_kernels_keep_their_registers():
    """A register spill inside a tile loop costs a drain of the tile loads per tile (parity stays green while the
    launch runs 1.7x slower), and the allocator decides per instantiation: compile the attention sources for
    gfx950 and check the compiler's own resource report.  The bf16 instantiations must use no scratch memory at
    all; the fp8 kernel is allowed its known 24 bytes (values parked across the loop and reloaded on the ragged-tile
    path and in the epilogue, not in the steady-state loop)."""
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    csrc = os.path.join(ROOT, "magi-1_amd", "csrc")
    flags = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + csrc,
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage", "-c", "-o", os.devnull]
    # The bf16 kernels must not spill at all (the 16x16x32 kernel once parked two accumulators around its first tile:
    # outside the steady-state loop, but a round trip to scratch memory for every workgroup, 12 % more bytes written).
    for src, limit in (("attn_fwd_bf16.hip", 0), ("attn_fwd_fp8.hip", 24), ("attn_fwd_bf16_w64.hip", 0),
                       ("attn_fwd_bf16_x16.hip", 0)):
        r = subprocess.run([hipcc] + flags + [os.path.join(csrc, src)], capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-2000:]
        names = re.findall(r"Function Name: (\S+)", r.stderr)
        scratch = [int(x) for x in re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", r.stderr)]
        vgprs = [int(x) for x in re.findall(r" VGPRs: (\d+)", r.stderr)]
        assert names and len(names) == len(scratch) == len(vgprs), (len(names), len(scratch), len(vgprs))
        seen = 0
        for n, sc, vg in zip(names, scratch, vgprs):
            if "attn_fwd" in n:
                seen += 1
                assert sc <= limit, f"{n}: {sc} bytes of scratch per lane"
                assert vg <= 256
        assert seen >= 2


def test_inference_params_swap_key_value_dict():
    """Batch rows of the (position, batch)-ordered caches are re-ordered in every layer; an empty dict raises, as in
    the reference (inference/common/dataclass.py:72-83)."""
    from magi_attn.params import InferenceParams

    ip = InferenceParams(3, 4)
    with pytest.raises(ValueError):
        ip.swap_key_value_dict([0, 1, 2])
    c = torch.arange(4 * 3 * 2 * 8, dtype=torch.float32).view(12, 2, 8)  # [max_seq * max_bs, Hkv, 2D]
    ip.key_value_memory_dict[0] = c.clone()
    ip.key_value_memory_dict[5] = c.clone() + 1000
    ip.swap_key_value_dict([2, 0, 1])
    want = c.view(4, 3, 2, 8)[:, [2, 0, 1]].reshape(12, 2, 8)
    assert torch.equal(ip.key_value_memory_dict[0], want) and torch.equal(ip.key_value_memory_dict[5], want + 1000)
    with pytest.raises(ValueError):
        ip.swap_key_value_dict([0, 1])


def test_copying_form_of_the_cache_update_matches_the_reference_semantics():
    """FullyParallelAttention.adjust_key_and_value_for_inference, the method with the reference's signature for
    callers that hold a materialised key_and_value (dit_module.py:891-946): pure tensor work, so it runs on the CPU.
    Against the oracle's list-of-rows model through a schedule with appends, reads without update, the distill form
    that drops the last chunk, no inference_params at all, and batch 2."""
    from magi_attn.module import FullyParallelAttention
    from oracle import magi_oracle as O
    Hkv, D, L_ = 2, 128, 5
    for bs in (1, 2):
        layer = FullyParallelAttention(64, 4, Hkv, layer_number=2, device="cpu")
        ip = P.InferenceParams(bs, 6 * L_)
        model = O.KVCacheModel(6 * L_, Hkv, D, max_batch_size=bs)
        g = torch.Generator().manual_seed(bs)
        written = 0
        # (slice_point, chunks, update, distill, fwd_extra_1st_chunk)
        for sp, dn, update, distill, extra in ((0, 2, True, False, True), (2, 2, False, False, False),
                                               (2, 2, True, True, False), (3, 3, True, False, False),
                                               (0, 1, True, False, False)):
            kv = torch.randn(dn * L_ * bs, Hkv, 2 * D, generator=g).bfloat16()
            ip.update_kv_cache = update
            meta = P.ModelMetaArgs(H=1, W=L_, cp_pad_size=None, cp_split_sizes=None, slice_point=sp, denoising_range_num=dn,
                                   range_num=sp + dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=extra,
                                   distill_nearly_clean_chunk=distill, clip_token_nums=L_, enable_cuda_graph=False,
                                   core_attn_params=None, cross_attn_params=None)
            k, v = layer.adjust_key_and_value_for_inference(kv, ip, meta)
            k_ref, v_ref = model.adjust(kv, has_inference_params=True, update_kv_cache=update, slice_point=sp,
                                        clip_token_nums=L_, fwd_extra_1st_chunk=extra, distill_nearly_clean_chunk=distill)
            assert torch.equal(k, k_ref) and torch.equal(v, v_ref), (bs, sp, dn)
            if update:
                written = max(written, (sp + dn - (1 if distill else 0)) * L_ * bs)
            # (the layer's cache is allocated uninitialised, as the reference's: rows written so far)
            assert torch.equal(ip.key_value_memory_dict[2][:written], model.mem[:written])
        k, v = layer.adjust_key_and_value_for_inference(kv, None, meta)
        assert torch.equal(k, kv[..., :D]) and torch.equal(v, kv[..., D:])
