"""The measurement-only library that bench.py reports its ceilings from does what its header says: the streaming
kernels move the bytes they are credited with, the MFMA-only loops report the FLOPs of the instruction they issue.
(Not part of the attention path: nothing in the package loads this library.)"""
import ctypes as C
import os

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def probe():
    path = os.path.join(ROOT, "magi-1_amd", "magi_attn", "libmagi_probe.so")
    assert os.path.exists(path), "build it with `make -C magi-1_amd/csrc`"
    lib = C.CDLL(path)
    lib.magi_probe_stream.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.POINTER(C.c_float)]
    lib.magi_probe_stream.restype = C.c_int
    lib.magi_probe_mfma_only.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                         C.POINTER(C.c_float), C.POINTER(C.c_double)]
    lib.magi_probe_mfma_only.restype = C.c_int
    return lib


@pytest.mark.parametrize("nbytes", [16, 4096 * 3 + 16, 1 << 24, (1 << 24) + 48])
def test_stream_kernels_move_what_they_are_credited_with(dev, probe, nbytes):
    g = torch.Generator(device=dev).manual_seed(5)
    src = torch.randint(0, 256, (nbytes + 64,), dtype=torch.uint8, device=dev, generator=g)
    dst = torch.full((nbytes + 64,), 7, dtype=torch.uint8, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ms = C.c_float(0)
    # copy: exactly nbytes arrive, nothing behind them is touched
    assert probe.magi_probe_stream(0, src.data_ptr(), dst.data_ptr(), nbytes, 2, stream, C.byref(ms)) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst[:nbytes], src[:nbytes]) and bool((dst[nbytes:] == 7).all()) and ms.value > 0
    # read-only: the destination keeps its bytes
    keep = dst.clone()
    assert probe.magi_probe_stream(1, src.data_ptr(), dst.data_ptr(), nbytes, 2, stream, C.byref(ms)) == 0
    torch.cuda.synchronize()
    assert torch.equal(dst, keep)
    # write-only: every 16-byte piece is written (its index in the first word, then 1, 2, 3), nothing behind
    assert probe.magi_probe_stream(2, None, dst.data_ptr(), nbytes, 2, stream, C.byref(ms)) == 0
    torch.cuda.synchronize()
    words = dst[:nbytes].view(torch.int32).view(-1, 4)
    assert torch.equal(words[:, 0].cpu(), torch.arange(nbytes // 16, dtype=torch.int32))
    assert bool((words[:, 1] == 1).all()) and bool((words[:, 2] == 2).all()) and bool((words[:, 3] == 3).all())
    assert bool((dst[nbytes:] == 7).all())


@pytest.mark.parametrize("kind,flop_per_round", [(0, 64 * 2 * 32 * 32 * 16), (1, 128 * 2 * 16 * 16 * 32),
                                                 (2, 32 * 2 * 32 * 32 * 64), (3, 64 * 2 * 16 * 16 * 128)])
def test_mfma_loops_report_the_flops_of_their_instruction(dev, probe, kind, flop_per_round):
    """FLOPs per launch = rounds x MFMAs per round x 2 M N K x one wave per SIMD on 256 CUs; the rate that follows from
    a short launch lies between a tenth of the nominal figure and the nominal figure (2.5 PFLOP/s bf16, 5 fp8)."""
    sink = torch.empty(256 * 256, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    ms, fl = C.c_float(0), C.c_double(0)
    rounds = 2000
    assert probe.magi_probe_mfma_only(kind, None, sink.data_ptr(), rounds, 3, stream, C.byref(ms), C.byref(fl)) == 0
    assert fl.value == float(flop_per_round) * rounds * 256 * 4
    rate = fl.value / (ms.value * 1e-3)
    nominal = 5.0e15 if kind >= 2 else 2.5e15
    assert 0.1 * nominal < rate <= 1.02 * nominal, rate
