"""The reference's fp8 linear layers in front of the prologue (inference/model/dit/dit_module.py:364-384 div_clamp_to,
:431-456 PerTensorQuantizedFp8Linear; q / qx / k / v of every layer but the first and the last under fp8_quant,
:405-409).

The input quantiser is integer-exact work: bit-identical to the oracle's restatement of div_clamp_to, bf16
intermediate included.  The GEMM behind it is the library's fp8 GEMM (fp32 accumulation of exact e4m3 products), so
the layer is compared with fp32 arithmetic on the de-quantised operands to one rounding of the bf16 result."""
import pytest
import torch

import magi_attn as M
from magi_attn import module as MOD
from oracle import magi_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols,per_column", [(1000, 6144, False), (333, 3072, True), (5, 8, False), (4099, 1536, True),
                                                  (1, 520, False)])
def test_div_clamp_to_bit_exact_with_oracle(dev, rows, cols, per_column):
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * 3.0).bfloat16()
    x[0, :8] = torch.tensor([0.0, -0.0, 1e-30, 1e30, -1e30, 447.0, 449.0, float("nan")]).bfloat16()
    scale = (torch.rand(cols if per_column else 1, generator=g) * 0.02 + 0.003)
    y = M.div_clamp_to(x.to(dev), scale.to(dev))
    ref = O.quantize_e4m3(x, scale, via_bf16=True)
    gb, rb = y.cpu().view(torch.uint8), ref.view(torch.uint8)
    nan = torch.isnan(x.float())
    assert torch.equal(gb[~nan], rb[~nan])
    assert torch.all((gb[nan] & 0x7f) == 0x7f)  # a NaN stays a NaN
    # saturation at +-448 and the double rounding: values that a direct conversion would round the other way exist
    direct = O.quantize_e4m3(x, scale, via_bf16=False).view(torch.uint8)
    assert y.float().abs()[~nan.to(dev)].max() <= 448
    if rows * cols > 100000:
        assert (direct[~nan] != rb[~nan]).any(), "the bf16 intermediate must matter somewhere in a sample this large"


def test_div_clamp_to_strided_rows_leading_axes_and_checks(dev):
    g = torch.Generator().manual_seed(3)
    wide = torch.randn(77, 2 * 512, generator=g).bfloat16()
    sc = torch.tensor([0.01])
    y = M.div_clamp_to(wide.to(dev)[:, 512:], sc.to(dev))
    assert torch.equal(y.cpu().view(torch.uint8), O.quantize_e4m3(wide[:, 512:], sc, via_bf16=True).view(torch.uint8))
    x3 = torch.randn(20, 3, 256, generator=g).bfloat16()
    y3 = M.div_clamp_to(x3.to(dev), sc.to(dev))
    assert y3.shape == x3.shape
    assert torch.equal(y3.cpu().view(torch.uint8), O.quantize_e4m3(x3, sc, via_bf16=True).view(torch.uint8))
    with pytest.raises(TypeError):
        M.div_clamp_to(x3.float().to(dev), sc.to(dev))
    with pytest.raises(ValueError):
        M.div_clamp_to(x3.to(dev), torch.ones(7, device=dev))
    with pytest.raises(M.MagiError):
        M.div_clamp_to(torch.zeros(4, 12, dtype=torch.bfloat16, device=dev), sc.to(dev))  # cols % 8


def test_per_tensor_fp8_linear_matches_dequantised_arithmetic(dev):
    torch.manual_seed(5)
    S, K, N = 640, 1024, 768
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16, device=dev)
    x = (torch.randn(S, 1, K, device=dev) * 1.3).bfloat16()
    q = MOD.PerTensorQuantizedFp8Linear.from_linear(lin, x.float().abs().max().item())
    assert q.weight.shape == (1, N, K) and q.weight.dtype == torch.float8_e4m3fn
    assert q.weight_scale.shape == (1,) and q.input_scale.shape == (K,)
    y = q(x)
    assert y.shape == (S, 1, N) and y.dtype == torch.bfloat16
    x8 = O.quantize_e4m3(x.cpu(), q.input_scale.cpu(), via_bf16=True).float().view(S, K)
    ref = (x8.double() @ q.weight[0].float().cpu().double().t()) * q.input_scale[0].item() * q.weight_scale.item()
    d = (y.view(S, N).double().cpu() - ref).abs()
    assert torch.all(d <= ref.abs() * 2.0 ** -7 + 1e-3)  # one bf16 rounding of an fp32-accumulated sum
    # and it approximates the bf16 layer it was made from to e4m3 precision
    full = torch.nn.functional.linear(x, lin.weight).float().view(S, N).cpu()
    cos = torch.nn.functional.cosine_similarity(y.view(S, N).float().cpu().flatten(), full.flatten(), dim=0).item()
    assert cos >= 0.998, cos


def test_layer_with_fp8_quant_projections(dev):
    """FullyParallelAttention(fp8_quant=True): q / qx / k / v through PerTensorQuantizedFp8Linear.  Against the same
    layer with bf16 projections made of the DE-QUANTISED weights, fed the same inputs: the only difference left is the
    e4m3 rounding of the normalised input (2.7 % per element, averaged over hidden-size products per output), so
    the attention outputs agree to cosine >= 0.999."""
    from magi_attn import params as P
    from magi_attn import ranges as R
    from magi_attn.rope import LearnableRotaryEmbeddingCat

    hidden, Hq, Hkv, D = 256, 8, 2, 128
    fr, H, W, dn = 2, 3, 4, 2
    L = fr * H * W
    S = dn * L
    torch.manual_seed(9)
    ref = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=1, device=dev)
    with torch.no_grad():
        for p in ref.parameters():
            p.copy_(torch.randn_like(p.float()) * (0.1 if p.dim() == 1 else hidden ** -0.5))
        ref.linear_qkv.layer_norm.weight.add_(1.0)
    q8 = MOD.FullyParallelAttention(hidden, Hq, Hkv, layer_number=1, device=dev, fp8_quant=True)
    sd = {k: v for k, v in ref.state_dict().items() if not k.startswith(("linear_qkv.q.", "linear_qkv.qx.", "linear_qkv.k.", "linear_qkv.v."))}
    q8.load_state_dict(sd, strict=False)
    for name in ("q", "qx", "k", "v"):
        lin = getattr(ref.linear_qkv, name)
        fq = MOD.PerTensorQuantizedFp8Linear.from_linear(lin, 6.0)  # normalised hidden states: |x| < 6
        setattr(q8.linear_qkv, name, fq)
        with torch.no_grad():  # the reference layer continues with the de-quantised weights
            lin.weight.copy_((fq.weight[0].float() * fq.weight_scale).to(lin.weight.dtype))
    g = torch.Generator().manual_seed(10)
    hs = torch.randn(S, 1, hidden, generator=g).bfloat16().to(dev)
    lens = torch.tensor([5, 8])
    mask = (torch.arange(8)[None] < lens[:, None]).float().view(dn, 1, 1, 8)
    y = (torch.randn(int(lens.sum()), hidden, generator=g) * 0.5).bfloat16().to(dev)
    kr = R.generate_kv_range_for_uncondition(dn, L)
    meta = P.ModelMetaArgs(H=H, W=W, cp_pad_size=None, cp_split_sizes=None, slice_point=0, denoising_range_num=dn,
                           range_num=dn, extract_prefix_video_feature=False, fwd_extra_1st_chunk=False,
                           distill_nearly_clean_chunk=False, clip_token_nums=L, enable_cuda_graph=False,
                           core_attn_params=P.build_core_attn_params(R.q_ranges_from_chunks(dn, L).to(dev), kr.to(dev), L),
                           cross_attn_params=P.build_cross_attn_params(mask.to(dev), L, 8))
    rope = LearnableRotaryEmbeddingCat(128, device=dev).get_embed_for_forward(dn * fr, H, W, 0, dn)
    with torch.no_grad():
        c0, x0 = ref(hs, y, None, rope, meta)
        c1, x1 = q8(hs, y, None, rope, meta)
    for a, b, nm in ((c1, c0, "core"), (x1, x0, "cross")):
        cos = torch.nn.functional.cosine_similarity(a.float().flatten(), b.float().flatten(), dim=0).item()
        assert torch.isfinite(a).all() and cos >= 0.999, (nm, cos)
