"""CPU tests of the host-side mirror of the reference's utils/quant.py API (no kernel launches)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr


@pytest.fixture(scope="module")
def Q(hip_lib):
    from latentq_llm_amd import quant
    return quant


REFERENCE_PUBLIC_NAMES = """python_compress python_decompress Qfunc_8bit_opt DeQfunc_8bit_opt GROUPSIZE Qfunc_4bit_g_res
DeQfunc_4bit_g Qfunc_8bit_res dict_temp QLinearFunctionW4 QLinearFunctionW4_eval QLinearFunctionA8W8_static
QLinearFunctionA8W8_dynamic0 QLinearFunctionA8W8_dynamic QLinearFunctionA8W8_static_eval QLinearFunctionA8W8_dynamic_eval
QLinearFunctionQAT_dynamic QLinearFunctionQAT_dynamic_eval backward_hook_fn QLinearA16W4 QLinearA8W8 QLinearQAT prodx
QuantTensor FPTensor three_fold_curve_4bit cuda_module EXT_type cuda_quant_linear cuda_quant_3fold cuda_dequant_linear
cuda_dequant_3fold python_quant_linear python_dequant_linear ResidualTensor GradientQTensor MyAdam""".split()


def test_every_public_name_of_the_reference_resolves(Q):
    missing = [n for n in REFERENCE_PUBLIC_NAMES if not hasattr(Q, n)]
    assert not missing, missing
    for n in ("quant", "dequant", "uniform_quant", "uniform_quant_s", "uniform_dequant"):
        assert hasattr(Q.cuda_module, n)


def test_compress_decompress_match_oracle(Q):
    allb = torch.arange(256, dtype=torch.uint8).view(torch.int8)
    codes = Q.python_decompress(allb)
    assert codes.dtype == torch.int8 and codes.shape == (256, 2)
    assert torch.equal(codes, tr.decompress(allb))
    assert np.array_equal(codes.numpy().reshape(-1).astype(np.uint8), co.unpack(allb.numpy()))
    back = Q.python_compress(codes)
    assert back.dtype == torch.int8 and torch.equal(back, allb)
    assert Q.python_compress(torch.tensor([15, 3, 8, 0, 7, 15])).tolist() == [-13, -128, 127]


def test_module_buffers_and_state_dict(Q):
    m = Q.QLinearA16W4(256, 48, bias=True, lbit=16, gbit=16)
    sd = m.state_dict()
    assert set(sd) == {"bias", "qweight", "zeros", "scales"}
    assert sd["zeros"].shape == (48 * 2, 1) and sd["scales"].dtype == torch.bfloat16
    assert m.weight.shape == [48, 256] and m.weight.wbit == 4 and m.wshape == [48, 256] and m.hook_handle is None
    assert "QLinearA16W4 input_features=256, output_features=48, bias=True" in repr(m)
    codes = torch.randint(-128, 128, (48 * 128,), dtype=torch.int8)
    m.weight.set_value(codes, [m.scales, m.zeros, m.wshape])
    assert m.weight.initial and m.weight.data is not codes and torch.equal(m.weight.data, codes)
    m.before_save()
    assert torch.equal(m.qweight, codes)
    assert m.to("cpu") is None and m.weight.qparam[0] is m.scales
    m.add_hook()
    assert m.hook_handle is not None

    a = Q.QLinearA8W8(128, 32, bias=False, lbit=16, gbit=8)
    assert set(a.state_dict()) == {"qweight", "clampv", "qscales"} and a.bias is None
    assert a.qscales.shape == (32, 1) and isinstance(a.weight.grad, Q.GradientQTensor)
    q = Q.QLinearQAT(128, 32, bias=True, lbit=16, gbit=16)
    assert isinstance(q.weight, Q.FPTensor) and q.weight.data.dtype == torch.bfloat16
    q.qscales.data.fill_(0.01)
    q.weight.data.copy_(torch.randn(32, 128))
    q.before_save()
    assert q.qweight.dtype == torch.int8 and q.qweight.shape == (32, 128)


def test_quant_tensor_latent_modes(Q):
    t16 = Q.QuantTensor([8, 128], wbit=4, gbit=16, lbit=16)
    assert t16.residual.dtype == torch.bfloat16 and t16.grad is None and t16.numel() == 1024
    t32 = Q.QuantTensor([8, 128], wbit=4, gbit=16, lbit=32)
    assert t32.residual.dtype == torch.float32
    t0 = Q.QuantTensor([8, 128], wbit=4, gbit=16, lbit=0)
    assert t0.residual is None
    assert t16.requires_grad_(False) is t16 and t16.requires_grad is False and t16.get_self() is t16
    assert hash(t16) != hash(t32)  # usable as optimizer-state keys


def test_8bit_optimizer_state_codec(Q):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4, 2048, generator=g)
    q, (scale, hi) = Q.Qfunc_8bit_opt(x.clone(), blocksize=4)
    assert q.dtype == torch.uint8 and q.shape == x.shape and scale.shape == (4, 1)
    back = Q.DeQfunc_8bit_opt(q, [scale, hi])
    assert (back - x).abs().max() <= scale.max() * 0.5 + 1e-6
    assert torch.equal(hi.view(-1), x.max(dim=1).values)


def test_cpu_uniform_residual_codec(Q):
    x = torch.rand(64, 8) - 0.5
    packed, carry = Q.python_quant_linear(x.clone())
    assert packed.dtype == torch.int32 and packed.shape == (64,)
    back = Q.python_dequant_linear(packed)
    err = (back + carry.view(-1, 8) - x).abs()  # a carry stands for one full step up
    assert float(err.max()) <= 1.0 / 16 + 1e-6


def test_three_fold_curve_table(Q):
    assert Q.three_fold_curve_4bit(0) == (2, 0.125, 4, 0.25)
    assert Q.three_fold_curve_4bit(2) == (2, 0.37272211741724515, 4, 0.4375)
    assert Q.three_fold_curve_4bit(7) == Q.three_fold_curve_4bit(0)


def test_myadam_accepts_latent_objects(Q):
    w = Q.QuantTensor([8, 128], wbit=4, gbit=16, lbit=16)
    b = torch.nn.Parameter(torch.zeros(8))
    opt = Q.MyAdam([{"params": [w], "weight_decay": 0.0}, {"params": [b], "weight_decay": 0.0}], lr=1e-3,
                   betas=(0.9, 0.95), obit=8, mu_updata_f=20, cpu=True)
    assert isinstance(opt, torch.optim.Adam) and opt.param_groups[0]["params"][0] is w
    with pytest.raises(ValueError):
        opt.add_param_group({"params": [w]})
    # a plain parameter steps like Adam (bf16 states for small tensors)
    b.grad = torch.ones(8)
    opt.step()
    assert torch.allclose(b.data, torch.full((8,), -1e-3), rtol=2e-2)
    assert b.grad is None and opt.state[b]["step"] == 1


def test_forward_requires_gpu(Q):
    from latentq_llm_amd._C import LatentQError
    m = Q.QLinearA16W4(128, 16, bias=False, lbit=16, gbit=16)
    m.weight.set_value(torch.zeros(16 * 64, dtype=torch.int8), [m.scales, m.zeros, m.wshape])
    with pytest.raises(LatentQError):
        m(torch.zeros(2, 128, dtype=torch.bfloat16))


def test_a8w8_default_lbit_keeps_a_latent_copy_like_the_reference():
    """main0.py:329-340 builds QLinearA8W8(..., lbit=args.lbit) and, for lbit != 4, writes the
    dequantised weight into weight.residual.data: an 8-bit weight always has a latent tensor (fp32
    for the default lbit = 0, utils/quant.py:606-627); only a 4-bit weight with lbit = 0 has none."""
    import torch
    from latentq_llm_amd import convert, quant as Q
    N, K = 16, 128
    layer = Q.QLinearA8W8(K, N, bias=True)  # constructor defaults: lbit = 0, gbit = 8
    assert isinstance(layer.weight.residual, torch.Tensor) and layer.weight.residual.dtype == torch.float32
    assert isinstance(layer.weight.grad, Q.GradientQTensor)
    g = torch.Generator().manual_seed(0)
    ckt = {"l.qweight": torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8),
           "l.scales": torch.rand(N, 1, generator=g) * 0.01 + 1e-3,
           "l.inp_absmax": torch.rand(K, generator=g) * 4,
           "l.bias": torch.randn(N, generator=g)}
    # the reference's own statements (main0.py:331-340), then the loader that wraps them
    ii = ckt["l.qweight"].to(torch.int32) - 128
    layer.qscales.data = ckt["l.scales"].to(torch.bfloat16)
    aa = (ii * layer.qscales).to(torch.bfloat16)
    layer.weight.set_value(ii.to(torch.int8), layer.qscales)
    layer.weight.residual.data = aa
    assert torch.equal(layer.weight.residual.data, aa)
    other = convert.load_a8w8(Q.QLinearA8W8(K, N, bias=True), ckt, "l")
    assert torch.equal(other.weight.residual.data.float(), aa.float())
    assert torch.equal(other.weight.data, ii.to(torch.int8))
    assert Q.QuantTensor([N, K], wbit=4, gbit=16, lbit=0).residual is None
