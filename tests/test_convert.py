"""Checkpoint-format converters (latentq_llm_amd/convert.py) against brute-force restatements of
the GPTQ bit layout (PTQ/quant/quant_linear.py:325-389) and of the loader in main0.py:316-342."""
import numpy as np
import pytest
import torch

from tests.util import bits, make_w4


def gptq_pack_bruteforce(codes_nk, zeros_ng, scales_ng):
    """The loops of QuantLinearGPTQ.pack, written out: qweight[k/8, n] |= code << 4*(k%8);
    qzeros[g, n/8] |= (zero - 1) << 4*(n%8); scales stored [G, N]."""
    N, K = codes_nk.shape
    G = K // 128
    qweight = np.zeros((K // 8, N), np.uint32)
    for k in range(K):
        qweight[k // 8] |= codes_nk[:, k].astype(np.uint32) << np.uint32(4 * (k % 8))
    qzeros = np.zeros((G, N // 8), np.uint32)
    zt = zeros_ng.T.astype(np.int64) - 1
    for n in range(N):
        qzeros[:, n // 8] |= (zt[:, n] & 0xF).astype(np.uint32) << np.uint32(4 * (n % 8))
    return qweight.astype(np.int32), qzeros.astype(np.int32), scales_ng.T.copy()


def test_zero_point_pack_unpack_bruteforce():
    from latentq_llm_amd import convert
    rng = np.random.default_rng(0)
    G, N = 5, 48
    z = rng.integers(1, 17, (N, G))
    _, qzeros, _ = gptq_pack_bruteforce(np.zeros((N, G * 128), np.uint8), z, np.ones((N, G), np.float16))
    got = convert.unpack_gptq_zeros(torch.from_numpy(qzeros), N)
    assert np.array_equal(got.numpy(), z.T)
    assert np.array_equal(convert.pack_gptq_zeros(torch.from_numpy(z.T.copy())).numpy(), qzeros)
    assert int(convert.a8w8_weight_from_checkpoint(torch.tensor([0, 128, 255], dtype=torch.uint8))[0]) == -128
    with pytest.raises(ValueError):
        convert._check_g_idx(torch.arange(256) // 64, 256, 128)


@pytest.mark.gpu
@pytest.mark.parametrize("N,K", [(16, 128), (72, 384), (256, 1024)])
def test_gptq_round_trip_and_dequant(hip_lib, N, K):
    from latentq_llm_amd import convert, ops
    from oracle import c_oracle as co
    codes, packed, scales, zeros = make_w4(N, K, N + K)       # native layout, zeros in 6..9
    G = K // 128
    s_ng = scales.reshape(N, G).to(torch.float16).numpy()
    z_ng = zeros.reshape(N, G).float().numpy().astype(np.int64)
    qweight, qzeros, s_gn = gptq_pack_bruteforce(codes.reshape(N, K).numpy().astype(np.uint8), z_ng, s_ng)
    g_idx = torch.arange(K, dtype=torch.int32) // 128
    c, s, z, shape = convert.gptq_to_native(torch.from_numpy(qweight).cuda(), torch.from_numpy(qzeros).cuda(),
                                            torch.from_numpy(s_gn).cuda(), g_idx.cuda())
    assert shape == (N, K)
    assert torch.equal(c.cpu(), packed)
    assert torch.equal(z.cpu(), zeros) and torch.equal(s.cpu(), torch.from_numpy(s_ng).to(torch.bfloat16).reshape(-1, 1))
    # the dequantised matrix equals the GPTQ formula (q - (z_stored + 1)) * s of quant_linear.py:339
    w = ops.a16w4_dequant(c, s, z, (N, K)).cpu()
    want = co.dequant(packed.numpy(), bits(s.cpu()), bits(z.cpu()), N, K)
    assert np.array_equal(bits(w), want)
    # and back
    qw2, qz2, s2, g2 = convert.native_to_gptq(c, s, z, (N, K))
    assert np.array_equal(qw2.cpu().numpy(), qweight) and np.array_equal(qz2.cpu().numpy(), qzeros)
    assert torch.equal(g2.cpu(), g_idx)


@pytest.mark.gpu
def test_loaders_fill_modules_like_the_reference_script(hip_lib):
    from latentq_llm_amd import convert, quant
    N, K = 64, 256
    codes, packed, scales, zeros = make_w4(N, K, 5)
    ckt = {"l.qweight": packed, "l.scales": scales.to(torch.float16), "l.zeros": zeros.to(torch.float16),
           "l.bias": torch.randn(N).to(torch.float16)}
    layer = convert.load_a16w4(quant.QLinearA16W4(K, N, bias=True, lbit=16, gbit=16), ckt, "l")
    assert layer.lname == "l" and layer.scales.dtype == torch.bfloat16 and torch.equal(layer.weight.data, packed)
    layer.to("cuda")
    x = torch.randn(8, K).to(torch.bfloat16).cuda()
    y = layer.forward_eval(x) if hasattr(layer, "forward_eval") else layer(x)
    ref = x.float().cpu() @ quant.DeQfunc_4bit_g(packed.cuda(), [scales.cuda(), zeros.cuda(), (N, K)]).float().cpu().t() \
        + ckt["l.bias"].to(torch.bfloat16).float()
    assert torch.allclose(y.float().cpu(), ref, rtol=2e-2, atol=2e-2)

    g = torch.Generator().manual_seed(1)
    q8 = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    ckt8 = {"m.qweight": q8, "m.scales": (torch.rand(N, 1, generator=g) * 0.01 + 1e-3).to(torch.float16),
            "m.inp_absmax": torch.rand(K, generator=g) * 4}
    l8 = convert.load_a8w8(quant.QLinearA8W8(K, N, bias=False, lbit=16, gbit=16), ckt8, "m")
    assert torch.equal(l8.weight.data, (q8.to(torch.int32) - 128).to(torch.int8))
    assert float(l8.clampv) == float(ckt8["m.inp_absmax"].max())
    assert l8.weight.residual.data.dtype == torch.bfloat16 and l8.weight.residual.data.shape == (N, K)
