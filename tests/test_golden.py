"""The committed exact-arithmetic vectors (tests/golden/hot_path_vectors.json, written by
tests/golden/make_golden.py from rational arithmetic and the published Philox known answers)
against the CPU oracle (no GPU needed) and against the HIP kernels (gpu)."""
import json
import os

import numpy as np
import pytest
import torch

from tests.util import bits, from_bits

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def vec():
    with open(os.path.join(HERE, "golden", "hot_path_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def co():
    from oracle import c_oracle
    return c_oracle


def _bf16_tensor(bit_list, shape):
    return from_bits(np.array(bit_list, np.uint16).reshape(shape))


def _pack(codes):
    c = np.array(codes, np.uint8).reshape(-1, 2)
    return ((c[:, 0] << 4) | c[:, 1]).astype(np.uint8)


def _uniform_of(a16):
    """The uniform a 16-bit draw stands for: (a + 1/2) * 2^-16, exact in fp32."""
    return ((np.array(a16, np.float64) + 0.5) * 2.0 ** -16).astype(np.float32)


def _lr(case):
    return float(np.array([case["lr_bits"]], np.uint32).view(np.float32)[0])


# ----------------------------------------------------------------- oracle (CPU) --
def test_oracle_philox_and_uniform(vec, co):
    for k in vec["philox_kat"]:
        assert list(co.philox4x32_10(k["ctr"], k["key"])) == k["out"]
    for s in vec["uniform"]:
        u = co.philox_uniform(len(s["a16"]), s["seed"], s["offset"])
        assert np.array_equal(u, _uniform_of(s["a16"]))


def test_oracle_dequant(vec, co):
    for q, zb, sb, wb in vec["dequant"]:
        got = co.dequant(_pack([q] * 128), np.array([sb], np.uint16), np.array([zb], np.uint16), 1, 128)
        assert int(got.reshape(-1)[0]) == wb and int(got.reshape(-1)[127]) == wb


def test_oracle_requant(vec, co):
    for c in vec["requant"]:
        N, K = c["N"], c["K"]
        args = (_pack(c["codes"]), np.array(c["scale_bits"], np.uint16), np.array(c["zero_bits"], np.uint16),
                np.array(c["grad_bits"], np.uint16), _lr(c), N, K)
        want = _pack(c["new_codes"])
        assert np.array_equal(co.requant(*args, u=_uniform_of(c["a16"])), want)
        assert np.array_equal(co.requant(*args, seed=c["seed"], offset=c["offset"]), want)


def _codec_words(nibbles):
    n = np.array(nibbles, np.uint32).reshape(-1, 8)
    return sum(n[:, k] << (28 - 4 * k) for k in range(8)).astype(np.uint32)


def test_oracle_residual_codec(vec, co):
    for c in vec["residual_codec"]:
        args = (0, c["k1"], c["b1"], c["k2"], c["b2"], c["k3"])
        q, carry = co.residual_quant(np.array(c["x_bits"], np.uint16), *args)
        assert np.array_equal(q, _codec_words(c["nibble"]))
        assert np.array_equal(carry, np.where(np.array(c["carry"]) == 1, 0x3F80, 0).astype(np.uint16))
        vals = co.residual_dequant(np.array([0x01234567, 0x89ABCDEF], np.uint32), *args)
        assert list(vals) == c["value_bits"]


# ------------------------------------------------------------------ HIP kernels --
@pytest.mark.gpu
def test_hip_residual_codec(vec):
    from latentq_llm_amd import ops
    for c in vec["residual_codec"]:
        args = (0, c["k1"], c["b1"], c["k2"], c["b2"], c["k3"])
        x = _bf16_tensor(c["x_bits"], (len(c["x_bits"]),)).cuda()
        q = torch.empty(len(c["x_bits"]) // 8, dtype=torch.int32, device="cuda")
        ops.residual_quant(x, q, *args)
        assert np.array_equal(q.cpu().numpy().view(np.uint32), _codec_words(c["nibble"]))
        assert np.array_equal(bits(x.cpu()), np.where(np.array(c["carry"]) == 1, 0x3F80, 0).astype(np.uint16))
        words = torch.from_numpy(np.array([0x01234567, 0x89ABCDEF], np.uint32).view(np.int32)).cuda()
        assert list(bits(ops.residual_dequant(words, *args).cpu()).reshape(-1)) == c["value_bits"]



@pytest.mark.gpu
def test_hip_uniform(vec):
    from latentq_llm_amd import ops
    for s in vec["uniform"]:
        u = ops.philox_uniform(len(s["a16"]), s["seed"], s["offset"]).cpu().numpy()
        assert np.array_equal(u, _uniform_of(s["a16"]))


@pytest.mark.gpu
def test_hip_dequant(vec):
    from latentq_llm_amd import ops
    cases = vec["dequant"]
    n = len(cases)
    codes = torch.from_numpy(np.concatenate([_pack([q] * 128) for q, _, _, _ in cases]).view(np.int8)).cuda()
    scales = _bf16_tensor([c[2] for c in cases], (n, 1)).cuda()
    zeros = _bf16_tensor([c[1] for c in cases], (n, 1)).cuda()
    w = bits(ops.a16w4_dequant(codes, scales, zeros, (n, 128)).cpu())
    assert np.array_equal(w[:, 0], np.array([c[3] for c in cases], np.uint16))
    assert np.array_equal(w[:, 127], w[:, 0])


@pytest.mark.gpu
def test_hip_requant(vec):
    from latentq_llm_amd import ops
    for c in vec["requant"]:
        N, K = c["N"], c["K"]
        codes = torch.from_numpy(_pack(c["codes"]).view(np.int8)).cuda()
        scales = _bf16_tensor(c["scale_bits"], (N, 1)).cuda()
        zeros = _bf16_tensor(c["zero_bits"], (N, 1)).cuda()
        grad = _bf16_tensor(c["grad_bits"], (N, K)).cuda()
        want = _pack(c["new_codes"])
        u = torch.from_numpy(_uniform_of(c["a16"])).reshape(N, K).cuda()
        got_u = ops.requant_sr(codes, scales, zeros, grad, _lr(c), (N, K), u=u)
        got_p = ops.requant_sr(codes, scales, zeros, grad, _lr(c), (N, K), seed=c["seed"], offset=c["offset"])
        assert np.array_equal(got_u.cpu().numpy().view(np.uint8), want)
        assert np.array_equal(got_p.cpu().numpy().view(np.uint8), want)
