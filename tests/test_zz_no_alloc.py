"""The entry point that allocates nothing (lq_a16w4_fwd_static) against lq_a16w4_fwd_ws, through the
C ABI: same bits, on two calls in a row of which the second is smaller (it reuses the first call's
scratch contents), and a clear error beyond the scratch size."""
import ctypes

import pytest
import torch

from tests.util import make_w4, randn_bf16

pytestmark = pytest.mark.gpu


def _case(_C, ops, M, N, K, seed, ws):
    _, packed, scales, zeros = make_w4(N, K, seed)
    x = randn_bf16((M, K), seed + 1).cuda()
    bias = randn_bf16((N,), seed + 2).cuda()
    p, s, z = packed.cuda(), scales.cuda(), zeros.cuda()
    st = torch.cuda.current_stream().cuda_stream
    want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    _C.call("lq_a16w4_fwd_ws", x.data_ptr(), p.data_ptr(), s.data_ptr(), z.data_ptr(), bias.data_ptr(), want.data_ptr(),
            M, N, K, 128, ws.data_ptr(), ws.numel(), st)
    got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    _C.call("lq_a16w4_fwd_static", x.data_ptr(), p.data_ptr(), s.data_ptr(), z.data_ptr(), bias.data_ptr(), got.data_ptr(),
            M, N, K, 128, st)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K)


def test_static_scratch_entry_point_equals_the_workspace_one(hip_lib):
    from latentq_llm_amd import _C, ops
    assert ops.STATIC_SCRATCH_BYTES == 32 << 20
    ws = torch.empty(ops.STATIC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda")
    big, small = (128, 4096, 11008), (48, 2048, 4096)
    for M, N, K in (big, small):
        kernel, splits, _ = ops.a16w4_plan(M, (N, K), workspace_bytes=ops.STATIC_SCRATCH_BYTES)
        assert splits >= 2, (kernel, splits)  # both cases really go through the scratch
    _case(_C, ops, *big, seed=1, ws=ws)
    _case(_C, ops, *small, seed=2, ws=ws)   # smaller, right after: stale partial tiles beyond its own must not matter
    _case(_C, ops, 8, 4096, 4096, seed=3, ws=ws)      # GEMV: no scratch involved
    _case(_C, ops, 400, 1024, 1024, seed=4, ws=ws)    # a square-ish case with a two-way split


def test_static_scratch_entry_point_rejects_what_does_not_fit(hip_lib):
    from latentq_llm_amd import _C, ops
    M, N, K = 2048, 4096, 128  # 8*M*N = 64 MiB > 32 MiB
    t = torch.zeros(16, device="cuda")
    with pytest.raises(_C.LatentQError, match="static scratch holds"):
        _C.call("lq_a16w4_fwd_static", t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), None, t.data_ptr(),
                M, N, K, 128, None)
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_C.LatentQError):
        ops.a16w4_forward_static(x, torch.zeros(N * K // 2, dtype=torch.int8, device="cuda"),
                                 torch.ones(N * K // 128, dtype=torch.bfloat16, device="cuda"),
                                 torch.zeros(N * K // 128, dtype=torch.bfloat16, device="cuda"), (N, K),
                                 out=torch.empty((M, N), dtype=torch.bfloat16, device="cuda"))
