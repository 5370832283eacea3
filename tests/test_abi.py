"""CPU tests of the C-ABI boundary: the shared library loads, exports every symbol that
include/latentq.h declares, and rejects bad arguments with an error code and message before
touching a device. No kernel is launched here."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "latentq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lq_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(hip_lib):
    syms = declared_symbols()
    assert len(syms) >= 11
    for s in syms:
        assert hasattr(hip_lib, s), f"{s} declared in include/latentq.h but not exported"


def test_binding_covers_header(hip_lib):
    from latentq_llm_amd import _C
    assert set(_C.SIGNATURES) | {"lq_last_error"} == set(declared_symbols())
    assert hip_lib.lq_abi_version() == _C.ABI_VERSION


def test_bad_arguments_are_rejected_without_a_gpu(hip_lib):
    from latentq_llm_amd import _C
    lib = hip_lib
    assert lib.lq_requant_sr(None, None, None, None, None, 0.0, 8, 128, 128, None, 0, 0, None) == -1
    assert b"null pointer" in lib.lq_last_error()
    buf = (C.c_char * 4096)()
    p = C.cast(buf, C.c_void_p)
    assert lib.lq_requant_sr(p, p, p, p, p, 0.0, 8, 100, 128, None, 0, 0, None) == -1
    assert b"multiple of 128" in lib.lq_last_error()
    assert lib.lq_requant_sr(p, p, p, p, p, 0.0, 8, 128, 64, None, 0, 0, None) == -1
    assert b"group" in lib.lq_last_error()
    assert lib.lq_a16w4_fwd(p, p, p, p, None, p, 4, 24, 128, 128, None) == -1
    assert b"multiple of 16" in lib.lq_last_error()
    assert lib.lq_a16w4_dx(p, p, p, p, p, 4, 48, 128, 128, None) == -1
    assert b"multiple of 64" in lib.lq_last_error()
    assert lib.lq_a8w8_fwd(p, p, p, p, None, p, None, 4, 16, 100, None) == -1
    misaligned = C.c_void_p(p.value + 2)
    assert lib.lq_a16w4_fwd(misaligned, p, p, p, None, p, 32, 16, 128, 128, None) == -1
    assert b"aligned" in lib.lq_last_error()
    assert lib.lq_a16w4_fwd_ws(p, p, p, p, None, p, 32, 16, 128, 128, misaligned, 4096, None) == -1
    assert b"workspace" in lib.lq_last_error()
    assert lib.lq_a16w4_dx_ws(p, p, p, p, p, 32, 64, 128, 128, misaligned, 4096, None) == -1
    assert b"workspace" in lib.lq_last_error()
    assert lib.lq_a16w4_dx_ws(p, p, p, p, p, 4, 48, 128, 128, None, 0, None) == -1
    assert b"multiple of 64" in lib.lq_last_error()
    res = C.cast((C.c_char * 4096)(), C.c_void_p)
    assert lib.lq_latent_w4_requant(p, p, p, p, res, 8, 100, 128, 2, 0.125, 2, 0.25, 4, None) == -1
    assert b"multiple of 128" in lib.lq_last_error()
    assert lib.lq_latent_w4_reconstruct(p, p, p, res, p, 8, 128, 128, 2, 0.3, 2, 0.25, 4, None) == -1
    assert b"b1 < b2" in lib.lq_last_error()
    assert lib.lq_calib_copy(p, p, 10, None) == -1
    assert lib.lq_transpose_bf16(p, p, 12, 64, None) == -1
    assert b"multiples of 8" in lib.lq_last_error()
    assert lib.lq_adam8_update(p, p, p, p, p, p, p, p, p, 2048, 2048, 0.9, 0.95, 1e-8, 1e-3, None) == -1
    assert b"exactly one of param and direction" in lib.lq_last_error()
    assert lib.lq_adam8_update(p, p, None, p, p, p, p, p, p, 2048, 512, 0.9, 0.95, 1e-8, 1e-3, None) == -1
    assert b"2048 or 128" in lib.lq_last_error()
    assert lib.lq_adam8_update(p, p, None, p, p, p, p, p, p, 3000, 2048, 0.9, 0.95, 1e-8, 1e-3, None) == -1
    assert b"multiple of the block" in lib.lq_last_error()
    assert lib.lq_adam8_latent_w4_step(p, p, res, p, p, p, p, p, p, p, p, 16, 128, 128, 2048, 2, 0.125, 2, 0.25, 4,
                                       2, 0.3, 2, 0.25, 4, 0.9, 0.95, 1e-8, 1e-3, None) == -1
    assert b"b1 < b2" in lib.lq_last_error()
    with pytest.raises(_C.LatentQError, match="lq_a16w4_dequant"):
        _C.call("lq_a16w4_dequant", None, None, None, None, 1, 128, 128, None)


def header_divisibility_constraints():
    """{entry point: {dimension: modulus}} from the 'X % n == 0 [for lq_name]' statements in the comment
    that precedes each declaration in include/latentq.h."""
    text = open(os.path.join(ROOT, "include", "latentq.h")).read()
    out = {}
    for m in re.finditer(r"/\*(.*?)\*/\s*((?:int\s+lq_[a-z0-9_]+\s*\([^;]*;\s*)+)", text, flags=re.S):
        comment, decls = m.group(1), m.group(2)
        names = re.findall(r"int\s+(lq_[a-z0-9_]+)\s*\(", decls)
        for dim, mod, only in re.findall(r"\b([MNK]) % (\d+) == 0(?: for (lq_[a-z0-9_]+))?", comment):
            for n in ([only] if only else names):
                out.setdefault(n, {})[dim] = int(mod)
    return out


def test_header_divisibility_constraints_are_the_ones_enforced(hip_lib):
    """The header is the contract: every 'X % n == 0' it states is what the entry point enforces.
    Shapes that miss a stated modulus by one (and by half of it) are rejected with a message naming
    that modulus; only rejected shapes are passed, so nothing is ever launched."""
    lib = hip_lib
    cons = header_divisibility_constraints()
    assert cons["lq_a16w4_fwd"] == {"K": 128, "N": 16} and cons["lq_a16w4_dx"] == {"K": 128, "N": 64}
    assert cons["lq_a8w8_fwd"] == {"K": 128, "N": 16} and cons["lq_gradq8_quant"] == {"K": 16}
    buf = (C.c_char * 4096)()
    p = C.cast(buf, C.c_void_p)

    def call(name, M, N, K):
        if name == "lq_a16w4_fwd":
            return lib.lq_a16w4_fwd(p, p, p, p, None, p, M, N, K, 128, None)
        if name == "lq_a16w4_dx":
            return lib.lq_a16w4_dx(p, p, p, p, p, M, N, K, 128, None)
        if name == "lq_a8w8_fwd":
            return lib.lq_a8w8_fwd(p, p, p, p, None, p, None, M, N, K, None)
        if name == "lq_gradq8_quant":
            return lib.lq_gradq8_quant(p, p, p, 0, N, K, None, 0, 0, None)
        raise KeyError(name)

    for name in ("lq_a16w4_fwd", "lq_a16w4_dx", "lq_a8w8_fwd", "lq_gradq8_quant"):
        good = {"M": 32, "N": 256, "K": 1024}
        for dim, mod in cons[name].items():
            for bad in (good[dim] + 1, good[dim] - 1, good[dim] + mod // 2):
                dims = dict(good, **{dim: bad})
                assert call(name, dims["M"], dims["N"], dims["K"]) == -1, (name, dims)
                assert f"multiple of {mod}".encode() in lib.lq_last_error(), (name, dims, lib.lq_last_error())
    # the plan query launches nothing and accepts exactly the stated multiples
    from latentq_llm_amd import ops
    from latentq_llm_amd._C import LatentQError
    for backward, name in ((False, "lq_a16w4_fwd"), (True, "lq_a16w4_dx")):
        n = cons[name]["N"]
        ops.a16w4_plan(32, (3 * n, 1024), backward=backward, compute_units=256)
        with pytest.raises(LatentQError, match=f"multiple of {n}"):
            ops.a16w4_plan(32, (3 * n + n // 2, 1024), backward=backward, compute_units=256)


def test_ops_refuse_cpu_tensors(hip_lib):
    import torch
    from latentq_llm_amd import _C, ops
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    codes = torch.zeros(16 * 64, dtype=torch.int8)
    sz = torch.zeros(16, 1, dtype=torch.bfloat16)
    with pytest.raises(_C.LatentQError, match="no CPU fallback"):
        ops.a16w4_forward(x, codes, sz, sz, (16, 128))


def test_product_does_not_import_the_oracle():
    """The package must never route through oracle/ (test infrastructure)."""
    pkg = os.path.join(ROOT, "latentq_llm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f
                assert "lq_oracle" not in src, f


def test_dispatch_plan_host_logic(hip_lib):
    """The kernel choice of the A16W4 entry points is host arithmetic over (M, N, K, workspace, CUs):
    checked here for a 256-CU device without launching anything."""
    from latentq_llm_amd import ops
    ws = 64 << 20

    def plan(M, N, K, backward=False, workspace=ws):
        return ops.a16w4_plan(M, (N, K), backward=backward, workspace_bytes=workspace, compute_units=256)

    # decode sizes
    assert plan(1, 11008, 4096) == ("gemv", 1, 0) and plan(16, 4096, 11008) == ("gemv", 1, 0)
    assert plan(17, 11008, 4096)[0] == "gemv_chunks"
    # 2048 tokens on the 7B MLP matrices: weights-direct forward, large staged tiles backward, no split
    assert plan(2048, 11008, 4096) == ("direct_128x256", 1, 0)
    assert plan(2048, 4096, 11008) == ("direct_128x256", 1, 0)
    assert plan(2048, 11008, 4096, backward=True) == ("staged_256x128", 1, 0)
    assert plan(2048, 4096, 11008, backward=True) == ("staged_256x128", 1, 0)
    # an odd number of groups per row rules the weights-direct kernel out
    assert plan(2048, 11008, 4096 + 128)[0] != "direct_128x256"
    # one workgroup per compute unit: the staged 128 x 128 tiles when K rules the weights-direct kernels out, else
    # the weights-direct kernel with 128 x 128 tiles (a little faster alone on a unit)
    assert plan(256, 11008, 4096 + 128) == ("staged_128x128", 1, 0)
    assert plan(256, 11008, 4096) == ("direct_128x128", 1, 0)
    assert plan(1024, 4096, 4096) == ("direct_128x128", 1, 0)
    # between one and two rounds of the 128 x 256 tiles the weights-direct kernel with 128 x 128 tiles (three
    # workgroups per compute unit) fills the device better
    for M in (384, 768, 1024, 1536):
        assert plan(M, 11008, 4096) == ("direct_128x128", 1, 0), M
    assert plan(3072, 4096, 11008) == ("direct_128x128", 1, 0)
    assert plan(2048, 11008, 4096 + 128)[0] not in ("direct_128x256", "direct_128x128")
    # skinny grids: split reduction, slices of an even number of steps >= 8 that cover the reduction
    for M, N, K, back in [(128, 11008, 4096, True), (512, 11008, 4096, True), (1024, 11008, 4096, True),
                          (128, 4096, 11008, False), (512, 4096, 11008, False), (200, 2048, 1280, False)]:
        kern, splits, per = plan(M, N, K, back)
        steps = (N if back else K) // 64
        assert kern.startswith("staged") and 2 <= splits <= 8, (M, N, K, back, kern, splits)
        assert per % 2 == 0 and per >= 8 and (splits - 1) * per < steps <= splits * per
        rows = 256 if kern == "staged_256x128" else 128
        cols = K if back else N
        assert -(-M // rows) * -(-cols // 128) * splits <= 256, "at most one workgroup per compute unit"
        # the partial tiles fit the workspace; without one there is no split
        assert splits * M * cols * 4 <= ws
        assert plan(M, N, K, back, workspace=0)[1] == 1
    # a workspace that holds two slices caps the split at two
    M, N, K = 128, 11008, 4096
    assert plan(M, N, K, True, workspace=2 * M * K * 4)[1] == 2
    # bad arguments
    from latentq_llm_amd._C import LatentQError
    with pytest.raises(LatentQError, match="multiple of 64"):
        plan(128, 11008 + 16, 4096, backward=True)
    with pytest.raises(LatentQError, match="multiple of 128"):
        plan(128, 11008, 4096 + 64)
