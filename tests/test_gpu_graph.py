"""GPU tests under HIP graph capture: the C-ABI entry points neither allocate nor synchronise, so a
decode or prefill step built from them can be captured once and replayed. Every replay is checked
against the eager result for the same inputs, with eager work and synchronisations between the
replays (a graph node that only works on its first replay would show here)."""
import pytest
import torch

from tests.util import make_w4, randn_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available()
    from latentq_llm_amd import ops
    return ops


def dev(t):
    return t.cuda()


class _Mlp:
    """down(silu(gate(x)) * up(x)) on preallocated buffers (nothing is allocated inside step())."""

    def __init__(self, ops, M, hid, ffn):
        self.ops, self.shape = ops, (M, hid, ffn)
        self.gate = [dev(t) for t in make_w4(ffn, hid, 1)[1:]]
        self.up = [dev(t) for t in make_w4(ffn, hid, 2)[1:]]
        self.down = [dev(t) for t in make_w4(hid, ffn, 3)[1:]]
        self.x = torch.zeros(M, hid, dtype=torch.bfloat16, device="cuda")
        self.g = torch.empty(M, ffn, dtype=torch.bfloat16, device="cuda")
        self.u = torch.empty_like(self.g)
        self.h = torch.empty_like(self.g)
        self.y = torch.empty(M, hid, dtype=torch.bfloat16, device="cuda")

    def step(self):
        M, hid, ffn = self.shape
        o = self.ops
        o.a16w4_forward(self.x, *self.gate, (ffn, hid), out=self.g)
        o.a16w4_forward(self.x, *self.up, (ffn, hid), out=self.u)
        torch.mul(torch.nn.functional.silu(self.g), self.u, out=self.h)
        o.a16w4_forward(self.h, *self.down, (hid, ffn), out=self.y)


# M = 4: the GEMV; M = 48: the GEMV in chunks or the split reduction; M = 200: split reduction (its
# scratch buffer comes from the graph's memory pool while capturing); M = 640: plain GEMM kernels
@pytest.mark.parametrize("M,hid,ffn", [(4, 512, 1408), (48, 1024, 2816), (200, 1024, 2816), (640, 512, 1408)])
def test_mlp_forward_replays_match_eager(ops, M, hid, ffn):
    blk = _Mlp(ops, M, hid, ffn)
    inputs = [dev(randn_bf16((M, hid), 10 + i)) for i in range(4)]
    want = []
    for x in inputs:  # eager results (also the warm-up that sizes the scratch buffer)
        blk.x.copy_(x)
        blk.step()
        want.append(blk.y.clone())
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        blk.step()  # warm-up on the capture stream (its own scratch buffer)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        blk.step()
    for rep in range(2):
        for x, w in zip(inputs, want):
            blk.x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(blk.y, w), f"replay differs from eager (M={M}, pass {rep})"
            # eager work between replays, through the same entry points and the same scratch
            blk.x.copy_(inputs[0])
            blk.step()
            torch.cuda.synchronize()
            assert torch.equal(blk.y, want[0])


def test_graphs_of_growing_token_counts_keep_their_own_scratch(ops):
    """Graphs captured one after another on one stream for 48, 200 and then 400 tokens (each needing
    more split-reduction scratch than the one before), eager calls of other sizes in between: every
    graph still gives the eager result when replayed afterwards, in any order. The scratch a captured
    call uses comes from its graph's memory pool, and the eager buffer of a stream never moves."""
    hid, ffn = 1024, 2816
    s = torch.cuda.Stream()
    blocks, graphs, wants, xs = [], [], [], []
    for i, M in enumerate((48, 200, 400)):
        blk = _Mlp(ops, M, hid, ffn)
        x = dev(randn_bf16((M, hid), 30 + i))
        blk.x.copy_(x)
        blk.step()
        wants.append(blk.y.clone())
        torch.cuda.synchronize()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            blk.step()
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            blk.step()
        blocks.append(blk); graphs.append(g); xs.append(x)
        # eager traffic of a larger shape on the capture stream and on the default stream
        big = _Mlp(ops, 512, hid, ffn)
        with torch.cuda.stream(s):
            big.step()
        big.step()
        torch.cuda.synchronize()
    for order in ((0, 1, 2), (2, 0, 1), (1, 1, 0)):
        for k in order:
            blocks[k].y.zero_()
            blocks[k].x.copy_(xs[k])
            graphs[k].replay()
            # allocations between replays may land where a freed eager scratch buffer was
            junk = [torch.full((1 << 20,), 7.0, device="cuda") for _ in range(8)]
            torch.cuda.synchronize()
            assert torch.equal(blocks[k].y, wants[k]), (order, k)
            del junk
    before = {k: v.data_ptr() for k, v in ops._WORKSPACE.items()}
    _Mlp(ops, 300, hid, ffn).step()
    torch.cuda.synchronize()
    assert all(ops._WORKSPACE[k].data_ptr() == p for k, p in before.items())
    dev0 = [k for k in ops._WORKSPACE if k[0] == torch.cuda.current_device()]
    assert len(dev0) <= ops.WORKSPACE_MAX_STREAMS


def test_requant_and_a8w8_replay(ops):
    """The requantizer (seed and offset are launch arguments, fixed at capture) and the int8 GEMM."""
    N, K = 256, 1024
    _, packed, scales, zeros = make_w4(N, K, 5)
    p, sc, z = dev(packed), dev(scales), dev(zeros)
    grad = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(p)
    x8 = torch.zeros(300, K, dtype=torch.int8, device="cuda")
    w8 = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda")
    sx, sw = torch.rand(300, device="cuda") + 0.1, torch.rand(N, device="cuda") + 0.1
    grads = [dev(randn_bf16((N, K), 20 + i, 1e-3)) for i in range(3)]
    xs = [torch.randint(-127, 128, (300, K), dtype=torch.int8, device="cuda") for _ in range(3)]
    want = []
    for g, x in zip(grads, xs):
        want.append((ops.requant_sr(p, sc, z, g, 1e-2, (N, K), seed=9, offset=3).clone(), ops.a8w8_forward(x, w8, sx, sw).clone()))
    y8 = [None]
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        ops.requant_sr(p, sc, z, grad, 1e-2, (N, K), seed=9, offset=3, out=out)
        y8[0] = ops.a8w8_forward(x8, w8, sx, sw)
    for rep in range(2):
        for (g, x), (wc, wy) in zip(zip(grads, xs), want):
            grad.copy_(g)
            x8.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, wc) and torch.equal(y8[0], wy), f"pass {rep}"
            ops.requant_sr(p, sc, z, grads[0], 1e-2, (N, K), seed=1, offset=0)  # eager work in between
            torch.cuda.synchronize()


@pytest.mark.parametrize("M", [3, 16, 300])
def test_fused_gate_up_replays_match_eager(ops, M):
    """lq_a16w4_gate_up_silu (the GEMV pass over both matrices for up to 16 tokens, the MFMA kernel above) followed
    by the down projection, captured once and replayed on fresh inputs."""
    hid, ffn = 512, 1408
    gate = [dev(t) for t in make_w4(ffn, hid, 1)[1:]]
    up = [dev(t) for t in make_w4(ffn, hid, 2)[1:]]
    down = [dev(t) for t in make_w4(hid, ffn, 3)[1:]]
    x = torch.zeros(M, hid, dtype=torch.bfloat16, device="cuda")
    h = torch.empty(M, ffn, dtype=torch.bfloat16, device="cuda")
    y = torch.empty(M, hid, dtype=torch.bfloat16, device="cuda")

    def step():
        ops.a16w4_gate_up_silu(x, gate, up, (ffn, hid), out=h)
        ops.a16w4_forward(h, *down, (hid, ffn), out=y)

    inputs = [dev(randn_bf16((M, hid), 30 + i)) for i in range(3)]
    want = []
    for xi in inputs:
        x.copy_(xi)
        step()
        want.append(y.clone())
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        step()
        torch.cuda.synchronize()
        with torch.cuda.graph(g, stream=s):
            step()
    torch.cuda.synchronize()
    for i in (2, 0, 1, 2):
        x.copy_(inputs[i])
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[i]), f"replay with input {i} differs from the eager result"
        _ = (x.float() @ x.float().t()).sum().item()  # eager work between replays
