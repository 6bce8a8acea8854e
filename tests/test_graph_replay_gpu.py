"""The hot operators under HIP graph capture: a captured launch sequence is
replayed several times, with eager work and synchronisations of the program's
own between the replays, and every replay is held against the eager result.
None of the captured C entry points allocates, synchronises or records a memset
(scratch is cleared by kernels).  The Python shim does allocate -- outputs, and
one TimestepNorm workspace per (device, stream, direction) -- so the capture runs
on the stream the warm-up ran on: the workspace then exists before the capture
and only the outputs come from the graph's private pool.  Graphs captured on one
stream share that stream's workspace, so their replays must not overlap."""
import pytest
import torch

from megalodon_amd import extension as ops
from megalodon_amd import synthetic

pytestmark = pytest.mark.gpu


def _replay_and_compare(build, inputs, refresh):
    """build() -> tuple of output tensors from static inputs; refresh(i) rewrites the inputs in place."""
    refresh(0)
    eager0 = [t.clone() for t in build()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):          # warm-up on the capture stream: workspaces and tables exist before capture
            build()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        outs = build()
    for i in (0, 1, 2, 1):
        refresh(i)
        want = [t.clone() for t in build()]        # eager work between the replays
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, want):
            assert torch.allclose(a.float(), b.float(), rtol=2e-2, atol=1e-3), "replay differs from the eager launch"
    refresh(0)
    g.replay()
    torch.cuda.synchronize()
    for a, b in zip(outs, eager0):
        assert torch.allclose(a.float(), b.float(), rtol=2e-2, atol=1e-3), "replay differs from the first eager launch"


def test_cema_recurrence_forward_and_backward_under_graph_replay():
    B, D, N, L = 2, 8, 16, 4096
    prm = {k: v.cuda() for k, v in synthetic.cema_params(D, N, 5).items()}
    lq = prm["q"].log()
    x = torch.empty(B, D, L, dtype=torch.bfloat16, device="cuda")
    dy = torch.empty_like(x)

    def refresh(i):
        g = torch.Generator(device="cuda").manual_seed(100 + i)
        x.copy_(torch.randn(B, D, L, generator=g, device="cuda"))
        dy.copy_(torch.randn(B, D, L, generator=g, device="cuda"))

    def build():
        y, _ = ops.cema_scan_fwd(x, prm["p"], lq, prm["gamma"], prm["omega"])
        dx, dp, dq, dg, dw = ops.cema_scan_bwd(dy, x, prm["p"], lq, prm["gamma"], prm["omega"])
        return y, dx, dp, torch.view_as_real(dq), torch.view_as_real(dg), dw

    _replay_and_compare(build, (x, dy), refresh)


def test_timestep_norm_under_graph_replay():
    B, L, D, G = 2, 1024, 512, 16
    io = {k: v.cuda() for k, v in synthetic.timestep_norm_inputs(B, L, D, G, 9).items()}
    x, dy = io["x"], io["dy"]

    def refresh(i):
        g = torch.Generator(device="cuda").manual_seed(200 + i)
        x.copy_(torch.randn(B, L, D, generator=g, device="cuda"))
        dy.copy_(torch.randn(B, L, D, generator=g, device="cuda"))

    def build():
        y, count, mean, var, cm, cr = ops.group_timestep_norm_fwd(x, io["prev_count"], io["prev_mean"], io["prev_var"],
                                                                  io["gamma"], io["beta"], io["mask"], G, 1e-5)
        dx, dpm, dpv, dg, db = ops.group_timestep_norm_bwd(dy, io["dmean"], io["dvar"], x, io["prev_mean"], count, cm, cr,
                                                           io["gamma"], io["mask"], G)
        return y, mean, var, dx, dg, db

    _replay_and_compare(build, (x, dy), refresh)


def test_float32_convolution_under_graph_replay_after_prepare():
    """The float32 FFT engine keeps a scratch block per stream.  `fftconv_prepare(L, stream=s)`
    makes it (and the tables) for the capture stream ahead of time, so the captured call only
    enqueues; the block then belongs to the graph and is not handed to other streams."""
    L, D = 4096, 64
    g_ = torch.Generator().manual_seed(11)
    x = torch.randn(2, D, L, generator=g_).cuda()
    k = (torch.randn(D, L, generator=g_) / L ** 0.5).cuda()
    base = [x.clone(), x.flip(-1).clone(), (2 * x).clone()]

    def refresh(i):
        x.copy_(base[i])

    refresh(0)
    eager0 = ops.fftconv_fwd(x, k).clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    ops.fftconv_prepare(L, stream=side)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        y = ops.fftconv_fwd(x, k)
    for i in (0, 1, 2, 1):
        refresh(i)
        want = ops.fftconv_fwd(x, k).clone()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), "replay differs from the eager launch"
    refresh(0)
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, eager0)


def test_float32_convolution_scratch_blocks_are_bounded():
    """Six streams run the float32 engine at one transform size: at most four scratch blocks
    (plus those a graph owns) exist afterwards, and a stream that took a block over gets the
    same result as the first."""
    L, D = 8192, 48
    g_ = torch.Generator().manual_seed(12)
    x = torch.randn(1, D, L, generator=g_).cuda()
    k = (torch.randn(D, L, generator=g_) / L ** 0.5).cuda()
    want = ops.fftconv_fwd(x, k)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(6)]
    outs = []
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            for _ in range(3):
                outs.append(ops.fftconv_fwd(x, k))
    torch.cuda.synchronize()
    for o in outs:
        assert torch.equal(o, want)
    assert 1 <= ops.fftconv_scratch_blocks(L) <= 4
