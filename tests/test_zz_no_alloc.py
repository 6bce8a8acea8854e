"""The TimestepNorm forward that allocates nothing (its scratch is a static
device array) against the workspace-taking entry point, through the C ABI:
two calls in a row, the second on a smaller input, so that whatever the first
left in the shared array must not leak into the second.  The look-back reads
the predecessors' records in an order that depends on timing, so the two
entry points agree to rounding, not bit for bit: the bars are those of the
operator itself (1e-4 for float32 tensors, 2e-2 for bfloat16 ones), and the
output is also held against the float64 oracle.  Once the first call has taken
the array's address, a call must leave the device's free memory where it was
(hipMemGetInfo before and after, outputs allocated beforehand), and it must be
capturable: a graph of the call is replayed and compared as well."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd import _lib, synthetic
from megalodon_amd import extension as ops
from oracle import timestep_norm as otn

pytestmark = pytest.mark.gpu


def _call_static(io, G, eps=1e-5):
    x = io["x"]
    B, L, D = x.shape
    dev = x.device
    y = torch.empty_like(x)
    count = torch.empty(B, dtype=torch.int64, device=dev)
    mean = torch.empty(B, G, dtype=x.dtype, device=dev)
    var = torch.empty(B, G, dtype=x.dtype, device=dev)
    cummean = torch.empty(B, L, G, dtype=torch.float32, device=dev)
    cumrstd = torch.empty(B, L, G, dtype=torch.float32, device=dev)
    mask = io["mask"].to(torch.uint8).contiguous()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    _lib.call("mega_group_timestep_norm_fwd_static", _lib.ptr(x), _lib.i32(_lib.dtype_code(x.dtype)),
              _lib.ptr(io["prev_count"]), _lib.ptr(io["prev_mean"]), _lib.ptr(io["prev_var"]), _lib.ptr(io["gamma"]),
              _lib.ptr(io["beta"]), _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G),
              _lib.f64(eps), _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(var), _lib.ptr(cummean),
              _lib.ptr(cumrstd), _lib.stream_ptr(dev))
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info(dev)[0]
    return (y, count, mean, var, cummean, cumrstd), free_before - free_after


def _check(B, L, D, G, seed, first_call=False):
    io = {k: v.cuda() for k, v in synthetic.timestep_norm_inputs(B, L, D, G, seed).items()}
    got, taken = _call_static(io, G)
    # (the very first call on a device may load the code object and take the array's address)
    assert first_call or taken == 0, f"the call took {taken} bytes of device memory"
    want = ops.group_timestep_norm_fwd(io["x"], io["prev_count"], io["prev_mean"], io["prev_var"], io["gamma"],
                                       io["beta"], io["mask"], G, 1e-5)
    # no tile of the static-scratch launch ran out of its bounded wait (NULL = the static buffer)
    _lib.call("mega_group_timestep_norm_status", _lib.ptr(None), _lib.stream_ptr(io["x"].device))
    torch.cuda.synchronize()
    assert torch.equal(got[1], want[1])                               # count: integers
    assert rel_err(got[0], want[0]) <= 2e-2                           # y, bfloat16
    assert rel_err(got[2], want[2]) <= 2e-2 and rel_err(got[3], want[3]) <= 2e-2
    live = ~io["mask"]                                                # statistics at unmasked steps
    assert rel_err(got[4][live], want[4][live]) <= 1e-4 and rel_err(got[5][live], want[5][live]) <= 1e-4
    cpu = {k: v.cpu() for k, v in io.items()}
    oy = otn.group_timestep_norm_fwd(cpu["x"].double(), cpu["prev_count"], cpu["prev_mean"].double(),
                                     cpu["prev_var"].double(), cpu["gamma"].double(), cpu["beta"].double(),
                                     cpu["mask"], G, 1e-5)[0]
    assert rel_err(got[0], oy) <= 2e-2


def test_static_scratch_forward_two_calls_in_a_row():
    _check(4, 2048, 1024, 32, 21, first_call=True)     # 0.1 MB of scratch
    _check(2, 640, 512, 16, 22)       # smaller: the array still holds the first call's records


def test_static_scratch_forward_under_graph_capture():
    """What the entry point is for: a capture of the call (nothing in it allocates), replayed on
    fresh inputs with eager work in between, against the eager call."""
    B, L, D, G = 2, 1024, 512, 16
    io = {k: v.cuda() for k, v in synthetic.timestep_norm_inputs(B, L, D, G, 23).items()}
    x = io["x"]
    y = torch.empty_like(x)
    count = torch.empty(B, dtype=torch.int64, device=x.device)
    mean, var = (torch.empty(B, G, dtype=x.dtype, device=x.device) for _ in range(2))
    cm, cr = (torch.empty(B, L, G, dtype=torch.float32, device=x.device) for _ in range(2))
    mask = io["mask"].to(torch.uint8).contiguous()

    def launch():
        _lib.call("mega_group_timestep_norm_fwd_static", _lib.ptr(x), _lib.i32(_lib.dtype_code(x.dtype)),
                  _lib.ptr(io["prev_count"]), _lib.ptr(io["prev_mean"]), _lib.ptr(io["prev_var"]),
                  _lib.ptr(io["gamma"]), _lib.ptr(io["beta"]), _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D),
                  _lib.i64(G), _lib.f64(1e-5), _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(var),
                  _lib.ptr(cm), _lib.ptr(cr), _lib.stream_ptr(x.device))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()                      # the array's address is taken outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        launch()
    for i in range(3):
        gen = torch.Generator(device="cuda").manual_seed(300 + i)
        x.copy_(torch.randn(B, L, D, generator=gen, device="cuda"))
        want = ops.group_timestep_norm_fwd(x, io["prev_count"], io["prev_mean"], io["prev_var"], io["gamma"],
                                           io["beta"], io["mask"], G, 1e-5)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert rel_err(y, want[0]) <= 2e-2 and torch.equal(count, want[1])
        live = ~io["mask"]
        assert rel_err(cm[live], want[4][live]) <= 1e-4 and rel_err(cr[live], want[5][live]) <= 1e-4


def test_static_scratch_forward_refuses_what_does_not_fit():
    fn = _lib.load().mega_group_timestep_norm_static_scratch_bytes
    fn.restype = _lib.ctypes.c_int64
    limit = int(fn())
    B, L, D, G = 64, 65536, 2048, 64
    assert ops._lib.load().mega_group_timestep_norm_workspace_bytes  # the query the limit is compared with
    x = torch.zeros(1, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="static"):
        _lib.call("mega_group_timestep_norm_fwd_static", _lib.ptr(x), _lib.i32(1), _lib.ptr(x), _lib.ptr(x),
                  _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(None), _lib.i64(B), _lib.i64(L), _lib.i64(D),
                  _lib.i64(G), _lib.f64(1e-5), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x), _lib.ptr(x),
                  _lib.ptr(x), _lib.stream_ptr(x.device))
    assert limit == 2 << 20
