"""The TimestepNorm forward that allocates nothing (its scratch is a static
device array) against the workspace-taking entry point, through the C ABI:
two calls in a row, the second on a smaller input, so that whatever the first
left in the shared array must not leak into the second.  The look-back reads
the predecessors' records in an order that depends on timing, so the two
entry points agree to rounding, not bit for bit: the bars are those of the
operator itself (1e-4 for float32 tensors, 2e-2 for bfloat16 ones), and the
output is also held against the float64 oracle."""
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
    _lib.call("mega_group_timestep_norm_fwd_static", _lib.ptr(x), _lib.i32(_lib.dtype_code(x.dtype)),
              _lib.ptr(io["prev_count"]), _lib.ptr(io["prev_mean"]), _lib.ptr(io["prev_var"]), _lib.ptr(io["gamma"]),
              _lib.ptr(io["beta"]), _lib.ptr(mask), _lib.i64(B), _lib.i64(L), _lib.i64(D), _lib.i64(G),
              _lib.f64(eps), _lib.ptr(y), _lib.ptr(count), _lib.ptr(mean), _lib.ptr(var), _lib.ptr(cummean),
              _lib.ptr(cumrstd), _lib.stream_ptr(dev))
    return y, count, mean, var, cummean, cumrstd


def _check(B, L, D, G, seed):
    io = {k: v.cuda() for k, v in synthetic.timestep_norm_inputs(B, L, D, G, seed).items()}
    got = _call_static(io, G)
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
    _check(4, 2048, 1024, 32, 21)     # 0.1 MB of scratch
    _check(2, 640, 512, 16, 22)       # smaller: the array still holds the first call's records


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
