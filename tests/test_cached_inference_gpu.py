"""A sequence fed to one Megalodon block piece by piece, with the cache handed
from call to call, must reproduce the single full pass: TimestepNorm continues
its running statistics, the CEMA layer its hidden state (bias term of the
kernel + last-state operator), and attention sees the cached keys and values
of the unfinished chunk in front of the new ones (L2 > L1, and the all-keys
case of a single new token).  Tolerance: the bfloat16 bar, 2e-2 of the
largest output."""
import pytest
import torch

from conftest import rel_err
from megalodon_amd.modules import MegaBlock

pytestmark = pytest.mark.gpu


def _block(chunk):
    torch.manual_seed(11)
    blk = MegaBlock(model_dim=256, z_dim=128, value_dim=512, num_heads=2, cema_ndim=16, chunk_size=chunk,
                    ffn_hidden_dim=512, norm_num_groups=8, init_std=0.05).cuda().bfloat16()
    blk.eval()
    return blk


def _empty_cache(bs, blk, dev):
    m = blk.mega
    k0 = torch.empty(bs, 0, m.local_heads, m.z_head_dim, dtype=torch.bfloat16, device=dev)
    v0 = torch.empty(bs, 0, m.local_heads, m.v_head_dim, dtype=torch.bfloat16, device=dev)
    return ((k0, v0, 0), (None, None, None), None)


@pytest.mark.parametrize("pieces", [
    [300, 212, 200, 1, 1, 310],   # inside a chunk, up to its end, single tokens, rest of the second chunk
    [512, 512],                   # whole chunks
    [1] * 5 + [507, 256, 256],    # decoding from an empty cache
])
def test_piecewise_equals_full_pass(pieces):
    chunk, bs = 512, 2
    assert sum(pieces) == 2 * chunk
    blk = _block(chunk)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(bs, 2 * chunk, 256, generator=g).bfloat16().cuda()
    with torch.no_grad():
        full, none = blk(x)
        assert none is None
        cache = _empty_cache(bs, blk, x.device)
        outs, pos = [], 0
        for n in pieces:
            y, cache = blk(x[:, pos:pos + n].contiguous(), None, None, cache)
            outs.append(y)
            pos += n
            cache_attn, cache_norm, hx = cache
            assert cache_attn[2] == pos % chunk and cache_attn[0].shape[1] == pos % chunk
            assert int(cache_norm[0][0]) == pos
            assert hx is not None and hx.shape == (bs, 256, 16)
    got = torch.cat(outs, dim=1)
    assert rel_err(got, full) <= 2e-2
