"""Host-side, bounds-checked emulation of the address arithmetic of the tiled
TimestepNorm kernels (megalodon_amd/csrc/timestep_norm.hip: tsn_fwd_kernel,
tsn_fwd_wave_kernel, tsn_bwd_kernel).  For every workgroup, wave, lane and pass
it restates which 16-byte vector of x / y (dy / dx), which statistics slot and
which look-back record the kernels touch, and checks that each access lies
inside its tensor, that every element of y is written exactly once and that the
records a tile polls belong to its own chain.  The shapes include the ragged
ones the GPU tests run (a last tile of 13 rows, groups narrower than a row of
lanes, 64 lanes per row)."""
import numpy as np
import pytest

K_TL, K_WAVE, K_WAVES, K_WIN = 64, 64, 4, 32


def _lanes_per_row(Dg, vec):
    lanes = Dg // vec
    for lpr in (4, 8, 16, 32, 64):
        if lanes <= lpr:
            return lpr
    raise AssertionError("fast path takes at most 64 lanes per row")


def _fast_path_ok(D, Dg, vec):
    return Dg % vec == 0 and D % vec == 0 and Dg // vec <= 64


def _emulate(B, L, D, G, vec, wave_kernel, backward, time_last=False):
    Dg = D // G
    assert _fast_path_ok(D, Dg, vec)
    LPR = _lanes_per_row(Dg, vec)
    NT = -(-L // K_TL)
    NC = B * G
    tiles = NC * NT
    written = np.zeros(B * L * D // vec, dtype=np.int32)     # 16-byte vectors of y / dx
    stats = np.zeros(B * L * G, dtype=np.int32)              # cummean / cumrstd slots
    # element strides of the statistics: (B, L, G) as the reference stores them, or (B, G, L)
    st_b, st_t, st_g = (G * L, 1, L) if time_last else (L * G, G, 1)
    rec_words = 3 if backward else 2
    n_rec = NC * NT * rec_words
    lane = np.arange(K_WAVE)
    if wave_kernel:
        RPW, P = K_WAVE // LPR, LPR
        work = [(tile // NC, tile % NC, w) for tile in range(tiles) for w in (0,)]
    else:
        RPW = K_WAVE // LPR
        RPP = RPW * K_WAVES
        P = K_TL // RPP
        # the grid holds NT workgroups per chain; the ticket hands out the tiles of a chain in order
        work = [(j, chain, None) for chain in range(NC) for j in range(NT)]
    for j, chain, _ in work:
        b, g = divmod(chain, G)
        t0 = j * K_TL
        col = lane % LPR
        col_ok = col * vec < Dg
        waves = (0,) if wave_kernel else range(K_WAVES)
        for wave in waves:
            for q in range(P):
                r = q * RPW + lane // LPR if wave_kernel else q * (RPW * K_WAVES) + wave * RPW + lane // LPR
                assert r.max() < K_TL
                t = t0 + r
                ok = (t < L) & col_ok
                off = (b * L + t) * D + g * Dg + col * vec
                assert (off[ok] >= 0).all() and (off[ok] + vec <= B * L * D).all()
                assert (off[ok] % vec == 0).all()
                np.add.at(written, off[ok] // vec, 1)
        # wave 0, lane = time step: the saved statistics
        t = t0 + lane
        o = b * st_b + t[t < L] * st_t + g * st_g
        assert (o >= 0).all() and (o < B * L * G).all()
        np.add.at(stats, o, 1)
        # records: own slot, and the window of predecessors (forward) / successors (backward)
        own = (chain * NT + j) * rec_words
        assert 0 <= own and own + rec_words <= n_rec
        base = j + 1 if backward else j - 1
        while True:
            idx = base + lane[:K_WIN] if backward else base - lane[:K_WIN]
            inside = (idx < NT) if backward else (idx >= 0)
            slots = (chain * NT + idx[inside]) * rec_words
            assert (slots >= chain * NT * rec_words).all() and (slots + rec_words <= (chain + 1) * NT * rec_words).all()
            if (~inside).any() or len(idx) == 0:
                break
            base = base + K_WIN if backward else base - K_WIN
    assert (written == 1).all(), "every vector of the output is written exactly once"
    assert (stats == 1).all(), "every (b, t, g) statistics slot is touched exactly once"


SHAPES = [
    # B, L, D, G, vec (4 = float32, 8 = 16-bit)
    (2, 77, 1024, 2, 8),      # 64 lanes per row, ragged last tile of 13 rows
    (2, 77, 1024, 2, 4),      # float32: the group does not fit the fast path's 64 lanes -> skipped below
    (1, 64, 256, 2, 8),       # 16 lanes per row, one full tile
    (3, 130, 96, 3, 8),       # 4 lanes per row, three tiles, the last with two rows
    (2, 200, 512, 4, 4),      # float32, 32 lanes per row
    (1, 8192, 128, 1, 8),     # 128 tiles in a chain: several look-back windows
    (2, 65, 48, 2, 8),        # 24 features per group: lanes past the group are masked off
]


@pytest.mark.parametrize("B,L,D,G,vec", SHAPES)
@pytest.mark.parametrize("time_last", [False, True])
@pytest.mark.parametrize("kernel", ["fwd_workgroup", "fwd_wave", "bwd_workgroup"])
def test_tile_kernels_stay_inside_their_tensors(B, L, D, G, vec, kernel, time_last):
    Dg = D // G
    if not _fast_path_ok(D, Dg, vec):
        pytest.skip("shape goes to the serial kernels")
    if kernel == "fwd_wave" and Dg // vec > 16:
        pytest.skip("the tile-per-wave kernel takes groups of at most 16 lanes")
    _emulate(B, L, D, G, vec, wave_kernel=(kernel == "fwd_wave"), backward=(kernel == "bwd_workgroup"),
             time_last=time_last)
