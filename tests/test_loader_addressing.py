"""CPU model of the fused kernel's K/V tile-copy addressing (natten_amd/csrc/fna_fwd.hpp,
make_copy / copy_one): every byte offset a lane forms must stay inside the K/V tensor and name
the row / chunk the LDS layout expects, for full tiles of the token-permuted layout, for tiles
gathered from the original layout (fused entry point), and for the clamped last tile of an
unpadded sequence.  32-bit unsigned arithmetic is modelled explicitly, because a wrapped
offset is an out-of-bounds access on the device."""

import itertools

import numpy as np
import pytest

U32 = np.uint32
IMM_BIAS = 3 * 1024


def _slots(D, row, slot):
    cpr = D // 8
    rpl = max(16 // cpr, 1)
    k = slot ^ ((row // rpl) % cpr)
    v = slot ^ (2 * ((row // rpl) % (cpr // 2)))
    return k, v


def _geometry(D, nwaves, kvt):
    cpr = D // 8
    chunks = kvt * cpr
    nt = nwaves * 64
    per = (chunks + nt - 1) // nt
    return cpr, chunks, per


@pytest.mark.parametrize("D", [32, 64, 128])
def test_ragged_tile_copy_addresses_stay_in_bounds(D):
    # the ragged instance: 4 waves, 64-key tiles, immediate taken off the uniform base
    nwaves, kvt = 4, 64
    cpr, chunks, per = _geometry(D, nwaves, kvt)
    for heads_kv in (1, 3):
        stride2 = heads_kv * D * 2
        for seqlen_kv in (1, 5, kvt - 1, kvt + 1, 3 * kvt + 17):
            total_bytes = seqlen_kv * stride2
            for kv_row0 in range(0, seqlen_kv, kvt):
                inside = kv_row0 + kvt <= seqlen_kv
                covered = set()
                for wave, i, lane in itertools.product(range(nwaves), range(per), range(64)):
                    if (wave * per + i) * 64 >= chunks:
                        continue
                    imm = (i % 4) * 1024
                    P = (wave * per + i) * 64 + lane
                    row, slot = P // cpr, P % cpr
                    ks, _ = _slots(D, row, slot)
                    # per-lane offset register of copy i % 4, rows of copy i shifted by the uniform base
                    P4 = (wave * per + i % 4) * 64 + lane
                    row4 = P4 // cpr
                    voff = U32(row4) * U32(stride2) + U32(_slots(D, row4, P4 % cpr)[0] * 16)
                    rows_per_4 = 256 // cpr
                    if not inside:
                        over = max(kv_row0 + row4 + (i // 4) * rows_per_4 - (seqlen_kv - 1), 0)
                        voff = U32(voff - U32(over) * U32(stride2))
                    base = kv_row0 * stride2 + (i // 4) * rows_per_4 * stride2 - imm
                    addr = base + int(voff) + imm  # hardware: uniform base + zero-extended offset + immediate
                    assert 0 <= addr and addr + 16 <= total_bytes, (D, heads_kv, seqlen_kv, kv_row0, wave, i, lane, addr)
                    want_row = min(kv_row0 + row, seqlen_kv - 1)
                    assert addr == want_row * stride2 + ks * 16
                    assert (wave * per * 1024) + (i // 4) * 4096 + imm + lane * 16 == P * 16
                    covered.add(P)
                assert covered == set(range(chunks))


def _tile_pos(r, kv_tile, tok_step):
    """Token offset of position r (dimension 0 fastest) of a KV tile; tok_step None = permuted rows."""
    if tok_step is None:
        return r
    t0 = r % kv_tile[0]
    r //= kv_tile[0]
    return t0 * tok_step[0] + (r % kv_tile[1]) * tok_step[1] + (r // kv_tile[1]) * tok_step[2]


LAYOUT_CASES = [
    # (layout X, dilation, kv_tile) with X % (d * t) == 0; None = token-permuted sequence
    None,
    ((30, 48, 80), (1, 1, 1), (1, 8, 8)),
    ((8, 16, 32), (2, 1, 2), (2, 4, 8)),
    ((16, 16, 16), (1, 2, 1), (4, 4, 4)),
    ((512, 1, 1), (2, 1, 1), (64, 1, 1)),
    ((1, 64, 1), (1, 1, 1), (1, 64, 1)),
    ((16, 24, 1), (1, 1, 1), (8, 8, 1)),
    ((4, 2, 64), (1, 1, 2), (1, 2, 32)),
]


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("nwaves", [2, 4, 8])
@pytest.mark.parametrize("case", LAYOUT_CASES)
def test_full_tile_copy_addresses(D, nwaves, case):
    kvt = 64
    cpr, chunks, per = _geometry(D, nwaves, kvt)
    noff = min(per, 4)
    rows_per_4 = 256 // cpr
    for heads_kv in (1, 3):
        stride2 = heads_kv * D * 2
        if case is None:
            kv_tile, tok_step = (kvt, 1, 1), None
            n_tokens = 3 * kvt
            origins = [0, kvt, 2 * kvt]  # first row of each tile
            group_tok = 0
        else:
            X, dil, kv_tile = case
            strides = (X[1] * X[2], X[2], 1)
            tok_step = tuple(d * s for d, s in zip(dil, strides))
            n_tokens = X[0] * X[1] * X[2]
            ext = tuple(x // d for x, d in zip(X, dil))
            group = tuple(d - 1 for d in dil)  # the last dilation group reaches furthest
            group_tok = sum(g * s for g, s in zip(group, strides))
            tiles = [range(0, e, t) for e, t in zip(ext, kv_tile)]
            corner = [(r[0], r[-1]) for r in tiles]
            origins = [sum(o * st for o, st in zip(org, tok_step)) for org in itertools.product(*corner)]
        total_bytes = n_tokens * stride2
        bytes_per_4 = _tile_pos(rows_per_4 % kvt, kv_tile, tok_step) * stride2
        for origin_tok in origins:
            tile_base = (group_tok + origin_tok) * stride2
            covered = set()
            for wave, i, lane in itertools.product(range(nwaves), range(per), range(64)):
                if (wave * per + i) * 64 >= chunks:
                    continue
                # per-lane offset register of copy i % 4
                P4 = (wave * per + i % 4) * 64 + lane
                row4, slot4 = P4 // cpr, P4 % cpr
                off = U32(_tile_pos(row4, kv_tile, tok_step)) * U32(stride2) + U32(_slots(D, row4, slot4)[0] * 16)
                off = U32(off + U32(IMM_BIAS - (i % 4) * 1024))
                assert i % 4 < noff
                src = tile_base - IMM_BIAS + (i // 4) * bytes_per_4
                addr = src + int(off) + (i % 4) * 1024
                P = (wave * per + i) * 64 + lane
                row, slot = P // cpr, P % cpr
                want = tile_base + _tile_pos(row, kv_tile, tok_step) * stride2 + _slots(D, row, slot)[0] * 16
                assert addr == want, (D, nwaves, case, heads_kv, origin_tok, wave, i, lane)
                assert 0 <= addr and addr + 16 <= total_bytes
                assert (wave * per * 1024) + (i // 4) * 4096 + (i % 4) * 1024 + lane * 16 == P * 16
                covered.add(P)
            assert covered == set(range(chunks))


EDGE_CASES = [
    # (layout X, dilation, kv_tile): some extent is not a multiple of dilation x KV tile
    ((57, 20, 88), (2, 1, 1), (2, 4, 8)),
    ((84, 19, 1), (1, 1, 1), (8, 8, 1)),
    ((84, 19, 1), (5, 1, 1), (8, 8, 1)),
    ((125, 1, 1), (1, 1, 1), (64, 1, 1)),
    ((19, 29, 1), (2, 3, 1), (8, 8, 1)),       # group extents (10|9, 10|9): smaller than no tile, uneven groups
    ((5, 25, 1), (1, 1, 1), (4, 16, 1)),       # extent 5 over tiles of 4
    ((3, 7, 9), (1, 2, 2), (4, 4, 4)),         # every group extent smaller than the tile
    ((13, 11, 9), (3, 2, 2), (1, 8, 8)),
]


@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("case", EDGE_CASES)
def test_edge_tile_gathers_stay_inside_the_group(D, case):
    """The instance that clamps (original layout, RAGGED): for every dilation group and every KV tile
    that starts inside the group's extent, each lane's address is that of the row the LDS position
    stands for, with coordinates past the group's extent replaced by the group's last one -- so it
    lies inside the tensor, and inside the group."""
    nwaves, kvt = 4, 64
    cpr, chunks, per = _geometry(D, nwaves, kvt)
    X, dil, kv_tile = case
    assert kv_tile[0] * kv_tile[1] * kv_tile[2] == kvt
    strides = (X[1] * X[2], X[2], 1)
    tok_step = tuple(d * s for d, s in zip(dil, strides))
    n_tokens = X[0] * X[1] * X[2]
    heads_kv = 2
    stride2 = heads_kv * D * 2
    total_bytes = n_tokens * stride2
    for group in itertools.product(*[range(d) for d in dil]):
        ext = tuple(-(-(x - g) // d) for x, g, d in zip(X, group, dil))
        group_tok = sum(g * s for g, s in zip(group, strides))
        for origin in itertools.product(*[range(0, e, t) for e, t in zip(ext, kv_tile)]):
            lim = tuple(min(e - o, t) for e, o, t in zip(ext, origin, kv_tile))
            assert all(l >= 1 for l in lim)
            inside = lim == tuple(kv_tile)
            tile_base = (group_tok + sum(o * st for o, st in zip(origin, tok_step))) * stride2
            for wave, i, lane in itertools.product(range(nwaves), range(per), range(64)):
                imm = (i % 4) * 1024
                P = (wave * per + i) * 64 + lane
                r, slot = P // cpr, P % cpr
                t = (r % kv_tile[0], (r // kv_tile[0]) % kv_tile[1], r // (kv_tile[0] * kv_tile[1]))
                if inside:
                    continue  # the unclamped arithmetic, covered above
                tc = tuple(min(a, l - 1) for a, l in zip(t, lim))
                voff = U32(sum(a * st for a, st in zip(tc, tok_step))) * U32(stride2) + U32(_slots(D, r, slot)[0] * 16)
                src = tile_base - imm
                addr = src + int(voff) + imm
                assert 0 <= addr and addr + 16 <= total_bytes, (case, group, origin, wave, i, lane)
                # the token it names belongs to this group and lies inside its extent
                tok = (addr // stride2)
                crd = (tok // strides[0], (tok // strides[1]) % X[1], tok % X[2])
                assert all(c % d == g for c, d, g in zip(crd, dil, group))
                assert all(c // d == o + a for c, d, o, a in zip(crd, dil, origin, tc))
                assert (wave * per * 1024) + (i // 4) * 4096 + imm + lane * 16 == P * 16
