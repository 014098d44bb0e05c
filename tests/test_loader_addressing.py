"""CPU model of the fused kernel's K/V tile-copy addressing (natten_amd/csrc/fna_fwd.hpp,
issue_tile_load): every byte offset a lane forms must stay inside the K/V tensor and name the
row / chunk the LDS layout expects, for full tiles and for the clamped last tile of an
unpadded sequence.  32-bit unsigned arithmetic is modelled explicitly, because a wrapped
offset is an out-of-bounds access on the device."""

import numpy as np
import pytest

U32 = np.uint32


def _slots(D, row, slot):
    cpr = D // 8
    rpl = max(16 // cpr, 1)
    k = slot ^ ((row // rpl) % cpr)
    v = slot ^ (2 * ((row // rpl) % (cpr // 2)))
    return k, v


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("nwaves", [2, 4, 8])
@pytest.mark.parametrize("kvt", [64, 128])
def test_tile_copy_addresses_stay_in_bounds(D, nwaves, kvt):
    cpr = D // 8
    chunks = kvt * cpr
    nt = nwaves * 64
    per = (chunks + nt - 1) // nt
    for heads_kv in (1, 3):
        stride2 = heads_kv * D * 2
        for seqlen_kv in (1, 5, kvt - 1, kvt, kvt + 1, 3 * kvt + 17):
            total_bytes = seqlen_kv * stride2
            for kv_row0 in range(0, seqlen_kv, kvt):
                inside = kv_row0 + kvt <= seqlen_kv
                covered = set()
                for wave in range(nwaves):
                    for i in range(per):
                        if (wave * per + i) * 64 >= chunks:
                            continue
                        imm = (i % 4) * 1024
                        for lane in range(64):
                            P = (wave * per + i) * 64 + lane
                            row, slot = P // cpr, P % cpr
                            ks, _ = _slots(D, row, slot)
                            voff = U32(row) * U32(stride2) + U32(ks * 16)
                            if not inside:
                                over = max(kv_row0 + row - (seqlen_kv - 1), 0)
                                voff = U32(voff - U32(over) * U32(stride2))
                            # hardware: base (64-bit, uniform) + zero-extended lane offset + immediate
                            addr = (kv_row0 * stride2 - imm) + int(voff) + imm
                            assert 0 <= addr and addr + 16 <= total_bytes + (heads_kv - 1) * 0 + 0 or addr + 16 <= total_bytes, (
                                D, nwaves, kvt, heads_kv, seqlen_kv, kv_row0, wave, i, lane, addr)
                            want_row = min(kv_row0 + row, seqlen_kv - 1)
                            assert addr == want_row * stride2 + ks * 16
                            lds = (wave * per * 1024) + (i // 4) * 4096 + imm + lane * 16
                            assert lds == P * 16
                            covered.add(P)
                assert covered == set(range(chunks))
