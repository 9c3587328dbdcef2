"""Host-side model of the LDS layout of sconv_dma_kernel (backup_1_amd/csrc/sconv_dma.hpp): where the LDS-DMA loads put
the 16-byte units of a K step and where the fragment reads look for them.  Checked for the shapes that are built: every
float a lane reads is the one the MFMA wants (row, k) and was written by exactly one lane of one load; loads and reads stay
inside their buffers and no two units overlap; the 32 lanes of either half of a wave read 32 different banks (what the
8-byte offset of every other group of 8 rows is for); a read's block and buffer offsets fit the 16-bit offset field."""
import pytest

BK, U, GROUPS = 32, 8, 8
CHUNK = 1024 + 8                     # bytes between the loads' groups of 8 rows
BLOCK_BYTES = 2 * CHUNK              # a block of 16 rows

SHAPES = ((13, 1, 1, 8), (8, 4, 2, 4))       # MI, NI, WAVES_M, WAVES_N


def geometry(mi, ni, wm, wn, stages=2):
    nwaves = wm * wn
    bm, bn = 16 * mi * wm, 16 * ni * wn
    a_loads = (bm * U + 64 * nwaves - 1) // (64 * nwaves)
    b_loads = bn * U // (64 * nwaves)
    a_rows = a_loads * nwaves * 8
    return dict(nwaves=nwaves, bm=bm, bn=bn, a_loads=a_loads, b_loads=b_loads, a_bytes=a_rows // 8 * CHUNK,
                b_bytes=bn // 8 * CHUNK, stages=stages)


def dma_writes(g, stage):
    """byte address in LDS -> (operand, row, unit) for every 16-byte unit the loads of one step write"""
    placed = {}
    for operand, loads, base in (("A", g["a_loads"], stage * g["a_bytes"]),
                                 ("B", g["b_loads"], g["stages"] * g["a_bytes"] + stage * g["b_bytes"])):
        for wave in range(g["nwaves"]):
            for j in range(loads):
                chunk = wave * loads + j
                for lane in range(64):
                    row = chunk * 8 + lane // 8
                    unit = (lane % 8) ^ (lane // 8)            # the unit this lane fetches: its slot is lane % 8
                    addr = base + chunk * CHUNK + 16 * lane
                    for b in range(addr, addr + 16, 4):
                        assert b not in placed, "two units overlap"
                        placed[b] = (operand, row, unit, (b - addr) // 4)
    return placed


def read_address(g, operand, stage, wave_block0, block, grp, lane):
    li, ls = lane % 16, lane // 16
    in_block = (li // 8) * CHUNK + (li % 8) * (U * 16) + ((grp ^ (li & 7)) * 16) + 4 * ls
    base = stage * g["a_bytes"] if operand == "A" else g["stages"] * g["a_bytes"] + stage * g["b_bytes"]
    return base + (wave_block0 + block) * BLOCK_BYTES + in_block


@pytest.mark.parametrize("shape", SHAPES)
def test_reads_find_what_the_loads_wrote(shape):
    mi, ni, wm, wn = shape
    g = geometry(*shape)
    lds_bytes = g["stages"] * (g["a_bytes"] + g["b_bytes"])
    assert lds_bytes <= 160 * 1024
    assert mi * BLOCK_BYTES <= 65536 and ni * BLOCK_BYTES <= 65536          # offset field of ds_read_b32
    assert g["a_bytes"] % 16 == 0 and g["b_bytes"] % 16 == 0
    for stage in range(g["stages"]):
        placed = dma_writes(g, stage)
        assert all(0 <= a < lds_bytes for a in placed)
        for wave in range(g["nwaves"]):
            for operand, blocks, block0 in (("A", mi, (wave // wn) * mi), ("B", ni, (wave % wn) * ni)):
                for block in range(blocks):
                    for grp in range(GROUPS):
                        for lane in range(64):
                            addr = read_address(g, operand, stage, block0, block, grp, lane)
                            want_row = 16 * (block0 + block) + lane % 16
                            assert placed[addr] == (operand, want_row, grp, lane // 16), (operand, wave, block, grp, lane)


@pytest.mark.parametrize("shape", SHAPES)
def test_half_waves_read_all_banks(shape):
    g = geometry(*shape)
    for operand in ("A", "B"):
        for grp in range(GROUPS):
            for half in (0, 1):
                banks = {(read_address(g, operand, 1, 0, 0, grp, lane) // 4) % 32 for lane in range(32 * half, 32 * half + 32)}
                assert len(banks) == 32, (operand, grp, half)


def test_without_the_eight_byte_offset_a_half_wave_shares_banks():
    # the layout on the 16-byte grid (rows of a block 128 bytes apart throughout): 16 banks for 32 lanes
    banks = {((lane % 16) * 32 + ((3 ^ (lane % 16 & 7)) * 4) + lane // 16) % 32 for lane in range(32)}
    assert len(banks) == 16
