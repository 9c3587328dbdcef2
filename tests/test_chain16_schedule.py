"""Host-side model of the K walk of sgemm_chain16_kernel (backup_1_amd/csrc/sgemm_chain16.hpp): whole chunks of BK travel
through DEPTH register sets and three LDS buffers, operands are read one chunk ahead of the MFMAs, a ragged last chunk is
handled apart.  The model replays the kernel's prologue, unrolled loop and guarded remainder for many K and checks what
the kernel relies on: the fetch pointers never leave the whole chunks (they stop on the last one), a register set holds
the chunk that is stored from it, an LDS buffer is read while it holds the chunk wanted and is not overwritten while a
chunk still to be computed has to be read from it, and every chunk is computed exactly once, in ascending order."""
import os

import pytest

BK = 64                    # Chain16::BK
DEPTHS = (2, 4, 8)           # Chain16::DEPTH of the shapes that are built


def replay(K, DEPTH):
    chunks, full = (K + BK - 1) // BK, K // BK
    state = {"pointer": 0}
    sets, lds, frag, computed = {}, {}, {}, []

    def fetch(set_):
        assert state["pointer"] < full, "fetch outside the whole chunks"
        sets[set_] = state["pointer"]
        if state["pointer"] + 1 < full:
            state["pointer"] += 1

    def chunk(c):
        assert frag[c & 1] == c, "the fragments do not hold the chunk being computed"
        computed.append(c)
        frag[(c + 1) & 1] = lds.get((c + 1) % 3)            # read ahead (anything, once past the end)
        victim = lds.get((c + 2) % 3)
        assert victim is None or victim < c or victim >= full, "overwriting a chunk that is still to be read"
        lds[(c + 2) % 3] = sets[(c + 2) % DEPTH]
        fetch((c + 2) % DEPTH)
        # barrier

    if full > 0:
        for d in range(DEPTH):
            fetch(d)
        lds[0], lds[1] = sets[0], sets[1]
        # barrier
        fetch(0)
        fetch(1)
        frag[0] = lds[0]
        c0 = 0
        while c0 + DEPTH <= full:
            for d in range(DEPTH):
                chunk(c0 + d)
            c0 += DEPTH
        for d in range(DEPTH):
            if c0 + d < full:
                chunk(c0 + d)
    if chunks > full:
        computed.append(full)                                # from registers filled before the loop
    assert computed == list(range(chunks))


@pytest.mark.parametrize("depth", DEPTHS)
def test_every_k_up_to_three_thousand(depth):
    for K in range(1, 3001):
        replay(K, depth)


@pytest.mark.parametrize("depth", DEPTHS)
@pytest.mark.parametrize("K", [4096, 4097, 16384, 65536, 65537, 262144])
def test_long_k(K, depth):
    replay(K, depth)


def test_kernel_source_has_the_modelled_constants_and_bounds():
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "backup_1_amd", "csrc")
    src = open(os.path.join(csrc, "sgemm_chain16.hpp")).read()
    assert "BK = 64" in src and "LDS_BUFFERS = 3" in src
    assert "fetch_chunk + 1 < full_chunks" in src and "c0 + DEPTH <= full_chunks" in src
    launches = open(os.path.join(csrc, "sgemm_dense.hip")).read()
    assert "Chain16<2, 1, 4, 4>" in launches and "Chain16<1, 1, 8, 2>" in launches and "Chain16<4, 2, 2, 3>" in launches
