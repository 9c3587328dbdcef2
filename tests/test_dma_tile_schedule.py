"""Host-side model of the K walk of sgemm_dma_kernel (backup_1_amd/csrc/sgemm_dma_tile.hpp): whole steps of BK travel
through STAGES LDS buffers by loads whose completion the waves count (vmcnt), the walk is whole unrolled passes over the
buffers followed by the steps that are left, the source pointers stop on the last whole step, and every step is
computed in two halves whose operands are read half a step ahead.  The model replays prologue, walk and barriers for
many K and checks what the kernel relies on: the wait before a barrier covers exactly the loads of the step about to
be read, a buffer is refilled only after every half read from it, the operands of each half come from the buffer that
holds that step, the loads never leave the whole steps, and every step is computed once, in ascending order."""
import pytest

SHAPES = ((32, 4, 4), (64, 3, 8), (32, 4, 8), (64, 3, 4), (64, 3, 6), (16, 2, 4), (16, 2, 2),      # (BK, STAGES, LOADS per wave and step) of the shapes that are built
          (32, 2, 6), (32, 2, 8))      # the convolution kernel of sconv_dma.hpp: same buffers, waits and barriers (its refills past the end fetch nothing instead of the last step again)


def replay(K, BK, STAGES, LOADS):
    full = K // BK
    if full == 0:
        return 0
    issued = []                      # steps in the order their loads went out (LOADS loads each, completing in order)
    pointer = {"step": 0, "fetched": 0}
    lds = {}                         # buffer -> step whose data it holds (once landed)
    pending = {}                     # buffer -> step in flight into it
    computed, reads = [], []

    def issue(buffer):
        assert 0 <= pointer["step"] < full, "a load outside the whole steps"
        assert buffer not in pending, "two steps in flight into one buffer"
        pending[buffer] = pointer["step"]
        issued.append(buffer)
        pointer["fetched"] += 1
        if pointer["fetched"] < full:
            pointer["step"] += 1

    def wait_until_outstanding(n_loads):
        # vmcnt(n): all but the n most recent loads have landed; loads land in issue order
        while len(issued) * LOADS > n_loads:
            buffer = issued.pop(0)
            lds[buffer] = pending.pop(buffer)

    for s in range(STAGES):
        issue(s)
    wait_until_outstanding(LOADS * (STAGES - 1))
    frag = {0: lds[0], 1: None}                           # set 0: first half of step 0

    def k_step(step, v):
        assert frag[0] == step, "first half computed from another step's operands"
        assert lds.get(v) == step, "the buffer of the pass does not hold the step"
        frag[1] = lds[v]                                   # second half's operands, read during the first half
        computed.append((step, 0))
        assert frag[1] == step
        computed.append((step, 1))                         # its first MFMA, then:
        wait_until_outstanding(LOADS * (STAGES - 2))       # own loads of step t+1 have landed
        # barrier: every wave has read both halves of buffer v
        nxt = (v + 1) % STAGES
        if step + 1 < full:
            assert lds.get(nxt) == step + 1, "the next step has not landed behind the barrier"
        del lds[v]
        issue(v)                                           # refill with step t+STAGES (or the last whole step again)
        frag[0] = lds.get(nxt)                             # first half of step t+1 (anything, once past the end)
        reads.append(nxt)

    t0 = 0
    while t0 + STAGES <= full:                             # whole passes
        for v in range(STAGES):
            k_step(t0 + v, v)
        t0 += STAGES
    for v in range(STAGES):                                # the steps that are left
        if t0 + v < full:
            k_step(t0 + v, v)
    wait_until_outstanding(0)
    assert computed == [(s, h) for s in range(full) for h in (0, 1)]
    return full


@pytest.mark.parametrize("shape", SHAPES)
def test_every_k_up_to_three_thousand(shape):
    bk, stages, loads = shape
    assert loads * (stages - 1) <= 63                      # vmcnt is a 6-bit counter
    for K in range(1, 3001):
        replay(K, bk, stages, loads)


@pytest.mark.parametrize("shape", SHAPES)
def test_long_walks(shape):
    bk, stages, loads = shape
    for K in (65536, 65537, 99999, 1 << 20):
        assert replay(K, bk, stages, loads) == K // bk
