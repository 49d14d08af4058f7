"""The counted waits of the generated GEMM loops with the early stage hand-back (csrc/gen_gemm_loop.py): a wave's
copy requests return in order, and every wait names how many of the youngest may still be out.  Simulated here for
whole K loops of two and three stages: at each wait the part of a stage that is about to be read (second weight half
at the mid-step wait, activations and first weight half of the next step at the end-of-step wait) must lie outside
the youngest `vmcnt` requests, whatever the wave's share of the copies.  A count that is too loose would let the
matrix instructions read a stage before its copy has landed."""
import importlib.util
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("gen_gemm_loop", os.path.join(HERE, "..", "g-core-gh_amd", "csrc", "gen_gemm_loop.py"))
gen = importlib.util.module_from_spec(spec)
spec.loader.exec_module(gen)

# name -> (configure arguments, [(requests in the mid part, requests in the end part)] for the kinds of wave in the tile)
LOOPS = {
    "big 256x256": ((256, 256, 4, 2, 1, False, 2, False, True), [(4 + 2, 2)]),
    "wide 256x288": ((256, 288, 4, 2, 1, False, 2, False, True, True), [(4 + 2, 3), (4 + 2, 2)]),        # waves 0..3 copy a fifth group
    "wide 256x224": ((256, 224, 4, 2, 1, False, 2, False, True, True), [(4 + 2, 2), (4 + 2, 1)]),        # waves 0..3 copy a fourth group
    "flat 128x256, three stages": ((128, 256, 2, 4, 1, False, 3, False, True), [(2 + 4, 0), (2, 4)]),    # first / second half of the waves
    # weights stored [K, N]: the activation rows mid-step, every weight row at the end of the step
    "big 256x256, weights stored [K, N]": ((256, 256, 4, 2, 1, True, 2, False, True, False, True, True, True), [(4, 4)]),
    "flat 128x256, three stages, weights stored [K, N]": ((128, 256, 2, 4, 1, True, 3, False, True, False, True, False, True), [(2, 4)]),
}


@pytest.mark.parametrize("name", list(LOOPS))
@pytest.mark.parametrize("trips", [1, 2, 5])
def test_waits_cover_what_is_read(name, trips):
    cfg, kinds = LOOPS[name]
    gen.configure(*cfg)
    nst, steps = gen.NSTAGE, 4 * trips
    for mid, end in kinds:
        issued = []                                   # one entry per request: (part, step it fills)
        # prologue: all stages requested in the order of the steady state
        for st in range(nst):
            issued += [("mid", st)] * mid + [("end", st)] * end
        for step in range(steps):
            c, last = step % 4, step // 4 == trips - 1
            for at_end in (False, True):
                if gen.NN and not at_end:
                    needs = []                        # the mid-step wait of these loops waits for no copy
                    allowed = len(issued)
                else:
                    allowed = gen.younger_requests(c, at_end, last)
                    # weights stored [K, N]: a step reads all of its stage from its first block on, so both parts of the
                    # next step's stage must have landed at the end of this one
                    needs = ([("mid", step + 1), ("end", step + 1)] if gen.NN else [("mid", step + 1)]) if at_end else [("end", step)]
                landed = issued[:len(issued) - allowed] if allowed else issued
                for need in needs:
                    if need[1] < steps:
                        n_need = sum(1 for r in issued if r == need)
                        assert n_need == (mid if need[0] == "mid" else end)
                        assert sum(1 for r in landed if r == need) == n_need, (name, step, at_end, allowed)
                # after the wait and the barrier this wave requests the freed part for the step nst ahead
                if step + nst < steps:
                    issued += [("mid" if not at_end else "end", step + nst)] * (mid if not at_end else end)
