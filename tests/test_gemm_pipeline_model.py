"""The LDS protocol of the grouped GEMM's four-wave loop, checked on a model.

The loop (csrc/grouped_gemm.hip, `NWAVES == 4`) keeps two tiles in LDS as four halves each (A lower / A upper / B lower /
B upper), copies tile kt + 2 over the halves of tile kt as they fall free, reads every half into registers one quarter
before it is multiplied, and synchronises with one wait on the copy counter plus one workgroup barrier per quarter.
Whether that schedule is free of hazards is a property of the table in the kernel's comment, not of the GPU, so it is
checked here for every length of the contraction range: epochs are the stretches between barriers, the waves of a
workgroup are unordered inside an epoch, a copy may land at any time between its request and the first barrier after
the wait that covers it, and a fragment read whose value is multiplied must see exactly the tile it is meant for.
The model follows the kernel's request order and wait counts (copies counted in groups of four: one half operand per
wave and quarter)."""

import pytest


AL, AU, BL, BU = "A lower", "A upper", "B lower", "B upper"
OUTSTANDING_GROUPS = 6  # s_waitcnt vmcnt(24): the 24 most recent copies of a wave = 6 quarters' worth


def simulate(n_full: int, outstanding: int = OUTSTANDING_GROUPS, swap_q2_q3_copies: bool = False):
    """Returns the list of protocol violations for a range of n_full whole tiles (n_full >= 2)."""
    copies = []  # in request order: half (stage, part), tile, epoch of the request, epoch from which it has landed for all
    reads = []   # half, tile expected, whether the fragments are multiplied, epoch
    epoch = 0

    def copy(stage, part, tile):
        copies.append({"half": (stage, part), "tile": tile, "requested": epoch, "landed": None})

    def quarter_end(leave=outstanding):
        nonlocal epoch
        for c in copies[: max(len(copies) - leave, 0)]:
            if c["landed"] is None:
                c["landed"] = epoch + 1  # after the wait of every wave and the barrier that ends this epoch
        epoch += 1

    def read(stage, part, tile, used=True):
        reads.append({"half": (stage, part), "tile": tile, "used": used, "epoch": epoch})

    X, Y = 0, 1
    # before the loop: tiles 0 and 1 in the loop's request order, A lower and B lower of tile 0 to the registers, then
    # A lower of tile 2 over A lower of tile 0
    for stage, tile in ((X, 0), (Y, 1)):
        for part in (AL, BL, BU, AU):
            copy(stage, part, tile)
    quarter_end()
    read(X, AL, 0)
    read(X, BL, 0)
    quarter_end(leave=10**9)  # a barrier after the reads, no wait on the copies
    copy(X, AL, min(2, n_full - 1))
    quarter_end()

    def step(kt, X, Y, last_pipelined):
        t2, t3 = min(kt + 2, n_full - 1), min(kt + 3, n_full - 1)
        # the fragments read for tile kt + 1 are dropped when the pipelined loop ends with this step
        next_used = not last_pipelined
        read(X, BU, kt)
        copy(X, BL, t2)
        quarter_end()
        read(X, AU, kt)
        copy(X, BU, t2)
        quarter_end()
        read(Y, AL, kt + 1, next_used)
        if swap_q2_q3_copies:
            copy(Y, AL, t3)
        else:
            copy(X, AU, t2)
        quarter_end()
        read(Y, BL, kt + 1, next_used)
        if swap_q2_q3_copies:
            copy(X, AU, t2)
        else:
            copy(Y, AL, t3)
        quarter_end()

    kt = 0
    while kt + 1 < n_full:
        step(kt, X, Y, last_pipelined=False)
        step(kt + 1, Y, X, last_pipelined=kt + 3 >= n_full)
        kt += 2
    quarter_end(leave=0)  # s_waitcnt vmcnt(0) and a barrier
    if kt < n_full:  # an odd number of tiles: the last one is multiplied from LDS, outside the pipeline
        for part in (AL, AU, BL, BU):
            read(X, part, kt)

    problems = []
    for r in reads:
        if not r["used"]:
            continue
        mine = [c for c in copies if c["half"] == r["half"]]
        for i, c in enumerate(mine):
            landed = c["landed"] if c["landed"] is not None else 10**9
            same_bytes = i > 0 and mine[i - 1]["tile"] == c["tile"]  # a repeated request rewrites what is there
            if c["requested"] <= r["epoch"] < landed and not same_bytes:
                problems.append(f"{r['half']} of tile {r['tile']} read in epoch {r['epoch']} while tile {c['tile']} is "
                                f"on its way there (requested {c['requested']}, landed by {landed})")
        there = [c for c in mine if c["landed"] is not None and c["landed"] <= r["epoch"]]
        if not there or there[-1]["tile"] != r["tile"]:
            problems.append(f"{r['half']} read in epoch {r['epoch']} for tile {r['tile']}, holds "
                            f"{there[-1]['tile'] if there else 'nothing'}")
    multiplied = {}
    for r in reads:
        if r["used"]:
            multiplied.setdefault(r["tile"], []).append(r["half"][1])
    for tile in range(n_full):
        if sorted(multiplied.get(tile, [])) != sorted([AL, AU, BL, BU]):
            problems.append(f"tile {tile} multiplied from {sorted(multiplied.get(tile, []))}")
    return problems


@pytest.mark.parametrize("n_full", list(range(2, 70)) + [224, 448])
def test_four_wave_loop_reads_every_half_after_it_landed_and_before_it_is_overwritten(n_full):
    assert simulate(n_full) == []


def test_the_model_sees_a_wait_that_is_too_short_and_a_copy_that_is_too_early():
    """The checker is not vacuous: one more quarter of copies left outstanding, or A lower of the next tile requested
    a quarter early (over the half that quarter still reads), are both reported."""
    assert simulate(8, outstanding=OUTSTANDING_GROUPS + 1)
    assert simulate(8, swap_q2_q3_copies=True)
    assert simulate(9, outstanding=OUTSTANDING_GROUPS + 1) and simulate(9, swap_q2_q3_copies=True)
