"""Host model of the wave-level row search of the scanning form of stage 3
(`combine_send_kernel` with `WaveStreamKeys` / `WaveExpertPrefix` / `RowsScan` /
`count_keys` in csrc/moe_a2a.hip), run on the CPU.

The kernel numbers the valid rows of the padded expert-major buffers g = 0..R-1
in (local expert, position) order. Lane l of every wave keeps the exclusive
prefix of expert l's row count in a register; a lane finds the expert of row g
by binary lifting over OTHER lanes' registers with a wave shuffle, and a shuffle
that names an inactive lane returns 0. The model below reproduces the lanes,
the shuffle (inactive lanes included), the fixed trip counts and the clamped
indices, and checks them against brute force:

  * with the kernel's wave-uniform trip count every lane stays active, every
    row index a lane computes is a valid row of the buffers, lanes past the row
    count are masked out of the counts, and the slots equal the stable order of
    all2all/reference.py:170-199;
  * with the trip count that lets lanes past the row count leave the loop (the
    mistake this replaced), the same search reads 0 from the lanes that left,
    walks to the last expert and indexes past the buffers — the model shows it
    on the host instead of on a GPU.
"""
import numpy as np
import pytest

from oracle import moe_a2a_oracle as orc

WAVE, ROWS, SCAN_UNROLL, META = 64, 4, 8, 5
BLK = WAVE * ROWS  # lanes of a stage-3 workgroup


class Wave:
    """Per-lane registers of one wave: excl / incl of WaveExpertPrefix."""

    def __init__(self, counts, max_recv):
        nle = len(counts)
        assert nle <= WAVE
        c = np.zeros(WAVE, np.int64)
        c[:nle] = np.minimum(np.maximum(counts, 0), max_recv)
        self.incl = np.cumsum(c)
        self.excl = self.incl - c  # lanes at or past nle hold the total
        self.total = int(self.incl[-1])
        self.nle, self.max_recv = nle, max_recv

    def shfl(self, src_lane, active):
        """__shfl(excl, src_lane): the value of another lane's register, 0 if that lane is inactive."""
        src_lane = np.asarray(src_lane)
        return np.where(active[src_lane], self.excl[src_lane], 0)

    def padded_rows(self, g, active):
        """WaveStreamKeys::fetch for one row index per lane (array of 64): the padded row each
        lane would load its key from. `active` marks the lanes still executing."""
        le = np.zeros(WAVE, np.int64)
        step = 32
        while step > 0:
            c = le + step  # at most 63
            v = self.shfl(c, active)
            le = np.where(v <= g, c, le)
            step >>= 1
        first = self.shfl(le, active)
        return le * self.max_recv + (g - first), le

    def locate(self, g):
        """WaveExpertPrefix::locate for a wave-uniform g < total (one ballot)."""
        le = int(np.count_nonzero(self.incl <= g))
        return le, int(self.excl[le])


def expert_major_meta(counts, max_recv, world_size, rng):
    """Padded meta buffer [nle, max_recv, 5] with valid rows in (source rank, token) order and a
    sentinel everywhere else; plus the valid rows in (le, j) order."""
    nle = len(counts)
    padded = np.full((nle, max_recv, META), -77, np.int32)
    for le, n in enumerate(counts):
        src = np.sort(rng.integers(0, world_size, n))
        padded[le, :n, 0] = le
        padded[le, :n, 1] = src
        padded[le, :n, 2] = rng.integers(0, 50, n)
        padded[le, :n, 3] = rng.integers(0, 4, n)
        padded[le, :n, 4] = 0
    stream = np.concatenate([padded[le, :n] for le, n in enumerate(counts)]) if sum(counts) else np.zeros((0, META), np.int32)
    return padded, stream


def model_slots(counts, max_recv, world_size, padded, uniform_trip_count=True):
    """Slots of every valid row as the scanning kernel computes them, workgroup by workgroup.
    Returns (slots, touched padded-row indices). Raises IndexError on an out-of-bounds row."""
    wave = Wave(counts, max_recv)
    R = wave.total
    flat_origin = padded.reshape(-1, META)[:, 1]
    limit = padded.shape[0] * padded.shape[1]
    slots = np.full(R, -1, np.int64)
    touched = set()
    groups = (R + ROWS - 1) // ROWS
    for grp in range(groups):
        g0 = grp * ROWS
        # origin of the group's rows, found by every wave with locate()
        rd = []
        for r in range(ROWS):
            le, first = wave.locate(min(g0 + r, R - 1))
            rd.append(int(padded[le, min(g0 + r, R - 1) - first, 1]))
        cnt = np.zeros(ROWS, np.int64)
        b = 0
        while b < R:  # RowsScan: batches of SCAN_UNROLL * BLK keys
            for w in range(ROWS):
                lanes = np.arange(WAVE) + w * WAVE
                for u in range(SCAN_UNROLL):
                    i = b + lanes + u * BLK
                    if uniform_trip_count:
                        active = np.ones(WAVE, bool)   # every lane runs every trip
                        idx = np.minimum(i, R - 1)      # clamped, masked below
                    else:
                        active = i < R                  # lanes past R have left the loop
                        idx = i
                    rows, _ = wave.padded_rows(idx, active)
                    for lane in np.flatnonzero(active):
                        row = int(rows[lane])
                        if not 0 <= row < limit:
                            raise IndexError(f"lane {lane} of wave {w} reads padded row {row} of {limit}")
                        touched.add(row)
                        if i[lane] < R:
                            d2 = int(flat_origin[row])
                            for r in range(ROWS):
                                before = (np.uint32(d2) < np.uint32(rd[r])) or (d2 == rd[r] and i[lane] < g0 + r)
                                cnt[r] += int(before)
            b += SCAN_UNROLL * BLK
        for r in range(ROWS):
            if g0 + r < R:
                slots[g0 + r] = cnt[r]
    return slots, touched


CASES = {
    "balanced": [5, 7, 3, 6],
    "empty_experts_between": [0, 4, 0, 0, 9, 0, 2, 0],
    "first_and_last_empty": [0, 0, 6, 1, 0],
    "one_row": [0, 1, 0],
    "sixty_four_experts": [1 if le % 3 else 0 for le in range(64)],
    "more_rows_than_one_wave": [70, 0, 66],
    "one_expert_has_everything": [0, 0, 0, 130],
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_search_with_uniform_trip_count_stays_in_bounds_and_is_stable(name):
    counts = CASES[name]
    rng = np.random.default_rng(len(name))
    max_recv, W = max(max(counts), 1) + 3, 4
    padded, stream = expert_major_meta(counts, max_recv, W, rng)
    slots, touched = model_slots(counts, max_recv, W, padded)
    # only valid rows are ever read: never the sentinel rows past an expert's count
    flat = padded.reshape(-1, META)
    assert all(flat[row, 1] != -77 for row in touched)
    # the slots are the stable partition by origin rank of the (le, j) stream
    _, order = orc.return_order(stream, W)
    want = np.empty(len(order), np.int64)
    want[order] = np.arange(len(order))
    assert np.array_equal(slots, want)


def test_locate_skips_empty_experts():
    wave = Wave([0, 3, 0, 2], 8)
    assert [wave.locate(g) for g in range(5)] == [(1, 0), (1, 0), (1, 0), (3, 3), (3, 3)]


def test_lanes_that_leave_the_loop_send_the_search_out_of_bounds():
    """The replaced trip count: in the last batch the lanes past the row count are inactive,
    active lanes read 0 from them, decide every prefix is below g and end at expert 63."""
    counts = [3, 2, 4]  # 9 rows: lanes 9.. of the first wave have nothing to do
    rng = np.random.default_rng(1)
    padded, _ = expert_major_meta(counts, 6, 2, rng)
    with pytest.raises(IndexError, match="reads padded row"):
        model_slots(counts, 6, 2, padded, uniform_trip_count=False)
    model_slots(counts, 6, 2, padded, uniform_trip_count=True)  # the kernel's form does not
