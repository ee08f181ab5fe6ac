"""The restatement of the reference's KV-cell bookkeeping (tests/oracle_lib.py: KVCells) against behaviour worked out by hand from
llama.cpp:1683-1848 and 6834-6842, 6936-6943: where a step's cells land, when the ring wraps, what the operations on sequences
leave behind, and when a step finds no slot although cells are free."""
import numpy as np

import oracle_lib as ol


def test_steps_land_behind_each_other_and_the_range_grows_in_whole_cells():
    c = ol.KVCells(64)
    first, n, mask = c.decode([0, 1, 2], [[0], [0], [0]])
    assert (first, n, c.head) == (0, 32, 3)                       # at least 32 cells are looked at
    assert np.array_equal(mask[:, :3] == 0, np.tril(np.ones((3, 3), bool)))          # causal inside the step
    assert np.all(mask[:, 3:] == -np.inf)                         # free cells are hidden
    for p in range(3, 40):
        first, n, _ = c.decode([p], [[0]])
        assert first == p and n == max(32, p + 1)
    assert c.head == 40


def test_sequences_do_not_see_each_other_unless_cells_are_shared():
    c = ol.KVCells(32)
    c.decode([0, 1], [[0], [0]])
    c.decode([0, 1], [[1], [1]])
    _, _, mask = c.decode([2, 2], [[0], [1]])
    assert np.array_equal(mask[0, :6] == 0, [True, True, False, False, True, False])
    assert np.array_equal(mask[1, :6] == 0, [False, False, True, True, False, True])
    c.seq_cp(0, 2, 0, 2)                                         # sequence 2 sees sequence 0's first two cells, nothing is copied
    assert c.head == 0
    assert c.seq[0] == {0, 2} and c.seq[1] == {0, 2} and c.seq[4] == {0}
    first, _, mask = c.decode([2], [[2]])
    assert first == 6                                            # the search starts at 0 and skips the six cells in use
    assert np.array_equal(mask[0, :7] == 0, [True, True, False, False, False, False, True])
    c.seq_rm(0, -1, -1)                                          # sequence 0 leaves: shared cells stay for sequence 2, its own are freed
    assert list(c.pos[:7]) == [0, 1, 0, 1, -1, 2, 2]
    assert c.seq[0] == {2} and c.pos[4] == -1 and c.head == 4


def test_freed_cells_are_found_again_and_a_step_needs_one_contiguous_run():
    c = ol.KVCells(32)
    for s in range(4):
        c.decode(list(range(8)), [[s]] * 8)                      # four sequences of eight cells fill the cache
    assert c.head == 0 and all(p >= 0 for p in c.pos)
    assert c.decode([8], [[0]]) is None                          # full
    c.seq_rm(1, 4, -1)                                           # cells 12..15
    c.seq_rm(3, 6, -1)                                           # cells 30, 31
    assert c.head == 30                                          # the last removal's first freed cell
    assert c.decode([0, 1, 2, 3, 4], [[5]] * 5) is None          # six cells are free, but no five in a row
    first, n, _ = c.decode([0, 1, 2, 3], [[5]] * 4)
    assert first == 12 and n == 32
    first, _, _ = c.decode([4, 5], [[5]] * 2)                    # head 16: occupied up to 29, then the two at the end
    assert first == 30 and c.head == 0                           # the head wraps when it reaches the end
    c.seq_keep(5)
    assert [i for i in range(32) if c.pos[i] >= 0] == [12, 13, 14, 15, 30, 31] and c.head == 0
    c.clear()
    assert c.cell_max() == 0 and c.head == 0


def test_a_cell_at_index_zero_alone_does_not_count():
    c = ol.KVCells(64)
    c.decode([0], [[0]])
    assert c.cell_max() == 0                                     # the reference's loop stops above cell 0
    c.decode([1], [[0]])
    assert c.cell_max() == 2


def test_a_context_shift_moves_positions_and_frees_what_falls_off():
    c = ol.KVCells(32)
    c.decode(list(range(10)), 0)
    c.seq_rm(0, 2, 6)                                            # cells 2..5 go
    assert c.head == 2
    c.seq_shift(0, 6, -1, -4)                                    # cells 6..9: positions 2..5
    assert list(c.pos[:10]) == [0, 1, -1, -1, -1, -1, 2, 3, 4, 5] and list(c.delta[6:10]) == [-4] * 4 and c.has_shift
    assert c.head == 0                                           # nothing was freed by the shift: the next search starts at 0
    first, n, mask = c.decode([6], 0)
    assert first == 2 and not c.has_shift and not c.delta.any()  # the step applies the pending shift
    assert np.array_equal(mask[0, :10] == 0, [True, True, True, False, False, False, True, True, True, True])
    c.seq_shift(0, 0, 2, -5)                                     # positions 0 and 1 fall below zero: their cells are freed
    assert c.pos[0] == -1 and c.pos[1] == -1 and not c.seq[0] and c.head == 0
