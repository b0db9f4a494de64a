"""Host-side bookkeeping of the batched engines that needs no device: how extents are cut into blocks
(reference optimizers/shampoo2.py:51-59), which parameters a bank takes, how the set of parameters of a
call is normalised, and the schedule by which the eigenbasis bank remembers matrices of low numerical
rank."""
import pytest
import torch

from optimizers.engine import ShampooBank, _Group
from optimizers.engine2 import ShampooBank2
from optimizers.shampoo_common import BlockPartitioner


@pytest.mark.parametrize("extent", [1, 3, 63, 64, 65, 100, 127, 128, 129, 768, 1024, 1025, 2304, 3072])
@pytest.mark.parametrize("block", [0, 1, 4, 64, 100, 128, 1024, 1200])
def test_bank_cuts_an_extent_like_the_partitioner(extent, block):
    pieces = ShampooBank._pieces(extent, block)
    assert sum(pieces) == extent and all(p > 0 for p in pieces)
    if extent * 3 <= 1 << 16:                                 # (the partitioner works on a real tensor)
        part = BlockPartitioner(torch.empty(extent, 3), block)
        rows = [b.shape[0] for b in part.partition(torch.empty(extent, 3))]
        # the second dimension (3) is cut as well when block < 3: take every row-block once
        cols = len(ShampooBank._pieces(3, block))
        assert rows[::cols] == pieces


def test_matrix_view_of_a_parameter():
    shape = ShampooBank.matrix_shape
    assert shape(torch.empty(768, 100)) == (768, 100)
    assert shape(torch.empty(4, 1, 3)) == (4, 3)
    assert shape(torch.empty(16, 3, 3, 3)) == (16, 27)
    assert shape(torch.empty(1, 24, 1, 5)) == (24, 5)
    assert shape(torch.empty(5)) is None
    assert shape(torch.empty(1, 80)) is None and shape(torch.empty(80, 1)) is None
    assert shape(torch.empty(())) is None


def test_bank_takes_only_fp32_gpu_matrices():
    kw = dict(prec_maxorder=1024, min_lowbit_size=4096, quan_blocksize=64)
    assert not ShampooBank.accepts(torch.empty(8, 8), prec_bits=4, **kw)               # a CPU tensor
    assert not ShampooBank.accepts(torch.empty(8, 8, device="meta"), prec_bits=4, **kw)


def test_the_set_of_parameters_of_a_call_is_normalised():
    only = ShampooBank._only
    assert only(None, 5) is None
    assert only(range(5), 5) is None                          # everybody: same as no restriction
    assert only([0, 2], 5) == frozenset({0, 2})
    assert only([], 5) == frozenset()
    assert only([0, 1, 2, 3, 7], 5) == frozenset({0, 1, 2, 3, 7})   # five indices, not the five parameters


def bare_bank():
    bank = object.__new__(ShampooBank2)
    bank.low_rank, bank.low_rank_rows, bank.rank_deficient = {}, {}, {}
    return bank


def test_known_low_rank_rows_are_looked_at_again_after_8_16_up_to_256_updates():
    bank = bare_bank()
    assert bank._known_low_rank(768) == []
    bank._note_repairs(768, [5])
    periods = []
    for _ in range(7):
        # the row counts as known for `period` updates, then goes through the plain sweep with its stack once
        count = 0
        while bank._known_low_rank(768) == [5]:
            count += 1
            assert count <= 256
        periods.append(count)
        bank._note_repairs(768, [5])                          # that look ended in the replacing sweep again
    assert periods == [8, 16, 32, 64, 128, 256, 256]
    # a row that is not repaired at its look is simply not noted again and stays out
    bank = bare_bank()
    bank._note_repairs(1024, [3, 1])
    assert bank._known_low_rank(1024) == [1, 3]
    for _ in range(7):
        bank._known_low_rank(1024)
    assert bank._known_low_rank(1024) == [] and bank._known_low_rank(1024) == []
    assert bank._known_low_rank(768) == []                    # other orders are not touched


def test_a_stack_of_mostly_low_rank_matrices_tries_the_plain_sweep_every_eighth_update():
    bank = bare_bank()
    assert bank._replace_first(768) is False                  # nothing known yet
    bank.low_rank[768][0] = True                              # its last plain sweep ended in the replacing one for most matrices
    answers = [bank._replace_first(768) for _ in range(2 * ShampooBank2.LOOK_AGAIN)]
    assert answers == ([True] * (ShampooBank2.LOOK_AGAIN - 1) + [False]) * 2


def test_low_rank_memory_travels_with_the_checkpoint(monkeypatch):
    bank = bare_bank()
    bank._note_repairs(768, [5])
    bank._note_repairs(768, [5])
    bank._known_low_rank(768)
    bank.low_rank[1024] = [True, 3]
    low_rank = torch.tensor([[o, int(s[0]), int(s[1])] for o, s in sorted(bank.low_rank.items())], dtype=torch.int64).reshape(-1, 3)
    rows = torch.tensor([[o, r, s[0], s[1]] for o, t in sorted(bank.low_rank_rows.items()) for r, s in sorted(t.items())],
                        dtype=torch.int64).reshape(-1, 4)
    other = bare_bank()
    # (the part of load_state_dict that is the bank's own; the tensors of the stacks need a device)
    monkeypatch.setattr(ShampooBank, "load_state_dict", lambda self, sd: None)
    ShampooBank2.load_state_dict(other, {"low_rank": low_rank, "low_rank_rows": rows})
    assert other.low_rank == {1024: [True, 3]}
    assert other.low_rank_rows == {768: {5: [16, 15]}}


def test_statistics_that_cannot_have_full_rank_are_known_from_the_block_shapes():
    # ViT-B/32 with blocks of at most 1024: the order-768 statistics of the 768 x 256 blocks (rank <= 384 + 256) and of the
    # 768 x 100 head (rank <= 384 + 100); every other statistic can have full rank
    shapes = {(768, 1024): 60, (768, 256): 12, (768, 768): 12, (1024, 768): 39, (768, 100): 1}
    groups, rows_of = [], {}
    for (bm, bn), count in shapes.items():
        g = _Group(bm, bn, bn)
        g.param_index = list(range(count))
        for side, order in enumerate((bm, bn)):
            g.slot[side] = (order, rows_of.get(order, 0))
            rows_of[order] = rows_of.get(order, 0) + count
        groups.append(g)
    found = ShampooBank2._rank_deficient_rows(groups)
    assert set(found) == {768}
    first_256 = groups[1].slot[0][1]
    head = groups[4].slot[0][1]
    assert found[768] == sorted(list(range(first_256, first_256 + 12)) + [head])
    bank = bare_bank()
    bank.rank_deficient = found
    assert bank._known_low_rank(768) == found[768] and bank._known_low_rank(768) == found[768]     # every update, no countdown
    bank._note_repairs(768, [0])
    assert bank._known_low_rank(768) == sorted(found[768] + [0])
    assert bank._known_low_rank(1024) == []
