"""A step flattened into one int32 buffer: what lies where, and what is refused."""

from __future__ import annotations

import pytest

from mercury_amd.cache import CacheManager
from mercury_amd.engine.batch import BatchError, SeqChunk, context_from_packed, host_ints
from mercury_amd.hostcore import core
from mercury_amd.parts import CacheSpec

PS = 8
FULL = CacheSpec(kv_heads=2, head_dim=16, window=None)
WINDOW = CacheSpec(kv_heads=2, head_dim=16, window=20)


def pack_step(chunks, manager, vocab_size, max_positions, pinned=False, table_width=-1):
    """Pack on the host alone (no GPU here): pageable memory, no program, no tile lists."""
    packer = core.StepPacker(manager, vocab_size, max_positions, pinned=pinned)
    return packer.pack(chunks, None, table_width)


def context(packed):
    return context_from_packed(packed, host_ints(packed))


def manager_with(requests: dict, slots=None) -> CacheManager:
    m = CacheManager(slots or {0: FULL}, 64, PS, 8)
    for key, tokens in requests.items():
        m.admit(key, [], tokens)
        assert m.grow(key, 0, tokens)
    return m


def test_a_mixed_step_is_laid_out_by_sequence():
    m = manager_with({"a": 21, "b": 9, "c": 3})
    chunks = [SeqChunk("a", [5, 6, 7], 18, [0, 2]),      # the end of a prompt
              SeqChunk("b", [9], 8, [0]),                # a decoded token
              SeqChunk("c", [1, 2, 3], 0, [])]           # a whole prompt, nothing wanted
    packed = pack_step(chunks, m, 100, 64, pinned=False)
    step = context(packed)
    assert step.token_ids.tolist() == [5, 6, 7, 9, 1, 2, 3]
    assert step.positions.tolist() == [18, 19, 20, 8, 0, 1, 2]
    assert step.token_seq.tolist() == [0, 0, 0, 1, 2, 2, 2]
    assert step.cu_q.tolist() == [0, 3, 4, 7]
    assert step.kv_len.tolist() == [21, 9, 3]
    assert step.logit_rows.tolist() == [0, 2, 3]
    assert step.spans == [(0, 3, 18), (3, 1, 8), (4, 3, 0)]
    assert (step.max_q_len, step.max_kv_len, step.all_decode) == (3, 21, False)
    assert step.fresh_slots == [m.sequence("c").state_slot]
    assert step.state_slots.tolist() == [m.sequence(k).state_slot for k in "abc"]
    table = step.block_tables[0]
    assert table.shape == (3, 3)                          # 21 tokens need 3 pages of 8
    assert table[0].tolist() == m.table("a", 0)
    assert table[1].tolist() == m.table("b", 0) + [-1]
    assert table[2].tolist() == m.table("c", 0) + [-1, -1]
    wide = pack_step(chunks, m, 100, 64, pinned=False, table_width=6)
    assert context(wide).block_tables[0].shape == (3, 6)
    assert packed.layout() != wide.layout()


def test_every_group_has_a_table_of_its_own():
    m = manager_with({"a": 40}, {0: FULL, 1: WINDOW})
    m.trim("a", 40)                                       # the window gives its first pages back
    packed = pack_step([SeqChunk("a", [1], 39, [0])], m, 100, 64, pinned=False)
    step = context(packed)
    full, window = step.block_tables
    assert full[0].tolist() == m.table("a", 0) and min(full[0].tolist()) >= 0
    assert window[0].tolist() == m.table("a", 1) and window[0, 0] == -1


@pytest.mark.parametrize("chunks,message", [
    ([], "at least one sequence"),
    ([SeqChunk("a", [], 0, [])], "at least one token"),
    ([SeqChunk("a", [100], 0, [])], "token id"),
    ([SeqChunk("a", [-1], 0, [])], "token id"),
    ([SeqChunk("a", [1, 2], 0, [2])], "wanted index"),
    ([SeqChunk("a", [1, 2], 0, [1, 1])], "twice"),
    ([SeqChunk("a", [1], 64, [])], "limit"),
    ([SeqChunk("a", [1] * 30, 0, [])], "pages"),          # more tokens than the request holds pages for
])
def test_what_cannot_run_is_refused(chunks, message):
    m = manager_with({"a": 21})
    with pytest.raises(BatchError, match=message):
        pack_step(chunks, m, 100, 64, pinned=False)
    with pytest.raises(BatchError, match="width"):
        pack_step([SeqChunk("a", [1], 20, [])], m, 100, 64, pinned=False, table_width=2)
