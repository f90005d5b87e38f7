"""The paging producer against the reference's own unit tests (singe/src/nn/decode/step.rs:490-653): every
expected vector below is the one the reference asserts, so this is bit-exact parity on the integers that
feed the kernels."""
import pytest

from singe_amd import error
from singe_amd.decode import PageTable


def integers(tensor):
    return tensor.tolist()


def test_page_tables_give_each_sequence_its_own_pages_and_lengths():
    table = PageTable.create(2, 5, 2)
    assert table.page_count() == 7  # three pages each, and the scratch page
    step = table.step("cpu", [[1, 2, 3], [4]])
    assert integers(step.tokens) == [1, 2, 3, 4]
    assert integers(step.positions) == [0, 1, 2, 0]
    assert integers(step.last_rows) == [2, 3]
    paging = step.paging()
    assert integers(paging.query_offsets) == [0, 3, 4]
    assert integers(paging.page_offsets) == [0, 2, 3]
    assert integers(paging.last_page_lengths) == [1, 1]
    pages = integers(paging.pages)
    assert len(pages) == 8 and pages[0] != pages[1] and pages[1] != pages[2]
    assert integers(step.write_slots) == [0, 1, 0, 0]
    assert integers(step.write_pages) == [pages[0], pages[0], pages[1], pages[2]]
    assert pages[:3] == [0, 1, 2]  # free pages in increasing order from page zero (step.rs:133)


def test_a_padded_step_adds_rows_that_only_padding_reads():
    table = PageTable.create(2, 5, 2).with_padding(6)
    scratch = table.layout().scratch_page
    assert table.table_length() == 6 + 2 + 3
    step = table.step_padded("cpu", [[1, 2, 3], [4]], 8)
    assert integers(step.tokens) == [1, 2, 3, 4, 0, 0, 0, 0]
    assert integers(step.positions) == [0, 1, 2, 0, 1, 2, 3, 4]
    assert integers(step.last_rows) == [2, 3]
    assert integers(step.real_tokens) == [3, 1]
    assert integers(step.sequence_ids) == [0, 0, 0, 1, 1, 1, 1, 1]
    paging = step.paging()
    assert integers(paging.query_offsets) == [0, 3, 8]
    assert integers(paging.page_offsets) == [0, 2, 5]
    assert integers(paging.pages)[3:5] == [scratch, scratch]
    assert integers(paging.last_page_lengths) == [1, 1]
    assert integers(step.write_pages)[4:] == [scratch] * 4
    assert integers(step.write_slots)[4:] == [1, 0, 1, 0]
    step = table.step("cpu", [[5], [6]])  # the padding took no capacity
    assert integers(step.positions) == [3, 1]


def test_padding_stays_within_what_the_table_allows():
    table = PageTable.create(1, 8, 2).with_padding(2)
    with pytest.raises(error.Error):
        table.step_padded("cpu", [[1, 2]], 1)
    with pytest.raises(error.Error):
        table.step_padded("cpu", [[1, 2]], 5)
    step = table.step_padded("cpu", [[1, 2]], 4)
    assert integers(step.last_rows) == [1] and integers(step.paging().query_offsets) == [0, 4]


def test_page_tables_refuse_tokens_past_capacity_and_start_over_after_reset():
    table = PageTable.create(1, 2, 2)
    table.step("cpu", [[1, 2]])
    with pytest.raises(error.Error):
        table.step("cpu", [[3]])
    table.reset()
    assert integers(table.step("cpu", [[3]]).positions) == [0]


def test_page_tables_refuse_steps_without_a_slice_per_sequence_or_any_token():
    table = PageTable.create(2, 2, 2)
    with pytest.raises(error.Error):
        table.step("cpu", [[1]])
    with pytest.raises(error.Error):
        table.step("cpu", [[], []])


def test_a_refused_step_leaves_every_sequence_where_it_was():
    table = PageTable.create(2, 2, 2)
    table.step("cpu", [[1], [2, 3]])
    with pytest.raises(error.Error):
        table.step("cpu", [[4], [5]])
    assert integers(table.step("cpu", [[4], []]).positions)[0] == 1


def test_a_held_sequence_takes_one_row_and_no_capacity():
    table = PageTable.create(2, 3, 2)
    table.step("cpu", [[1, 2], [3]])
    for _ in range(4):
        try:
            step = table.step("cpu", [[], [4]])
        except error.Error:
            continue  # the second sequence runs out, and the held one never does
        assert integers(step.last_rows) == [0, 1] and integers(step.real_tokens) == [0, 1]
        assert integers(step.positions)[0] == 2 and integers(step.paging().last_page_lengths)[0] == 2
        assert integers(step.write_pages)[0] == 4  # the scratch page
    assert integers(table.step("cpu", [[9], []]).positions) == [2, 2]


def test_holding_takes_no_page():
    table = PageTable.create_shared(2, 8, 2, 4)
    table.step("cpu", [[1, 2], [3]])
    assert table.free_pages() == 0
    step = table.step("cpu", [[], [4]])
    assert table.free_pages() == 0 and integers(step.write_pages)[0] == 2


def test_a_released_sequence_starts_over_and_its_pages_serve_another():
    table = PageTable.create_shared(2, 8, 2, 4)
    first = table.step("cpu", [[1, 2, 3], []])
    taken = integers(first.paging().pages)[:2]
    assert table.free_pages() == 0
    with pytest.raises(error.Error):
        table.step("cpu", [[], [5]])
    table.release(0)
    assert table.free_pages() == 2
    step = table.step("cpu", [[], [5]])
    assert integers(step.positions) == [0, 0] and integers(step.write_pages)[1] in taken
    paging = step.paging()
    assert integers(paging.pages)[0] == 2 and integers(paging.page_offsets) == [0, 1, 2]
    assert integers(paging.last_page_lengths) == [1, 1]
    with pytest.raises(error.Error):
        table.release(2)


def test_a_step_that_overruns_the_pool_changes_nothing():
    table = PageTable.create_shared(2, 8, 2, 2)
    with pytest.raises(error.Error):
        table.step("cpu", [[1, 2], [3]])
    assert table.free_pages() == 1
    assert integers(table.step("cpu", [[1, 2], []]).positions) == [0, 1, 0]


def test_a_full_sequence_holds_in_its_last_slot():
    table = PageTable.create(2, 2, 2)
    table.step("cpu", [[1, 2], [3]])
    step = table.step("cpu", [[], [4]])
    assert integers(step.positions) == [1, 1] and integers(step.paging().last_page_lengths) == [2, 2]
