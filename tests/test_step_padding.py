"""How steps are filled up to sizes that run well: the rule for rows, and the entry that stands
for a request that does not exist (host logic, no GPU)."""

from types import SimpleNamespace

from from_scratch_inference_engine_amd.engine.context import HostBatch, filler_entry, padded_tokens
from from_scratch_inference_engine_amd.engine.graphs import padded_rows


def test_rows_of_a_step_that_is_not_a_decode_step():
    assert [padded_tokens(n) for n in (1, 2, 64)] == [1, 2, 64]
    assert [padded_tokens(n) for n in (65, 100, 128)] == [128, 128, 128]
    # the next multiple of 256 where that adds at most a fifth, or 64 rows
    assert [padded_tokens(n) for n in (129, 192, 200, 300, 448, 777, 1000, 1088, 2048, 3000)] == \
        [129, 256, 256, 300, 512, 777, 1024, 1280, 2048, 3072]
    for n in range(1, 5000):
        up = padded_tokens(n)
        assert n <= up < n + 256 and (up == n or up % 128 == 0) and padded_tokens(up) == up


def test_rows_of_a_decode_graph():
    assert [padded_rows(n) for n in range(1, 10)] == [1, 2, 4, 4, 8, 8, 8, 8, 16]
    for n in range(1, 300):
        up = padded_rows(n)
        assert n <= up <= max(2 * n, n + 31) and padded_rows(up) == up


def test_the_filler_reads_and_writes_spare_places_only():
    # two groups of layers; a page of the second holds 16 positions (a need with a geometry of its own)
    storage = SimpleNamespace(spare_slot=5, spare_pages=[40, 17], tokens_per_page=[8, 16])
    e = filler_entry(storage, 37)
    assert len(e.tokens) == 37 and set(e.tokens) == {0} and tuple(e.want) == ()
    assert e.cache.length == 0 and e.cache.slot == 5
    assert e.cache.tables == [[40] * 5, [17] * 3]          # every page of its table is the spare one
    host = HostBatch([e], page_size=8)
    assert host.n_tokens == 37 and host.positions.tolist() == list(range(37)) and host.want_rows.size == 0
