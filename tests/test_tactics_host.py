"""Host-side behaviour of the tuned tactic table (no GPU): text export/import round trip, lookup by
the next profiled row count (gemmPluginProfiler.cpp:221-250), rejection of foreign text."""
import pytest
import torch


@pytest.fixture(autouse=True)
def _clean(pkg):
    pkg.functional.clear_tactics()
    yield
    pkg.functional.clear_tactics()


HEADER = "woq-tactics 1\n"
# n k quant_algo group_size out_dtype m | regime mt ns waves pf lds skinny rt k_splits
STREAM_8 = "4096 4096 1 128 2 8 1 1 2 8 4 1 0 0 0\n"
GEMM_64 = "4096 4096 1 128 2 64 2 0 0 0 0 0 0 4 2\n"


def _dtype_code(pkg):
    return pkg.functional._WOQ_DT[torch.bfloat16]


def test_import_export_round_trip(pkg):
    F = pkg.functional
    text = HEADER + STREAM_8.replace(" 2 8 1", " %d 8 1" % _dtype_code(pkg), 1) \
        + GEMM_64.replace(" 2 64 2", " %d 64 2" % _dtype_code(pkg), 1)
    F.import_tactics(text)
    assert F.tactic_count() == 2
    assert F.export_tactics() == text
    F.clear_tactics()
    assert F.tactic_count() == 0 and F.export_tactics() == HEADER


def test_lookup_uses_next_profiled_row_count(pkg):
    F = pkg.functional
    dt = _dtype_code(pkg)
    F.import_tactics(HEADER + "4096 4096 1 128 %d 8 1 1 2 8 4 1 0 0 0\n" % dt
                     + "4096 4096 1 128 %d 64 2 0 0 0 0 0 0 4 2\n" % dt)
    d = lambda m, n=4096, g=128: F.describe_tactic(m, n, 4096, g, 1, torch.bfloat16)
    assert d(8) == "stream mt=1 ns=2 waves=8 pf=4 lds=1"
    assert d(3) == d(8)
    assert d(9) == "gemm exact rt=4 splits=2" and d(64) == d(9)
    assert d(65) == "heuristic"          # above the largest profiled row count
    assert d(8, n=8192) == "heuristic"   # another layer
    assert d(8, g=64) == "heuristic"     # another group size


@pytest.mark.parametrize("text", [
    "", "something else\n", "woq-tactics 2\n", HEADER + "1 2 3\n",
    HEADER + "4096 4096 1 128 2 8 7 1 2 8 4 1 0 0 0\n",    # regime 7
    HEADER + "4096 4096 1 128 2 64 2 0 0 0 0 0 0 5 2\n",   # tile height 5
    HEADER + "4096 4096 1 128 2 0 1 1 2 8 4 1 0 0 0\n",    # m = 0
])
def test_import_rejects(pkg, text):
    F = pkg.functional
    with pytest.raises(Exception):
        F.import_tactics(text)
    assert F.tactic_count() == 0


def test_import_is_all_or_nothing(pkg):
    F = pkg.functional
    with pytest.raises(Exception):
        F.import_tactics(HEADER + STREAM_8 + "garbage\n")
    assert F.tactic_count() == 0
