"""The launch rules are thresholds fitted to measurements; this pins what they decide for every (shape, activation
rows, w_bits) of the benchmark configurations, so that a rule edit cannot move a headline shape unseen.  The expected
table is tests/golden/routing_table.json (written by tests/golden/make_routing_table.py from the shipped rules; see
there for when to regenerate it).  No GPU: the queries only evaluate the rules."""
import importlib.util
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def _maker():
    spec = importlib.util.spec_from_file_location("make_routing_table", os.path.join(HERE, "golden", "make_routing_table.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_routes_of_the_benchmark_shapes_are_the_recorded_ones():
    with open(os.path.join(HERE, "golden", "routing_table.json")) as f:
        want = json.load(f)
    got = json.loads(json.dumps(_maker().build_table()))     # tuples -> lists, as the file has them
    for section in want:
        moved = {k: (want[section][k], got[section].get(k)) for k in want[section] if got[section].get(k) != want[section][k]}
        assert not moved, f"{section}: {len(moved)} entries moved, e.g. {list(moved.items())[:4]}"
        assert set(got[section]) == set(want[section])


def test_the_module_asks_the_library_for_its_crossovers():
    """AnyPrecisionLinear's dispatch (linear.py) and the C rules cannot drift: the Python side has no thresholds."""
    from any_precision_amd import _capi
    from any_precision_amd.linear import fused_gemm_pays, fused_set_pays
    for N, K in ((4096, 4096), (11008, 4096), (4096, 11008), (1024, 4096)):
        for M in (9, 33, 129, 257, 513, 16384):
            for b in range(3, 9):
                assert fused_gemm_pays(M, N, b, K) == _capi.gemm_pays(M, N, K, b)
    for rows in ([4096] * 3, [11008] * 2, [4096, 1024, 1024]):
        for M in (9, 33, 129, 257, 513):
            for b in range(3, 9):
                assert fused_set_pays(M, rows, b, 4096) == _capi.gemm_group_pays(M, rows, 4096, b)
    assert not fused_set_pays(64, [4096] * 5, 3, 4096)      # more members than one launch takes
