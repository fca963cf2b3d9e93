"""The committed rocprofv3 summaries are what bench.py reads its measured HBM traffic from: every benchmark
workload's dominant kernel must be found in its file, with a figure."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# (workload, timeline label of its dominant kernel, matrix-core tiles?, the dense second table?)
CASES = [
    ("cfg5_transh", "bwd_tile_kernel", False, False),
    ("cfg1_transe", "score_pos_kernel", False, False),
    ("cfg2_distmult", "bwd_tile_kernel", True, False),
    ("cfg2_complex", "bwd_tile_kernel", True, False),
    ("cfg3_transr", "transr_plan_kernel + transr_fwd_back_kernel", False, False),
    ("cfg3_transr", "transr_plan_kernel + transr_fwd_back_kernel", False, True),
    ("cfg4_rotate", "bwd_tile_kernel", False, False),
]


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("workload,label,mfma,dense", CASES)
def test_profile_holds_the_dominant_kernels_traffic(bench, workload, label, mfma, dense):
    by, names = bench.measured_traffic(workload, label, matrix_core_tiles=mfma, dense=dense)
    assert names, f"profiles/score_path_kernels_{workload}.txt has no row for {label}"
    assert by is not None and by > 0
    want = bench.PROFILE_KERNELS[label]
    assert len(names) == len(want), f"{label}: expected one profile row per kernel of {want}, found {names}"
    if mfma:
        assert all(n.endswith("true>") for n in names), "the matrix-core form of the tile kernel"


def test_every_profile_states_its_commands_and_calibration():
    for w in bench_workloads():
        text = open(os.path.join(ROOT, "profiles", f"score_path_kernels_{w}.txt")).read()
        assert "rocprofv3 --kernel-trace --stats" in text and "--pmc FETCH_SIZE" in text and "--pmc WRITE_SIZE" in text
        assert "-- python3 bench.py" in text, "the program follows -- directly"
        assert "scale factors" in text, "the copy-kernel calibration of the two counters"


def bench_workloads():
    return sorted({c[0] for c in CASES})
