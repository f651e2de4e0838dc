"""The C++ driver with the reference's sspmm_test command line, run on CVSE files and synthetic input."""
import os
import shutil
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "sspmm_amd", "bin", "sspmm_test")
GOLDEN = os.path.join(ROOT, "tests", "golden")


def run(args, cwd, env=None):
    e = dict(os.environ)
    e.update(env or {})
    print("run", args, flush=True)
    return subprocess.run([BIN] + [str(a) for a in args], cwd=cwd, env=e, capture_output=True, text=True, timeout=120)


@pytest.mark.parametrize("mixed", [0, 1])
def test_synthetic_runs_and_verifies(built_library, tmp_path, mixed):
    r = run(["--synthetic", 512, 512, 8, 0.9, 256, mixed, 1], tmp_path)
    assert r.returncode == 0, r.stderr
    assert "Results verified" in r.stdout and "GFlops" in r.stdout


@pytest.mark.parametrize("V", [8, 16])
def test_reference_command_line_on_cvse_files(built_library, tmp_path, V):
    """Ten positional arguments, pattern files from RowMerge, one CSV row per matrix."""
    bench = tmp_path / "benchmark" / ("dlmc-v%d" % V)
    bench.mkdir(parents=True)
    names = ["rand_64x512", "skew_24x70000", "empty_17x32"]
    for n in names:
        shutil.copy(os.path.join(GOLDEN, "%s.v%d.smtx" % (n, V)), bench / (n + ".smtx"))
    work = tmp_path / "run"
    (work / "data").mkdir(parents=True)
    (work / "paths.txt").write_text("".join(n + ".smtx\n" for n in names))
    r = run(["paths.txt", 128, V, 1, 1, 1, 0, 1, 0, "gfx950"], work, {"SSPMM_BENCHMARK_DIR": str(tmp_path / "benchmark")})
    assert r.returncode == 0, r.stderr + r.stdout
    assert r.stdout.count("Results verified") == len(names)
    assert "matrix num:3" in r.stdout
    rows = (work / "data" / ("gfx950_rospmm_%d_v0.csv" % V)).read_text().strip().splitlines()
    assert len(rows) == len(names)
    first = rows[0].split(",")
    assert len(first) >= 5 and int(first[3]) == 128  # nnz, m_vec, K, N, GFLOP/s, ...


def test_a_mismatch_fails_the_run(built_library, tmp_path):
    """The verification decides the exit status: with a tolerance no fp16 result can meet, the run fails."""
    r = run(["--synthetic", 256, 256, 8, 0.9, 128, 1, 1], tmp_path, {"SSPMM_REL_TOL": "1e-12"})
    assert r.returncode == 2, r.stdout
    assert "does not agree" in r.stdout


def test_wrong_argument_count_prints_usage(built_library, tmp_path):
    r = run(["paths.txt", 128], tmp_path)
    assert r.returncode == 1 and "sspmm_test <paths.txt>" in r.stdout
