"""Host-side parts of the measurement script that need no GPU: the multi-GPU refusal, the measurement recipe and the
summariser's handling of a directory without raw files."""
import os
import subprocess
import sys

import bench_summaries

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_recipe_runs_committed_files_only_and_keeps_counter_sets_apart():
    lines = bench_summaries.recipe("OUT")
    assert len(lines) > 40
    for line in lines:
        # every line is bench.py itself or rocprofv3 with bench.py right behind "--"
        assert line.startswith("python3 bench.py") or (line.startswith("rocprofv3 ") and " -- python3 bench.py" in line), line
        if "--pmc" in line:
            assert "--kernel-trace" not in line and "--sys-trace" not in line and "--stats" not in line
            counters = line.split("--pmc ")[1].split(" -d ")[0].split()
            assert sum(c.startswith("SQ_") for c in counters) <= 8
            # FETCH_SIZE takes 3 of the 4 TCC counters of a run, WRITE_SIZE 2
            tcc = sum({"FETCH_SIZE": 3, "WRITE_SIZE": 2}.get(c, 1 if c.startswith("TCC_") else 0) for c in counters)
            assert tcc <= 4, line


def test_summarise_on_an_empty_directory_names_what_is_missing(tmp_path):
    out = tmp_path / "out"
    r = _bench("--summarise", str(tmp_path), "--out", str(out))
    assert r.returncode == 0, r.stderr
    said = r.stdout.strip().splitlines()
    assert len(said) == len(bench_summaries.SECTIONS) and all("needs" in line for line in said)
    assert not any(out.iterdir())


def test_kernel_names_are_read_from_their_mangled_form():
    f = bench_summaries._template_args
    assert f("_ZN12_GLOBAL__N_121segment_reduce_kernelIDF16_Li8EEEvPKT_iPKlS5_liPS1_") == "segment_reduce_kernel<f16, 8>"
    assert f("_ZN12_GLOBAL__N_117pair_wstat_kernelIDF16bEEvPKT_iS3_iPS1_PKiS6_S6_i") == "pair_wstat_kernel<bf16>"
    assert f("(anonymous namespace)::vh_insert_kernel(int const*, long, (anonymous namespace)::VoxelHash)") == "vh_insert_kernel"
