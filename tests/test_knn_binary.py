"""The `knn` driver: command line, CSV rows, checksums (reference src/main.cpp, docs/knn.md,
docs/data-format.md).  The CPU tests cover everything that happens before the device is touched;
the GPU tests reproduce reference-held checksums end to end through the binary, which also pins
the driver's own input generation."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KNN = os.path.join(ROOT, "bits-knn-jpdc2024_amd", "knn")

HEADER = ("algorithm,generator,preprocessor,iteration,point_count,query_count,dim,block_size,k,"
          "items_per_thread,deg,phase,time")
PHASES = ["prepare", "transfer-in", "distances", "selection", "postprocessing", "finish", "transfer-out"]


def run(*args, timeout=300, env=None):
    assert os.path.exists(KNN), "build the driver with `make -C bits-knn-jpdc2024_amd knn`"
    return subprocess.run([KNN, *args], capture_output=True, text=True, timeout=timeout, env=env)


def checksums(proc):
    return [int(line.split(":")[1]) for line in proc.stderr.splitlines() if line.startswith("Checksum:")]


# ---------------------------------------------------------------------------------------------
# no GPU needed
# ---------------------------------------------------------------------------------------------

def test_header():
    p = run("--header")
    assert p.returncode == 0 and p.stdout.strip() == HEADER


def test_help_lists_options_and_algorithms_on_stderr():
    p = run("--help")
    assert p.returncode == 0 and p.stdout == ""
    for token in ("--algorithm", "--items-per-thread", "--point-layout", "--deg", "--no-output",
                  "Available algorithms:", "- bits", "- bits-prefetch", "- bits-sq", "- fused-cache", "- fused-cache-mfma", "- fused-cache-bf16x3",
                  "- magma-dist", "- magma-part-dist", "- magma-part-dist-bf16x3", "- cublas-dist", "- serial", "- parallel"):
        assert token in p.stderr


def test_unknown_algorithm_prints_help_and_fails():
    p = run("-a", "does-not-exist", "-n", "16", "-q", "1", "--seed", "1")
    assert p.returncode == 1
    assert "Unknown algorithm: 'does-not-exist'" in p.stderr and "Available algorithms:" in p.stderr


@pytest.mark.parametrize("args,msg", [
    (("-d", "0"), "Dimension must be greater than 0"),
    (("-n", "0"), "Number of objects in the database must be greater than 0"),
    (("-q", "0"), "Number of query objects must be greater than 0"),
    (("-k", "0"), "Number of nearest neighbors must be greater than 0"),
    (("--block-size", "0"), "Block size must be greater than 0"),
    (("-g", "poisson"), "Unknown generator: 'poisson'"),
    (("-p", "shuffled", "--seed", "3", "-n", "8", "-q", "1"), "Unknown preprocessor: 'shuffled'"),
])
def test_validation_messages(args, msg):
    p = run(*args)
    assert p.returncode == 1 and msg in p.stderr


# ---------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------

@pytest.mark.gpu
def test_csv_rows_and_phases():
    p = run("-a", "bits", "-n", "64k", "-q", "16", "-k", "32", "--seed", "24", "-r", "3",
            "--block-size", "256", "--items-per-thread", "8")
    assert p.returncode == 0, p.stderr
    rows = [line.split(",") for line in p.stdout.strip().splitlines()]
    assert len(rows) == 3 * len(PHASES)
    for i, row in enumerate(rows):
        # items_per_thread is quoted "a,b,c" and therefore splits into three fields
        assert row[:3] == ["bits", "uniform", "identity"]
        assert row[3] == str(i // len(PHASES))
        assert row[4:9] == ["65536", "16", "1", "256", "32"]
        assert row[9:12] == ['"8', "1", '1"']
        assert row[12] == "1" and row[13] == PHASES[i % len(PHASES)]
        assert "e" in row[14] and float(row[14]) >= 0
    assert len(set(checksums(p))) == 1 and len(checksums(p)) == 3


@pytest.mark.gpu
@pytest.mark.parametrize("alg", ["bits", "bits-prefetch"])
def test_golden_kselection_checksums_end_to_end(golden, alg):
    for rec in golden:
        if rec["family"] != "kselection" or (rec["n"], rec["q"]) != (1 << 20, 1024):
            continue
        p = run("-a", alg, "-n", "1M", "-q", "1k", "-k", str(rec["k"]), "--seed", "24",
                "--block-size", "256", "--items-per-thread", "8")
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (rec["k"], checksums(p))


@pytest.mark.gpu
@pytest.mark.parametrize("pre", ["ascending", "descending"])
def test_golden_buffer_checksums_end_to_end(golden, pre):
    for rec in golden:
        if rec["family"] != "buffer" or rec["preprocessor"] != pre or (rec["n"], rec["q"]) != (1 << 18, 4096):
            continue
        if rec["k"] not in (32, 256, 2048):
            continue
        p = run("-a", "bits", "-n", "256k", "-q", "4k", "-k", str(rec["k"]), "--seed", "24", "-p", pre,
                "--block-size", "128", "--items-per-thread", "1")
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (pre, rec["k"], checksums(p))


@pytest.mark.gpu
def test_golden_buffer_checksums_partial_bitonic_regs(golden):
    """The reference's runs of partial-bitonic-regs (data/buffer-*.err) on the same seeded input."""
    done = 0
    for rec in golden:
        if rec["family"] != "buffer" or "partial-bitonic-regs" not in rec["algorithms"]:
            continue
        if (rec["n"], rec["q"]) != (1 << 18, 4096) or rec["preprocessor"] != "descending" or rec["k"] not in (32, 512):
            continue
        p = run("-a", "partial-bitonic-regs", "-n", "256k", "-q", "4k", "-k", str(rec["k"]), "--seed", "24",
                "-p", "descending", "--block-size", "256")
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (rec["k"], checksums(p))
        done += 1
    assert done == 2


@pytest.mark.gpu
def test_golden_fused_checksums_end_to_end(golden):
    done = 0
    for rec in golden:
        if rec["family"] != "fused" or (rec["n"], rec["q"]) != (131072, 8192) or rec["k"] not in (16, 32):
            continue
        p = run("-a", "fused-cache", "-n", "128k", "-q", "8k", "-d", str(rec["d"]), "-k", str(rec["k"]),
                "--seed", "24", "--items-per-thread", "8,4,2", "--block-size", "1", "--deg", "1")
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (rec, checksums(p))
        done += 1
    assert done == 6


@pytest.mark.gpu
@pytest.mark.parametrize("algorithm", ["fused-cache-bf16x3", "fused-cache-mfma"])
def test_golden_fused_checksums_with_the_other_arithmetics(golden, algorithm):
    """The reference's own checksums for d = 16 (the dimension of its fused runs that takes the
    bf16 pieces), reproduced with the other arithmetics of the products."""
    done = 0
    for rec in golden:
        if rec["family"] != "fused" or rec["d"] != 16 or (rec["n"], rec["q"]) != (131072, 8192) or rec["k"] not in (16, 32):
            continue
        p = run("-a", algorithm, "-n", "128k", "-q", "8k", "-d", "16", "-k", str(rec["k"]),
                "--seed", "24", "--items-per-thread", "8,4,2", "--block-size", "1", "--deg", "1")
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (rec, checksums(p))
        done += 1
    assert done == 2


@pytest.mark.gpu
def test_fused_launch_parameters_from_the_environment(golden):
    """BITSKNN_FUSED_TUNING hands the driver's fused run the launch parameters a tuning sweep varies;
    the checksum of the reference's run must come out whatever they are, and the reference's own
    parameters are still validated."""
    import os
    rec = next(r for r in golden if r["family"] == "fused" and (r["n"], r["q"], r["d"], r["k"]) == (131072, 8192, 8, 64))
    args = ("-a", "fused-cache", "-n", "128k", "-q", "8k", "-d", "8", "-k", "64", "--seed", "24",
            "--items-per-thread", "8,4,2", "--block-size", "1", "--deg", "1")
    for tuning in ("ranges=1,first_radius=-1", "ranges=16,first_radius=64", "ranges=0,first_radius=0",
                   "ranges=4,first_radius=0,image=1", "ranges=0,first_radius=0,image=-1"):
        p = run(*args, env=dict(os.environ, BITSKNN_FUSED_TUNING=tuning))
        assert p.returncode == 0, p.stderr
        assert str(checksums(p)[0]) in rec["checksums"], (tuning, checksums(p))
    p = run(*args[:-6], "--items-per-thread", "3,4,2", "--block-size", "1", "--deg", "1",
            env=dict(os.environ, BITSKNN_FUSED_TUNING="ranges=2,first_radius=-1"))
    assert p.returncode != 0 and "Unsupported queries_reg value: 3" in p.stderr
    p = run(*args, env=dict(os.environ, BITSKNN_FUSED_TUNING="ranges=99,first_radius=0"))
    assert p.returncode != 0 and "ranges must be" in p.stderr
    p = run(*args, env=dict(os.environ, BITSKNN_FUSED_TUNING="ranges=0,first_radius=0,image=3"))
    assert p.returncode != 0 and "image must be" in p.stderr


@pytest.mark.gpu
def test_algorithms_agree_and_verify_is_silent():
    base = ("-n", "32k", "-q", "64", "-d", "4", "-k", "16", "--seed", "7")
    sums = {}
    # verify() compares within its tolerance, so a result is checked against a reference that
    # reports the same kind of distance: full squared L2 (serial, bits) or ||p||^2 - 2 q.p
    # (parallel, fused-cache)
    for alg, extra, against in (("serial", (), "serial"), ("parallel", (), "parallel"),
                                ("bits", ("--items-per-thread", "4"), "serial"),
                                ("bits-sq", ("--deg", "4", "--items-per-thread", "4"), "serial"),
                                ("fused-cache", ("--items-per-thread", "8,4,2", "--block-size", "1"), "parallel")):
        p = run("-a", alg, *base, *extra, "-v", against)
        assert p.returncode == 0, (alg, p.stderr)
        assert "Difference" not in p.stderr, (alg, p.stderr[:2000])
        sums[alg] = checksums(p)[0]
    assert len(set(sums.values())) == 1, sums


@pytest.mark.gpu
@pytest.mark.parametrize("d", [72, 128, 300])
def test_fused_cache_in_wide_dimensions_agrees_with_the_cpu_path(d):
    """65 to 128 dimensions take the reference's arithmetic in the fused kernel too, and so does the
    plain kernel of more than 256: the driver's run verifies against the CPU path and gives the same
    checksum of labels."""
    base = ("-n", "32k", "-q", "300", "-d", str(d), "-k", "16", "--seed", "11")
    cpu = run("-a", "parallel", *base)
    assert cpu.returncode == 0, cpu.stderr
    gpu = run("-a", "fused-cache", *base, "--items-per-thread", "8,4,2", "--block-size", "1", "-v", "parallel")
    assert gpu.returncode == 0, gpu.stderr
    assert "Difference" not in gpu.stderr, gpu.stderr[:2000]
    assert checksums(gpu)[0] == checksums(cpu)[0]


@pytest.mark.gpu
def test_layouts_and_distance_runners():
    for alg in ("magma-dist", "magma-part-dist", "cublas-dist"):
        p = run("-a", alg, "-n", "8k", "-q", "128", "-d", "16", "-k", "4", "--seed", "5",
                "--point-layout", "column", "--query-layout", "column", "-r", "2")
        assert p.returncode == 0, (alg, p.stderr)
        assert len(p.stdout.strip().splitlines()) == 14
    a = run("-a", "bits", "-n", "8k", "-q", "8", "-d", "3", "-k", "16", "--seed", "5")
    b = run("-a", "bits", "-n", "8k", "-q", "8", "-d", "3", "-k", "16", "--seed", "5",
            "--point-layout", "column", "--query-layout", "column")
    assert checksums(a) == checksums(b)


@pytest.mark.gpu
@pytest.mark.parametrize("args,msg", [
    (("-a", "bits", "--block-size", "100"), "Unsupported block size: 100"),
    (("-a", "bits", "--items-per-thread", "17"), "Unsupported batch size: 17"),
    (("-a", "bits", "-k", "4096", "-n", "8k"), "Unsupported k value: 4096"),
    (("-a", "fused-cache", "-k", "5", "--items-per-thread", "8,4,2", "--block-size", "1"), "Unsupported k value: 5"),
    (("-a", "fused-cache", "-k", "4", "--items-per-thread", "8,4,2", "--block-size", "4", "--deg", "2"),
     "Dimension of vectors must not be lower than 4, but is 1"),
])
def test_unsupported_parameters_exit_with_the_reference_messages(args, msg):
    p = run(*args, "-q", "4", "--seed", "3")
    assert p.returncode == 1 and msg in p.stderr


@pytest.mark.gpu
def test_no_output_skips_checksum():
    p = run("-a", "bits", "-n", "8k", "-q", "8", "-k", "16", "--seed", "5", "--no-output", "--items-per-thread", "4")
    assert p.returncode == 0 and checksums(p) == []
