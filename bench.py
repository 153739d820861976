#!/usr/bin/env python3
"""Benchmark of the k-NN hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only LEG,...] [--skip LEG,...]
                    [--k 32] [--block-size 256] [--items-per-thread 8] [--prefetch]
                    [--fused-d D] [--fused-k K] [--fused-workspace-only] [--no-verify]

A step is one bits top-k pass (through the C ABI) over a resident 1024 x 1,048,576 fp32 matrix
of i.i.d. uniform [0,1) values (4 GiB, generated on the device).  The printed JSON line follows
the reference's throughput convention: elements/s = rows*cols / mean step time
(reference scripts/plot-kselection.py:161).  `roofline` prices the top-k kernel against HBM
bandwidth with its algorithmic bytes (4 B read per matrix element + 8 B written per output pair)
over the kernel's mean duration measured with events on the launch stream.

The same line carries the other workloads of the path, each leg with the fraction of the roofline
that bounds it (`frac`) and `verified`: after a leg's timed launches a sample of its rows or
queries is compared with the CPU oracle (top-k: values and labels bit for bit; distances: k-th
neighbour distance within 1e-5 of the scale of its terms and recall >= 0.999), so that a launch
which did not do its work cannot produce a figure.

  headline     the step described above (`value`, `roofline`)
  calibration  a plain streaming read of the same matrix with the same row-per-workgroup mapping
               (the read rate this machine reaches) and 1 GiB device copies (known traffic for
               scaling byte counters read under a profiler)
  sweep        the 4 GiB matrix at k in {16,32,128,512,2048} x block size {128,256,512} with 2048
               values of a row in flight per iteration (16 / 8 / 4 values per thread) and with the
               larger batches 256 and 512 threads can take, plus the configuration the shipped
               optima file names for each k
  hard         16,384 x 65,536 rows sorted ascending / descending / drawn from 256 values, k = 32, 256,
               with one fixed configuration and with the one the optima file names
  sq           bits-sq: 64 and 256 rows of 524,288 values, every row cut into parts (k = 16, 64)
  gemm         ||p||^2 - 2 q.p on fp32 MFMA for 1,048,576 points x 4,096 queries, d = 64 (a 16 GiB
               matrix), then bits top-k (k = 64) on it
  fused        bits-fused, 1,048,576 points x 65,536 queries, d in {8,16,32} x k in {4,16,32}, through
               the plain entry points: distances in the reference's arithmetic for the pairs that
               pass a filter on the bf16 matrix instructions.  Priced against the bf16 matrix peak
               with the matrix flops the filter executes, with the algorithmic 2*q*n*d flops over the
               fp32 matrix peak beside it; `fused` itself is the d = 32, k = 32 case (queries/s, also
               with every distance from the fp32 matrix instructions and from bf16x3 products),
               `fused.grid` the nine cases; `fused.long_lists` the same shape at k in {64,128,256};
               `fused.few_queries` the reference's own fused shape (8192 queries, 131,072 points,
               d = 8) through the entry point that cuts the points into ranges
  cpu          `cpu_baseline`: the CPU restatement of the reference's parallel top-k (reference
               src/topk/parallel_knn.cpp:30-65) on the host cores and of its serial top-k
               (src/topk/serial_knn.cpp:35-43) on one core, on a 1024 x 65,536 matrix
"""
import argparse
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "bits-knn-jpdc2024_amd")
sys.path.insert(0, ROOT)
sys.path.insert(0, PKG)

HBM_PEAK_GBS = 8000.0       # MI355X published peak
MFMA_F32_PEAK_TFLOPS = 157.3  # dense fp32 matrix peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 matrix peak
LEGS = ("headline", "calibration", "sweep", "hard", "sq", "gemm", "fused", "cpu")
# values per thread in the block-size sweep: the same 2048 values of a row in flight per iteration
# whatever the workgroup size (fewer waves per row need more loads each), and the larger batches
# that long lists need where few rows fit a compute unit
SWEEP_ITEMS = {128: (16,), 256: (8, 16), 512: (4, 8, 16)}
REL = 1e-5
MIN_RECALL = 0.999

# the sources the top-k kernel is built from; the profiled traffic figure is only quoted while
# they are the ones that were profiled
TOPK_SOURCES = ("csrc/topk_bits_kernel.hpp", "csrc/bitonic_net.hpp", "csrc/common.hpp",
                "csrc/topk_bits_inst.hip", "csrc/topk_bits.hip")
TOPK_PROFILE = os.path.join(ROOT, "profiles", "bits_topk_1024x1048576_k32.md")


def topk_sources_sha256():
    digest = hashlib.sha256()
    for name in TOPK_SOURCES:
        with open(os.path.join(PKG, name), "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()


def profiled_traffic(rows, cols, k):
    """HBM bytes per launch of the headline kernel from the two counter passes recorded in the
    profile summary, or None when the summary is for another workload or for other kernel sources
    than the ones in the tree (the figure cannot be taken live: counters need a profiler)."""
    try:
        with open(TOPK_PROFILE) as handle:
            text = handle.read()
    except OSError:
        return None
    fields = dict(re.findall(r"^(\w+) = (\S+)$", text, flags=re.M))
    if (fields.get("workload") != f"{rows}x{cols}_k{k}" or
            fields.get("kernel_sources_sha256") != topk_sources_sha256()):
        return None
    return int(fields["traffic_bytes_per_launch"])


class Timer:
    """Mean duration of launches on the current stream, from events around every launch."""

    def __init__(self, torch):
        self.torch = torch

    def run(self, fn, steps, warmup):
        torch = self.torch
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        t0 = time.perf_counter()
        for i in range(steps):
            starts[i].record()
            fn()
            ends[i].record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        kernel_ms = sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / steps
        return wall / steps, kernel_ms / 1e3


def sample_indices(count, samples):
    step = max(1, count // samples)
    return list(range(step // 2, count, step))[:samples]


def verify_topk(oracle, cache, matrix, sample, k, out_d, out_l):
    """Bit-exact comparison of the sampled rows with the oracle's top-k of the same rows."""
    import numpy as np
    key = (id(matrix), k)
    if key not in cache:
        host = cache.setdefault((id(matrix), "rows"), matrix[sample].cpu().numpy())
        cache[key] = oracle.topk(host, k)
    exp_d, exp_l = cache[key]
    got_d = out_d[sample].cpu().numpy()
    got_l = out_l[sample].cpu().numpy()
    return bool(np.array_equal(got_d.view(np.uint32), exp_d.view(np.uint32)) and np.array_equal(got_l, exp_l))


RESOLUTION = 2.0 ** -20  # of the scale of the cancelling terms: 16 units in the last place


def verify_neighbours(np, points, queries, exp_d, exp_l, got_d, got_l, k):
    """The bar of the parity tests on the sampled queries: recall >= MIN_RECALL against the oracle's
    lists of partial distances (a reported point outside the oracle's list counts when its exact
    distance is within the tolerance of the k-th distance: neighbours closer together than fp32
    resolves), ascending lists, and the k-th neighbour distance within REL -- of the scale of its
    terms (|value| + ||q||^2) always; of the completed distance value + ||q||^2 from 16 dimensions
    on; below that of the reported value itself, except for queries whose error is within
    RESOLUTION of the scale (the value is a small difference of its terms there).  Every error is
    reported uncapped, with the number of queries that took the exception."""
    dim = queries.shape[1]
    qn = (queries.astype(np.float64) ** 2).sum(1)
    kth_e = exp_d[:, k - 1].astype(np.float64)
    kth_g = got_d[:, k - 1].astype(np.float64)
    scale = np.abs(kth_e) + qn
    diff = np.abs(kth_g - kth_e)
    of_scale = diff / scale
    completed = diff / np.maximum(kth_e + qn, 1e-30)
    of_value = np.where(diff == 0, 0.0, diff / np.maximum(np.abs(kth_e), 1e-300))
    excused = (diff != 0) & (of_scale <= RESOLUTION) & (of_value > REL)
    hits = 0
    for row in range(queries.shape[0]):
        want = set(exp_l[row].tolist())
        for label in got_l[row].tolist():
            if label in want:
                hits += 1
                continue
            p = points[label].astype(np.float64)
            exact = float((p * p).sum() - 2.0 * (p * queries[row].astype(np.float64)).sum())
            hits += exact <= kth_e[row] + REL * scale[row]
    recall = hits / (queries.shape[0] * k)
    ascending = bool(np.all(got_d[:, 1:] >= got_d[:, :-1]))
    value_ok = bool(np.all(completed <= REL)) if dim >= 16 else bool(np.all((of_value <= REL) | excused))
    ok = bool(np.all(of_scale <= REL)) and value_ok and recall >= MIN_RECALL and ascending
    bit_exact = bool(np.array_equal(got_d.view(np.uint32), exp_d.view(np.uint32)) and np.array_equal(got_l, exp_l))
    return ok, {"bit_exact_values_and_labels": bit_exact,
                "kth_err_of_scale": float(of_scale.max()), "kth_err_of_completed_distance": float(completed.max()),
                "kth_err_of_value": float(of_value.max()), "queries": int(queries.shape[0]),
                "queries_excused_below_resolution": int(excused.sum()), "recall": recall}


def leg_calibration(bitsknn, torch, timer, matrix, steps):
    rows, cols = matrix.shape
    out = torch.empty(rows, dtype=torch.float32, device=matrix.device)
    _, seconds = timer.run(lambda: bitsknn.stream_read(matrix, out), steps, 3)
    verified = bool(torch.equal(out, matrix.min(dim=1).values))
    gbs = 4.0 * rows * cols / seconds / 1e9
    src = torch.empty(1 << 28, dtype=torch.float32, device=matrix.device).fill_(1.0)
    dst = torch.empty_like(src)
    _, copy_s = timer.run(lambda: dst.copy_(src), 3, 1)
    return {"streaming_read": {"workload": f"row minima of the {rows}x{cols} matrix, 256 threads per row, "
                                           "two 16-byte non-temporal loads in flight per thread",
                               "GBps": gbs, "frac": gbs / HBM_PEAK_GBS, "ms": seconds * 1e3, "verified": verified},
            "device_copy": {"bytes_read_per_copy": 1 << 30, "bytes_written_per_copy": 1 << 30, "copies": 4,
                            "GBps_read_plus_written": 2.0 * (1 << 30) / copy_s / 1e9}}


def leg_sweep(bitsknn, torch, timer, oracle, matrix, steps, check):
    from bitsknn import tuning
    rows, cols = matrix.shape
    cache = {}
    sample = sample_indices(rows, 8)
    out = []
    for k in (16, 32, 128, 512, 2048):
        out_d = torch.empty((rows, k), dtype=torch.float32, device=matrix.device)
        out_l = torch.empty((rows, k), dtype=torch.int32, device=matrix.device)
        tuned_block, _, tuned_batch, _, _ = tuning.config_algorithm("bits", rows, k)
        cases = [(block, items, False) for block in (128, 256, 512) if k // block <= 16
                 for items in SWEEP_ITEMS[block]]
        cases.append((tuned_block, tuned_batch, True))
        for block, items, tuned in cases:
            out_d.fill_(-1.0)
            s, ks = timer.run(lambda: bitsknn.topk_bits(matrix, k, block, items, out_dist=out_d, out_label=out_l),
                              steps, 3)
            entry = {"k": k, "block": block, "items_per_thread": items, "elements_per_s": rows * cols / s,
                     "kernel_ms": ks * 1e3, "frac": (4.0 * rows * cols + 8.0 * rows * k) / ks / 1e9 / HBM_PEAK_GBS}
            if tuned:
                entry["tuned"] = True
            if check:
                entry["verified"] = verify_topk(oracle, cache, matrix, sample, k, out_d, out_l)
            out.append(entry)
    return out


# workgroup size and values per thread of the hard-input leg: the best single choice over its six cases
HARD_CONFIG = (128, 16)


def leg_hard(bitsknn, torch, timer, oracle, dev, steps, check, rows=16384, cols=65536):
    """Config 3: rows sorted ascending, descending, or drawn from 256 distinct values."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(24)
    base = torch.rand((rows, cols), device=dev, generator=gen)
    asc = torch.sort(base, dim=1).values
    inputs = {"ascending": asc, "descending": torch.flip(asc, dims=[1]).contiguous(),
              "256-values": torch.floor(base * 256) / 256}
    del base
    from bitsknn import tuning
    sample = sample_indices(rows, 32)
    out = []
    for name, matrix in inputs.items():
        cache = {}
        for k in (32, 256):
            out_d = torch.full((rows, k), -1.0, dtype=torch.float32, device=dev)
            out_l = torch.empty((rows, k), dtype=torch.int32, device=dev)
            tuned_block, _, tuned_items, _, _ = tuning.config_algorithm("bits", rows, k)
            for block, items, tuned in (HARD_CONFIG + (False,), (tuned_block, tuned_items, True)):
                out_d.fill_(-1.0)
                _, ks = timer.run(lambda: bitsknn.topk_bits(matrix, k, block, items, out_dist=out_d, out_label=out_l),
                                  steps, 2)
                entry = {"rows": name, "k": k, "block": block, "items_per_thread": items,
                         "elements_per_s": rows * cols / ks, "kernel_ms": ks * 1e3,
                         "frac": (4.0 * rows * cols + 8.0 * rows * k) / ks / 1e9 / HBM_PEAK_GBS}
                if tuned:
                    entry["tuned"] = True
                if check:
                    entry["verified"] = verify_topk(oracle, cache, matrix, sample, k, out_d, out_l)
                out.append(entry)
    return out


def leg_sq(bitsknn, torch, timer, oracle, dev, steps, check, cols=1 << 19):
    """bits-sq: few long rows (64 and 256 rows of 2^19 values), every row cut into the parts the
    optima file names, through bitsknn_topk_bits_parts_f32; against the HBM roofline with the bytes
    of the rows."""
    from bitsknn import tuning
    gen = torch.Generator(device=dev)
    gen.manual_seed(24)
    matrix = torch.rand((256, cols), device=dev, generator=gen)
    out = []
    for rows in (64, 256):
        part = matrix[:rows]
        sample = sample_indices(rows, 8)
        cache = {}
        for k in (16, 64):
            block, parts, items, _, _ = tuning.config_algorithm("bits-sq", rows, k)
            scratch = {}
            out_d = torch.full((rows, k), -1.0, dtype=torch.float32, device=dev)
            out_l = torch.empty((rows, k), dtype=torch.int32, device=dev)
            _, seconds = timer.run(lambda: bitsknn.topk_bits_parts(part, k, parts, block, items, scratch=scratch,
                                                                   out_dist=out_d, out_label=out_l), max(steps, 20), 5)
            entry = {"rows": rows, "cols": cols, "k": k, "parts": parts, "block": block, "items_per_thread": items,
                     "us": seconds * 1e6, "elements_per_s": rows * cols / seconds,
                     "frac": (4.0 * rows * cols + 8.0 * rows * k) / seconds / 1e9 / HBM_PEAK_GBS}
            if check:
                entry["verified"] = verify_topk(oracle, cache, part, sample, k, out_d, out_l)
            out.append(entry)
    return out


def leg_gemm(bitsknn, torch, timer, oracle, dev, steps, check, q=4096, n=1 << 20, d=64, k=64):
    """Config 4: ||p||^2 - 2 q.p on MFMA into a q x n matrix (16 GiB), then bits top-k on it."""
    import numpy as np
    gen = torch.Generator(device=dev)
    gen.manual_seed(24)
    points = torch.rand((d, n), device=dev, generator=gen)
    queries = torch.rand((d, q), device=dev, generator=gen)
    dist = torch.empty((q, n), dtype=torch.float32, device=dev)
    out_d = torch.full((q, k), -1.0, dtype=torch.float32, device=dev)
    out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
    _, t_split = timer.run(lambda: bitsknn.distances(queries, points, bitsknn.DIST_PARTIAL_L2_BF16X3, out=dist),
                           steps, 2)
    dist.fill_(-1.0)
    _, t_dist = timer.run(lambda: bitsknn.distances(queries, points, bitsknn.DIST_PARTIAL_L2, out=dist), steps, 2)
    _, t_topk = timer.run(lambda: bitsknn.topk_bits(dist, k, 256, 8, out_dist=out_d, out_label=out_l), steps, 2)
    dist_rows = dist[sample_indices(q, 16)].clone()  # what the checks below look at
    tflops = 2.0 * q * n * d / t_dist / 1e12
    bytes_dist = 4.0 * q * n + 4.0 * (q + n) * d
    result = {"workload": f"GEMM distance + bits, {n} points x {q} queries, d={d}, k={k}",
              "distance_ms": t_dist * 1e3, "pairs_per_s": q * n / t_dist,
              "frac": tflops / MFMA_F32_PEAK_TFLOPS,
              "distance_roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_F32_PEAK_TFLOPS,
                                    "unit": "TFLOP/s", "frac": tflops / MFMA_F32_PEAK_TFLOPS,
                                    "store_GBps": 4.0 * q * n / t_dist / 1e9,
                                    "hbm_frac": bytes_dist / t_dist / 1e9 / HBM_PEAK_GBS},
              "distance_bf16x3": {"arithmetic": "three bf16 pieces per fp32 operand, six bf16 matrix products per "
                                                "product, fp32 accumulation",
                                  "ms": t_split * 1e3, "pairs_per_s": q * n / t_split,
                                  "roofline": {"bound": "hbm", "achieved": bytes_dist / t_split / 1e9,
                                               "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                               "frac": bytes_dist / t_split / 1e9 / HBM_PEAK_GBS}},
              "selection_ms": t_topk * 1e3, "selection_elements_per_s": q * n / t_topk,
              "selection_frac": (4.0 * q * n + 8.0 * q * k) / t_topk / 1e9 / HBM_PEAK_GBS}
    result["end_to_end_ms"] = (t_dist + t_topk) * 1e3
    result["end_to_end_bf16x3_ms"] = (t_split + t_topk) * 1e3
    # the same problem without the matrix: bits-fused through the entry point that cuts the points
    # into ranges (4096 queries are 32 workgroups of 128 queries)
    del dist
    torch.cuda.empty_cache()
    space = torch.empty(max(1, bitsknn.fused_workspace_bytes(q, n, k)), dtype=torch.uint8, device=dev)
    alt_d = torch.full((q, k), -1.0, dtype=torch.float32, device=dev)
    alt_l = torch.empty((q, k), dtype=torch.int32, device=dev)
    _, t_fused = timer.run(lambda: bitsknn.fused_l2_topk(queries, points, k, out_dist=alt_d, out_label=alt_l,
                                                         workspace=space), steps, 2)
    result["fused_alternative"] = {
        "workload": f"bits-fused over ranges of points (workspace of {space.numel()} bytes), same {n} points x "
                    f"{q} queries, d={d}, k={k}; no distance matrix",
        "ms": t_fused * 1e3, "queries_per_s": q / t_fused, "roofline": fused_roofline(q, n, d, t_fused)}
    if check:
        sample = sample_indices(q, 16)
        points_h = np.ascontiguousarray(points.cpu().numpy().T)
        queries_h = np.ascontiguousarray(queries[:, sample].cpu().numpy().T)
        part = oracle.dist(queries_h, points_h, "partial")
        got_rows = dist_rows.cpu().numpy()
        qn = (queries_h.astype(np.float64) ** 2).sum(1)[:, None]
        matrix_err = float(np.max(np.abs(got_rows.astype(np.float64) - part) / (np.abs(part) + qn)))
        # the selection is exact on the matrix it was given ...
        sel_d, sel_l = oracle.topk(got_rows, k)
        got_d = out_d[sample].cpu().numpy()
        got_l = out_l[sample].cpu().numpy()
        exact = bool(np.array_equal(got_d.view(np.uint32), sel_d.view(np.uint32)) and np.array_equal(got_l, sel_l))
        # ... and the neighbours are the reference arithmetic's
        exp_d, exp_l = oracle.topk(part, k)
        ok, detail = verify_neighbours(np, points_h, queries_h, exp_d, exp_l, got_d, got_l, k)
        detail["matrix_err_of_scale"] = matrix_err
        detail["selection_bit_exact_on_the_matrix"] = exact
        result["verified"] = bool(ok and exact and matrix_err <= REL)
        result["verification"] = detail
        ok_alt, detail_alt = verify_neighbours(np, points_h, queries_h, exp_d, exp_l, alt_d[sample].cpu().numpy(),
                                               alt_l[sample].cpu().numpy(), k)
        result["fused_alternative"]["verified"] = bool(ok_alt and detail_alt["bit_exact_values_and_labels"])
        result["fused_alternative"]["verification"] = detail_alt
    return result


def filter_flops_per_pair(d):
    """bf16 matrix flops the default fused kernel executes per (query, point) pair: matrix
    instructions of 32 x 32 x 16, two per tile up to 8 dimensions, else three per 16 dimensions
    (two pieces per operand, the smallest product left out) and one for the norm; 65 .. 128
    dimensions are padded to 128 and take two for the norm (sixteen shares of it)"""
    if d > 64:
        return (3 * 8 + 2) * 32.0
    terms = 2 if d <= 8 else 3 * ((d + 15) // 16) + 1
    return terms * 32.0


def fused_roofline(q, n, d, seconds):
    """The default fused kernel against the matrix unit it runs on: the bf16 matrix instructions of
    its filter (executed flops, padding included) against the bf16 peak; next to it the
    algorithmic 2*q*n*d flops of the distance over the time, and what fraction of the fp32 matrix
    peak that is (above 1: the contraction does not run on the fp32 unit)."""
    algorithmic = 2.0 * q * n * d / seconds / 1e12
    if d > 128:
        # 129 .. 256 dimensions: the filter runs on the fp32 matrix instructions (256 dimensions and
        # four norm rows per pair); above 256 a vector-unit kernel, priced by its algorithmic flops
        flops = 2.0 * (256 + 4) if d <= 256 else 2.0 * d
        executed = flops * q * n / seconds / 1e12
        return {"bound": "mfma", "achieved": executed, "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": executed / MFMA_F32_PEAK_TFLOPS,
                "matrix_instructions": ("v_mfma_f32_32x32x2_f32, %d flops per pair executed" % flops) if d <= 256
                else "none (vector unit), priced against the fp32 matrix peak",
                "algorithmic_tflops": algorithmic, "algorithmic_over_fp32_matrix_peak": algorithmic / MFMA_F32_PEAK_TFLOPS}
    executed = filter_flops_per_pair(d) * q * n / seconds / 1e12
    return {"bound": "mfma", "achieved": executed, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": executed / MFMA_BF16_PEAK_TFLOPS,
            "matrix_instructions": "v_mfma_f32_32x32x16_bf16, %d flops per pair executed" % filter_flops_per_pair(d),
            "algorithmic_tflops": algorithmic, "algorithmic_over_fp32_matrix_peak": algorithmic / MFMA_F32_PEAK_TFLOPS}


def leg_fused(bitsknn, torch, timer, oracle, dev, steps, check, dims, ks, q=65536, n=1 << 20, long_ks=(),
              workspace=False, plain_too=True):
    """Config 5: bits-fused at d x k in the default arithmetic (the reference's, behind a filter on
    the bf16 matrix instructions) through the workspace entry point, as the knn driver calls it: the
    workspace has room for the stage image, so the points are cut into bf16 pieces once per call
    (that launch is inside the timed call); `ms_plain_entry_point` is the entry point without a
    workspace beside it.  The d = 32, k = 32 case also with the distances from the fp32 matrix
    instructions and from bf16x3 products.  long_ks: list lengths beyond the configuration's,
    reported apart (`long_lists`).  workspace: room for partial lists as well, so that few queries
    search the points in ranges."""
    import numpy as np
    grid = []
    long_lists = []
    headline = None
    sample = sample_indices(q, 64)
    for d in dims:
        gen = torch.Generator(device=dev)
        gen.manual_seed(24 + d)
        points = torch.rand((d, n), device=dev, generator=gen)
        queries = torch.rand((d, q), device=dev, generator=gen)
        part = None
        for k in tuple(ks) + tuple(long_ks):
            out_d = torch.full((q, k), -1.0, dtype=torch.float32, device=dev)
            out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
            lists = bitsknn.fused_workspace_bytes(q, n, k) if workspace else 0
            space = torch.empty(max(1, (lists + 255) // 256 * 256 + bitsknn.fused_image_bytes(d, n)),
                                dtype=torch.uint8, device=dev)
            plain_s = None
            if not workspace and plain_too:
                _, plain_s = timer.run(lambda: bitsknn.fused_l2_topk(queries, points, k, out_dist=out_d,
                                                                     out_label=out_l), steps, 2)
                out_d.fill_(-1.0)
            _, seconds = timer.run(lambda: bitsknn.fused_l2_topk(queries, points, k, out_dist=out_d, out_label=out_l,
                                                                 workspace=space), steps, 2)
            roof = fused_roofline(q, n, d, seconds)
            entry = {"d": d, "k": k, "ms": seconds * 1e3, "queries_per_s": q / seconds,
                     "pairs_per_s": q * n / seconds, "frac": roof["frac"],
                     "algorithmic_over_fp32_matrix_peak": roof["algorithmic_over_fp32_matrix_peak"]}
            if plain_s is not None:
                entry["ms_plain_entry_point"] = plain_s * 1e3
            del space
            if check:
                if part is None:
                    points_h = np.ascontiguousarray(points.cpu().numpy().T)
                    queries_h = np.ascontiguousarray(queries[:, sample].cpu().numpy().T)
                    part = oracle.dist(queries_h, points_h, "partial")
                exp_d, exp_l = oracle.topk(part, k)
                ok, detail = verify_neighbours(np, points_h, queries_h, exp_d, exp_l, out_d[sample].cpu().numpy(),
                                               out_l[sample].cpu().numpy(), k)
                # the default arithmetic is the reference's: nothing but bit for bit counts
                entry["verified"] = bool(ok and detail["bit_exact_values_and_labels"])
                entry["verification"] = detail
            (grid if k in ks else long_lists).append(entry)
            if d == 32 and k == 32 and not workspace:
                headline = {"workload": f"bits-fused, {n} points x {q} queries, d={d}, k={k}, fp32 uniform[0,1)",
                            "arithmetic": "sequential fp32 fused multiply-adds in dimension order (the reference's) "
                                          "for every pair that passes a guaranteed lower bound from bf16 matrix "
                                          "instructions",
                            "entry_point": "bitsknn_fused_l2_topk_f32_ws with room for the stage image in the "
                                           "workspace (one launch that cuts the points, one fused launch)",
                            "launches_timed": steps,
                            "queries_per_s": q / seconds, "ms": seconds * 1e3, "pairs_per_s": q * n / seconds,
                            "roofline": roof}
                if plain_s is not None:
                    headline["ms_plain_entry_point"] = plain_s * 1e3
                if check:
                    headline["verified"] = entry["verified"]
                for name, arithmetic, text, flops_per_pair, peak in (
                        ("mfma_f32", bitsknn.FUSED_FP32, "every distance from fp32 matrix instructions", 2.0 * d,
                         MFMA_F32_PEAK_TFLOPS),
                        ("bf16x3", bitsknn.FUSED_BF16X3, "three bf16 pieces per fp32 operand, six bf16 matrix products "
                         "per product, fp32 accumulation", 12.0 * d, MFMA_BF16_PEAK_TFLOPS)):
                    out_d.fill_(-1.0)
                    _, other_s = timer.run(
                        lambda: bitsknn.fused_l2_topk(queries, points, k, out_dist=out_d, out_label=out_l,
                                                      arithmetic=arithmetic), steps, 1)
                    tflops = flops_per_pair * q * n / other_s / 1e12
                    headline[name] = {"arithmetic": text, "queries_per_s": q / other_s, "ms": other_s * 1e3,
                                      "pairs_per_s": q * n / other_s,
                                      "roofline": {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s",
                                                   "frac": tflops / peak}}
                    if check:
                        ok, detail = verify_neighbours(np, points_h, queries_h, exp_d, exp_l,
                                                       out_d[sample].cpu().numpy(), out_l[sample].cpu().numpy(), k)
                        headline[name]["verified"] = bool(ok)
        del points, queries
    result = headline if headline is not None else {"workload": f"bits-fused, {n} points x {q} queries"}
    result["grid"] = grid
    if long_lists:
        result["long_lists"] = long_lists
    return result


def cpu_model():
    try:
        with open("/proc/cpuinfo") as handle:
            for line in handle:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def leg_cpu(rows, cols, k, budget_s=8.0):
    """The reference's CPU paths restated in oracle/, on config 1's matrix: the OpenMP heap per row
    on the host cores this job may use, and the full sort of every row on one core."""
    from oracle import binding as oracle
    m = oracle.uniform_matrix(24, rows, cols)
    # the cores this job may use: the OpenMP setting of the environment when there is one (a GPU
    # box hands a job a share of its cores), else every core of the host
    threads = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
    reps, spent = 0, 0.0
    oracle.topk_parallel(m, k, threads)  # warm
    while spent < budget_s and reps < 50:
        t0 = time.perf_counter()
        _, _, used = oracle.topk_parallel(m, k, threads)
        spent += time.perf_counter() - t0
        reps += 1
    t0 = time.perf_counter()
    oracle.topk_serial(m, k)
    serial_s = time.perf_counter() - t0
    return {"value": rows * cols * reps / spent, "unit": "elements/s", "cores": used, "kind": "port",
            "sample": f"{reps} passes of parallel_knn::selection restated (OpenMP heap) over a "
                      f"{rows}x{cols} fp32 uniform matrix, k={k} (the GPU figure is for {rows}x1048576)",
            "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
            "serial": {"value": rows * cols / serial_s, "unit": "elements/s", "cores": 1,
                       "sample": f"one pass of serial_knn::selection restated (std::sort of every row) over "
                                 f"the same {rows}x{cols} matrix"}}


def collect_verified(node, found):
    """every `verified` flag anywhere in the result"""
    if isinstance(node, dict):
        for key, value in node.items():
            if key == "verified":
                found.append(bool(value))
            else:
                collect_verified(value, found)
    elif isinstance(node, list):
        for value in node:
            collect_verified(value, found)
    return found


def summarise(result):
    """The fractions of the roofline of every leg in a few hundred bytes, placed at the end of the
    line: per list length the worst, best and tuned configuration of the sweep, the hard-input
    cases, both kernels of the GEMM k-NN against both roofs, the fused grid, and whether every
    comparison with the oracle passed."""
    r3 = lambda x: round(float(x), 3)
    out = {}
    if "roofline" in result:
        out["headline_frac"] = r3(result["roofline"]["frac"])
    if "sweep" in result:
        by_k = {}
        for entry in result["sweep"]:
            slot = by_k.setdefault(str(entry["k"]), {"min": 1e9, "max": 0.0})
            if entry.get("tuned"):
                slot["tuned"] = r3(entry["frac"])
            else:
                slot["min"] = min(slot["min"], r3(entry["frac"]))
                slot["max"] = max(slot["max"], r3(entry["frac"]))
        out["sweep_frac_hbm_by_k"] = by_k
    if "hard_inputs" in result:
        out["hard_inputs_frac_hbm"] = {
            f"{e['rows']}_k{e['k']}{'_tuned' if e.get('tuned') else ''}": r3(e["frac"]) for e in result["hard_inputs"]}
    if "gemm_knn" in result:
        g = result["gemm_knn"]
        out["gemm_knn"] = {"distance_frac_mfma": r3(g["distance_roofline"]["frac"]),
                           "distance_frac_hbm": r3(g["distance_roofline"]["hbm_frac"]),
                           "distance_bf16x3_frac_hbm": r3(g["distance_bf16x3"]["roofline"]["frac"]),
                           "selection_frac_hbm": r3(g["selection_frac"]),
                           "distance_ms": r3(g["distance_ms"]), "distance_bf16x3_ms": r3(g["distance_bf16x3"]["ms"]),
                           "selection_ms": r3(g["selection_ms"]), "end_to_end_ms": r3(g["end_to_end_ms"]),
                           "fused_alternative_ms": r3(g["fused_alternative"]["ms"]),
                           "fused_alternative_frac_bf16_mfma": r3(g["fused_alternative"]["roofline"]["frac"])}
    if "fused" in result:
        f = result["fused"]
        out["fused_grid_ms"] = {f"d{e['d']}_k{e['k']}": r3(e["ms"]) for e in f.get("grid", [])}
        out["fused_grid_ms_plain_entry_point"] = {f"d{e['d']}_k{e['k']}": r3(e["ms_plain_entry_point"])
                                                  for e in f.get("grid", []) if "ms_plain_entry_point" in e}
        out["fused_grid_frac_bf16_mfma"] = {f"d{e['d']}_k{e['k']}": r3(e["frac"]) for e in f.get("grid", [])}
        out["fused_grid_algorithmic_over_fp32_mfma_peak"] = {
            f"d{e['d']}_k{e['k']}": r3(e["algorithmic_over_fp32_matrix_peak"]) for e in f.get("grid", [])}
        if "long_lists" in f:
            out["fused_long_lists_ms"] = {f"d{e['d']}_k{e['k']}": r3(e["ms"]) for e in f["long_lists"]}
        if "queries_per_s" in f:
            out["fused_d32_k32"] = {"queries_per_s": round(f["queries_per_s"]), "ms": r3(f["ms"]),
                                    "frac_bf16_mfma": r3(f["roofline"]["frac"]),
                                    "algorithmic_over_fp32_mfma_peak": r3(f["roofline"]["algorithmic_over_fp32_matrix_peak"]),
                                    "launches_timed": f.get("launches_timed")}
            for name in ("mfma_f32", "bf16x3"):
                if name in f:
                    out["fused_d32_k32"][name + "_queries_per_s"] = round(f[name]["queries_per_s"])
                    out["fused_d32_k32"][name + "_frac"] = r3(f[name]["roofline"]["frac"])
        if "few_queries" in f:
            out["fused_few_queries_ms"] = {f"d{e['d']}_k{e['k']}": r3(e["ms"]) for e in f["few_queries"]["cases"]}
    if "bits_sq" in result:
        out["bits_sq_frac_hbm"] = {f"rows{e['rows']}_k{e['k']}": r3(e["frac"]) for e in result["bits_sq"]}
    flags = collect_verified(result, [])
    out["verified_checks"] = len(flags)
    out["all_verified"] = bool(flags) and all(flags)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--k", type=int, default=32)
    ap.add_argument("--block-size", type=int, default=256)
    ap.add_argument("--items-per-thread", type=int, default=8)
    ap.add_argument("--prefetch", action="store_true", help="the bits-prefetch variant")
    ap.add_argument("--rows", type=int, default=1024)
    ap.add_argument("--cols", type=int, default=1 << 20)
    ap.add_argument("--only", default="", help="comma-separated legs to run: " + ", ".join(LEGS))
    ap.add_argument("--skip", default="", help="comma-separated legs to leave out")
    ap.add_argument("--fused-d", type=int, default=0, help="restrict the fused grid to this dimension")
    ap.add_argument("--fused-k", type=int, default=0, help="restrict the fused grid to this list length")
    ap.add_argument("--fused-workspace-only", action="store_true",
                    help="time the fused grid through the workspace entry point only (counter passes)")
    ap.add_argument("--no-verify", action="store_true", help="leave out the comparison with the oracle")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (--gpus 1); multi-GPU figures are not "
              "part of it", file=sys.stderr)
        sys.exit(2)
    legs = set(x for x in args.only.split(",") if x) or set(LEGS)
    legs -= set(x for x in args.skip.split(",") if x)
    unknown = legs - set(LEGS)
    if unknown:
        print(f"bench.py: unknown legs {sorted(unknown)}; known: {', '.join(LEGS)}", file=sys.stderr)
        sys.exit(2)

    import torch
    import bitsknn
    bitsknn.lib()
    check = not args.no_verify
    oracle = None
    if check:
        from oracle import binding as oracle  # the checker of every leg, never the thing measured
        oracle.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    timer = Timer(torch)
    rows, cols = args.rows, args.cols
    few = max(3, args.steps // 4)

    result = {"metric": "bits top-k selected-from elements/s (rows*cols / step time)", "value": None,
              "unit": "elements/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": None,
              "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
              "data": "synthetic",
              "config": {"workload": f"bits top-k, fp32 matrix {rows}x{cols} uniform[0,1) resident in HBM, "
                                     f"k={args.k}, block {args.block_size}, items/thread {args.items_per_thread}, "
                                     f"prefetch {int(args.prefetch)}"}}

    if legs & {"headline", "calibration", "sweep"}:
        gen = torch.Generator(device=dev)
        gen.manual_seed(24)
        matrix = torch.rand((rows, cols), device=dev, generator=gen)
        if "headline" in legs:
            k = args.k
            out_d = torch.full((rows, k), -1.0, dtype=torch.float32, device=dev)
            out_l = torch.empty((rows, k), dtype=torch.int32, device=dev)
            step_s, kernel_s = timer.run(
                lambda: bitsknn.topk_bits(matrix, k, args.block_size, args.items_per_thread, args.prefetch,
                                          out_dist=out_d, out_label=out_l), args.steps, args.warmup)
            bytes_alg = 4.0 * rows * cols + 8.0 * rows * k
            achieved = bytes_alg / kernel_s / 1e9
            result["value"] = rows * cols / step_s
            result["ms_per_step"] = step_s * 1e3
            result["roofline"] = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": achieved / HBM_PEAK_GBS, "traffic": profiled_traffic(rows, cols, k),
                                  "kernel_ms": kernel_s * 1e3, "algorithmic_bytes": bytes_alg}
            if check:
                result["verified"] = verify_topk(oracle, {}, matrix, sample_indices(rows, 8), k, out_d, out_l)
        if "calibration" in legs:
            result["calibration"] = leg_calibration(bitsknn, torch, timer, matrix, few)
        if "sweep" in legs:
            result["sweep"] = leg_sweep(bitsknn, torch, timer, oracle, matrix, few, check)
        del matrix
        torch.cuda.empty_cache()
    if "hard" in legs:
        result["hard_inputs"] = leg_hard(bitsknn, torch, timer, oracle, dev, few, check)
        torch.cuda.empty_cache()
    if "sq" in legs:
        result["bits_sq"] = leg_sq(bitsknn, torch, timer, oracle, dev, few, check)
        torch.cuda.empty_cache()
    if "gemm" in legs:
        result["gemm_knn"] = leg_gemm(bitsknn, torch, timer, oracle, dev, few, check)
        torch.cuda.empty_cache()
    if "fused" in legs:
        dims = (args.fused_d,) if args.fused_d else (8, 16, 32)
        ks = (args.fused_k,) if args.fused_k else (4, 16, 32)
        whole = not args.fused_d and not args.fused_k
        result["fused"] = leg_fused(bitsknn, torch, timer, oracle, dev, max(5, args.steps // 4), check, dims, ks,
                                    long_ks=(64, 128, 256) if whole else (),
                                    plain_too=not args.fused_workspace_only)
        if whole:
            # the reference's own fused shape with few queries (its plots: 8192 queries, 2^17 points):
            # the entry point with a workspace, which cuts the points into ranges
            few = leg_fused(bitsknn, torch, timer, oracle, dev, max(5, args.steps // 4), check, (8,), (32,),
                            q=8192, n=1 << 17, long_ks=(64, 256), workspace=True)
            result["fused"]["few_queries"] = {"workload": few["workload"] + ", points cut into ranges (workspace)",
                                              "cases": few["grid"] + few["long_lists"]}
        # no wave of any fused launch above gave up a wait for a stage
        try:
            bitsknn.fused_status()
            result["fused"]["kernel_status"] = {"verified": True}
        except bitsknn.BitsKnnError as error:
            result["fused"]["kernel_status"] = {"verified": False, "message": str(error)}
        torch.cuda.empty_cache()
    if "cpu" in legs:
        result["cpu_baseline"] = leg_cpu(1024, 65536, 32)
    result["summary"] = summarise(result)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
