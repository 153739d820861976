"""Launch-parameter tuning for the bits kernels on one MI355X.

Two halves, matching the reference's tuning workflow:

* ``sweep()`` times `bits` and `bits-prefetch` over the grid of the reference's parameter search
  (reference scripts/run-opt-ipt.sh:38-47: n = 512k, q in 64..8192, k in 2..2048, block size
  128/256/512; of its batch sizes 1..16 only 4, 8, 12 and 16, because the kernels load 16 bytes
  per thread at a time and batches that round up to the same number of loads are the same
  kernel), ``sweep_bits_sq()`` times `bits-sq` with every row cut into 2..16 parts for the query
  counts that do not fill the GPU with one row per workgroup, ``sweep_partial_bitonic()`` times
  `partial-bitonic-regs` over the grid of scripts/run-opt-bitonic-sort.sh:27-43 (q*n = 2^30, q in
  64..4096, k in 32..2048, block size 64..512), ``sweep_fused()`` times `fused-cache` (whose
  tuning parameters do not steer the matrix-core kernel: its rows carry the reference's fixed
  choice 8,4,2 / 1 / 1), and ``write_optima()`` keeps the fastest configuration of every
  (algorithm, q, k, dim) in a CSV with the columns of the reference's scripts/optima.csv
  (hostname, GPU, algorithm, point_count, query_count, k, dim, block_size, items_per_thread,
  items_per_thread2, items_per_thread3, deg, time), as scripts/plot-analyze-opt.py does.
* ``config_algorithm()`` is the lookup the reference's run scripts perform on that file
  (reference scripts/config.sh:97-214, ``config_generic`` / ``config_algorithm``): among the rows
  of the algorithm (and host), prefer rows whose query_count / k / dim are not below the request,
  and among those the row with the smallest product of ratios to the request.

    python -m bitsknn.tuning --out optima.csv        # on a GPU box; a few minutes

The timed matrix is generated on the device (uniform [0,1), as `knn -g uniform`); one
8192 x 524288 matrix (16 GiB) serves every query count as a row prefix.
"""
import argparse
import csv
import os
import sys

OPTIMA_COLUMNS = ("hostname", "GPU", "algorithm", "point_count", "query_count", "k", "dim",
                  "block_size", "items_per_thread", "items_per_thread2", "items_per_thread3",
                  "deg", "time")
DEFAULT_OPTIMA = os.path.join(os.path.dirname(os.path.abspath(__file__)), "optima.csv")

QUERY_COUNTS = (64, 256, 512, 1024, 2048, 4096, 8192)
K_VALUES = (2, 4, 8, 16, 32, 64, 128, 256, 512, 1024, 2048)
BLOCK_SIZES = (128, 256, 512)
# Many short rows (the shape of the sorted / tie-heavy benchmark rows) want other launch parameters
# than the long rows of the grid above: a row of 65,536 values is over after a few iterations of 512
# threads.  The lookup is keyed by the query count alone, so these rows serve requests for 16,384
# queries and more.
SHORT_ROWS_QUERY_COUNT = 16384
SHORT_ROWS_POINT_COUNT = 65536
# values per thread and iteration: the kernels issue 16-byte loads, so 1..4, 5..8, 9..12 and 13..16
# are one kernel each; the sweep times the distinct ones
BATCH_SIZES = (4, 8, 12, 16)
ALGORITHMS = (("bits", False), ("bits-prefetch", True))
# bits-sq: parts a row is cut into, for query counts that leave compute units without a row
SQ_QUERY_COUNTS = (64, 256)
SQ_DEGREES = (2, 4, 8, 16, 32)
# fused-cache: (queries, points) shapes of the reference's fused runs (scripts/run-fused.sh) that
# bound the lookup's range, dimensions and list lengths
FUSED_SHAPES = ((1024, 1 << 20), (8192, 1 << 17))
FUSED_DIMS = (8, 16, 32)
FUSED_K_VALUES = (4, 8, 16, 32, 64, 128, 256)


def config_algorithm(algorithm, query_count=None, k=None, dim=None, hostname=None,
                     optima_file=DEFAULT_OPTIMA):
    """(block_size, deg, items_per_thread, items_per_thread2, items_per_thread3) for a problem.

    Restates the awk program of reference scripts/config.sh:103-200.  ``None`` for query_count,
    k, dim or hostname means "do not care" (the script's literal "None").  Without a matching
    row the defaults of the script are returned: (256, 1, 1, 1, 1).  A parameter that no row up
    to the chosen one states comes back as None (an empty word in the script's output, which the
    run scripts replace by their own default).
    """
    names = ("block_size", "deg", "items_per_thread", "items_per_thread2", "items_per_thread3")
    best = {"block_size": 256, "deg": 1, "items_per_thread": 1, "items_per_thread2": 1,
            "items_per_thread3": 1}
    # the script keeps the last non-empty field it saw, row after row; a field it has not seen
    # yet is empty (None here) and stays empty in the answer
    carried = dict.fromkeys(names)
    score, slack = 0, 0.0
    with open(optima_file, newline="") as handle:
        reader = csv.reader(handle)
        header = next(reader, None)
        if header is None or "algorithm" not in header or "hostname" not in header:
            raise ValueError(f"{optima_file}: no algorithm/hostname columns")
        col = {name: i for i, name in enumerate(header)}

        def field(row, name):
            i = col.get(name)
            return row[i] if i is not None and i < len(row) else ""

        for row in reader:
            if field(row, "algorithm") != algorithm:
                continue
            if hostname is not None and field(row, "hostname") != hostname:
                continue
            new_score, new_slack = 0, 1.0
            for name in names:
                text = field(row, name)
                if text != "":
                    carried[name] = int(float(text))
            for name, wanted in (("query_count", query_count), ("k", k), ("dim", dim)):
                text = field(row, name)
                if wanted is None or text == "":
                    continue
                have = float(text)
                if have >= wanted:
                    new_score += 1
                    new_slack *= have / wanted
                else:
                    new_slack *= wanted / have
            if new_score >= score and (slack == 0 or new_slack < slack):
                score, slack = new_score, new_slack
                best = dict(carried)
    return (best["block_size"], best["deg"], best["items_per_thread"], best["items_per_thread2"],
            best["items_per_thread3"])


def sweep(repeats=10, point_count=512 * 1024, query_counts=QUERY_COUNTS, k_values=K_VALUES,
          block_sizes=BLOCK_SIZES, batch_sizes=BATCH_SIZES, algorithms=ALGORITHMS, seed=17,
          progress=None):
    """Time every grid point on cuda:0; yields dict rows (seconds per pass, mean of `repeats`)."""
    import torch
    import bitsknn

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    matrix = torch.rand((max(query_counts), point_count), device=dev, generator=gen)
    for q in query_counts:
        rows = matrix[:q]
        for k in k_values:
            out_d = torch.empty((q, k), dtype=torch.float32, device=dev)
            out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
            for name, prefetch in algorithms:
                for block in block_sizes:
                    for batch in batch_sizes:
                        bitsknn.topk_bits(rows, k, block, batch, prefetch, out_dist=out_d, out_label=out_l)
                        start = torch.cuda.Event(enable_timing=True)
                        end = torch.cuda.Event(enable_timing=True)
                        start.record()
                        for _ in range(repeats):
                            bitsknn.topk_bits(rows, k, block, batch, prefetch, out_dist=out_d,
                                              out_label=out_l)
                        end.record()
                        end.synchronize()
                        yield {"algorithm": name, "point_count": point_count, "query_count": q,
                               "k": k, "dim": 1, "block_size": block, "items_per_thread": batch,
                               "items_per_thread2": 1, "items_per_thread3": 1, "deg": 1,
                               "time": start.elapsed_time(end) / 1e3 / repeats}
            if progress is not None:
                progress(q, k)


def bits_sq(rows, k, deg, block, batch, scratch=None):
    """`bits-sq` through the C ABI (reference src/topk/singlepass/bits_knn.cu:132-186): every row
    is cut into `deg` parts that are selected independently with their labels shifted by the part's
    offset, then the deg*k partial results of a row are selected again with their labels -- in one
    launch (bitsknn_topk_bits_parts_f32)."""
    import bitsknn
    return bitsknn.topk_bits_parts(rows, k, deg, block, batch, scratch=scratch if scratch is not None else {})


def sweep_bits_sq(repeats=10, point_count=512 * 1024, query_counts=SQ_QUERY_COUNTS, k_values=K_VALUES,
                  block_sizes=BLOCK_SIZES, batch_sizes=BATCH_SIZES, degrees=SQ_DEGREES, seed=17,
                  progress=None):
    """Time bits-sq on cuda:0 over the parts per row; yields dict rows like sweep()."""
    import torch

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    matrix = torch.rand((max(query_counts), point_count), device=dev, generator=gen)
    for q in query_counts:
        rows = matrix[:q]
        for k in k_values:
            scratch = {}
            for deg in degrees:
                if k * deg > point_count // deg:
                    continue
                for block in block_sizes:
                    if k > block * 16:
                        continue
                    for batch in batch_sizes:
                        bits_sq(rows, k, deg, block, batch, scratch)
                        start = torch.cuda.Event(enable_timing=True)
                        end = torch.cuda.Event(enable_timing=True)
                        start.record()
                        for _ in range(repeats):
                            bits_sq(rows, k, deg, block, batch, scratch)
                        end.record()
                        end.synchronize()
                        yield {"algorithm": "bits-sq", "point_count": point_count, "query_count": q,
                               "k": k, "dim": 1, "block_size": block, "items_per_thread": batch,
                               "items_per_thread2": 1, "items_per_thread3": 1, "deg": deg,
                               "time": start.elapsed_time(end) / 1e3 / repeats}
            if progress is not None:
                progress(q, k)


def sweep_fused(repeats=3, shapes=FUSED_SHAPES, dims=FUSED_DIMS, k_values=FUSED_K_VALUES, seed=17,
                progress=None):
    """Time fused-cache (with the workspace its entry point asks for) on cuda:0.  The reference's
    parameters do not change the kernel, so there is one row per problem, with the reference's
    fixed choice of them (scripts/optima-fixed-max_slowdown.csv: 8,4,2, block 1, deg 1)."""
    import torch
    import bitsknn

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    for q, n in shapes:
        for dim in dims:
            points = torch.rand((dim, n), device=dev, generator=gen)
            queries = torch.rand((dim, q), device=dev, generator=gen)
            for k in k_values:
                out_d = torch.empty((q, k), dtype=torch.float32, device=dev)
                out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
                workspace = torch.empty(max(1, bitsknn.fused_workspace_bytes(q, n, k)), dtype=torch.uint8,
                                        device=dev)

                def run():
                    bitsknn.fused_l2_topk(queries, points, k, (8, 4, 2), 1, 1, out_dist=out_d, out_label=out_l,
                                          workspace=workspace)
                run()
                start = torch.cuda.Event(enable_timing=True)
                end = torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(repeats):
                    run()
                end.record()
                end.synchronize()
                yield {"algorithm": "fused-cache", "point_count": n, "query_count": q, "k": k, "dim": dim,
                       "block_size": 1, "items_per_thread": 8, "items_per_thread2": 4,
                       "items_per_thread3": 2, "deg": 1, "time": start.elapsed_time(end) / 1e3 / repeats}
            if progress is not None:
                progress(q, dim)


# ---- launch parameters of the fused kernels (bitsknn_fused_tuning) -------------------------------
FUSED_TUNING_COLUMNS = ("hostname", "GPU", "point_count", "query_count", "dim", "k", "arithmetic", "ranges",
                        "first_radius", "image", "workgroup", "time", "time_with_the_librarys_choice")
DEFAULT_FUSED_TUNING = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fused_tuning.csv")
FUSED_TUNING_SHAPES = ((1024, 1 << 20), (8192, 1 << 17), (65536, 1 << 20))
FUSED_RANGES = (1, 2, 4, 8, 16, 32, 64)
FUSED_FIRST_RADII = (-1, 64, 256)
ARITHMETIC_NAMES = {0: "fp32-matrix", 1: "bf16x3", 2: "exact"}


def sweep_fused_tuning(repeats=3, shapes=FUSED_TUNING_SHAPES, dims=FUSED_DIMS, k_values=(4, 16, 32, 64, 128, 256),
                       arithmetics=(2, 0), seed=17, progress=None):
    """Time bits-fused on cuda:0 over what bitsknn_fused_l2_topk_f32_tuned lets a caller choose: the
    number of ranges the points are cut into, whether (and how densely) a sample of the points
    gives the first radii, and (exact arithmetic) whether the points are cut into stages once per
    call and whether a workgroup has 128 or 256 queries, per arithmetic.  The counterpart of the reference's sweep over the register tiling of its
    fused kernel (scripts/run-fused-cache-params.sh).  Yields one dict per measurement; `ranges` 0,
    `first_radius` 0, `image` 0 and `workgroup` 0 are the library's own choice."""
    import torch
    import bitsknn

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    for q, n in shapes:
        for dim in dims:
            points = torch.rand((dim, n), device=dev, generator=gen)
            queries = torch.rand((dim, q), device=dev, generator=gen)
            for k in k_values:
                out_d = torch.empty((q, k), dtype=torch.float32, device=dev)
                out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
                lists = (8 * q * 64 * k + 255) // 256 * 256
                workspace = torch.empty(lists + bitsknn.fused_image_bytes(dim, n), dtype=torch.uint8, device=dev)
                for arithmetic in arithmetics:
                    choices = [(0, 0, 0, 0)]
                    for ranges in FUSED_RANGES:
                        # more workgroups than eight per compute unit gain nothing
                        if ranges > 1 and (q // 128) * ranges > 2048:
                            continue
                        for first_radius in FUSED_FIRST_RADII:
                            for image in ((-1, 1) if arithmetic == 2 else (-1,)):
                                choices.append((ranges, first_radius, image, 128))
                            # (workgroups of 256 queries take no stage image)
                            if arithmetic == 2 and dim <= 64 and (k <= 32 or (dim <= 8 and k <= 128)):
                                choices.append((ranges, first_radius, -1, 256))
                    for ranges, first_radius, image, workgroup in choices:
                        def run():
                            bitsknn.fused_l2_topk(queries, points, k, out_dist=out_d, out_label=out_l,
                                                  workspace=workspace, arithmetic=arithmetic,
                                                  tuning=(ranges, first_radius, image, workgroup))
                        run()
                        start = torch.cuda.Event(enable_timing=True)
                        end = torch.cuda.Event(enable_timing=True)
                        start.record()
                        for _ in range(repeats):
                            run()
                        end.record()
                        end.synchronize()
                        yield {"point_count": n, "query_count": q, "dim": dim, "k": k,
                               "arithmetic": ARITHMETIC_NAMES[arithmetic], "ranges": ranges,
                               "first_radius": first_radius, "image": image, "workgroup": workgroup,
                               "time": start.elapsed_time(end) / 1e3 / repeats}
            if progress is not None:
                progress(q, dim)
    bitsknn.fused_status()


def fused_optima(rows):
    """The fastest (ranges, first_radius, image, workgroup) per problem and arithmetic, with the time
    of the library's own choice beside it."""
    best = {}
    own = {}
    for row in rows:
        key = (row["point_count"], row["query_count"], row["dim"], row["k"], row["arithmetic"])
        if row["ranges"] == 0 and row["first_radius"] == 0 and row.get("image", 0) == 0 and row.get("workgroup", 0) == 0:
            own[key] = row["time"]
        elif key not in best or row["time"] < best[key]["time"]:
            best[key] = row
    return [dict(best[key], time_with_the_librarys_choice=own.get(key, float("nan"))) for key in sorted(best)]


def write_fused_tuning(rows, path, hostname="mi355x", gpu="MI355X"):
    with open(path, "w", newline="") as handle:
        writer = csv.writer(handle, lineterminator="\n")
        writer.writerow(FUSED_TUNING_COLUMNS)
        for row in rows:
            full = dict(row, hostname=hostname, GPU=gpu)
            for name in ("time", "time_with_the_librarys_choice"):
                if name in full:
                    full[name] = f"{full[name]:.10g}"
            writer.writerow([full.get(name, "") for name in FUSED_TUNING_COLUMNS])


def config_fused(query_count, point_count, dim, k, arithmetic="exact", tuning_file=DEFAULT_FUSED_TUNING):
    """(ranges, first_radius, image, workgroup) for bitsknn_fused_l2_topk_f32_tuned from the shipped
    measurements: the row of the arithmetic whose problem is nearest to the request (sum of the
    absolute log ratios of queries, points, dimension and list length); (0, 0, 0, 0), the library's
    choice, without a file."""
    import math
    best, best_cost = (0, 0, 0, 0), None
    try:
        with open(tuning_file, newline="") as handle:
            for row in csv.DictReader(handle):
                if row["arithmetic"] != arithmetic:
                    continue
                cost = sum(abs(math.log(float(row[name]) / float(want)))
                           for name, want in (("query_count", query_count), ("point_count", point_count),
                                              ("dim", dim), ("k", k)))
                if best_cost is None or cost < best_cost:
                    best, best_cost = (int(row["ranges"]), int(row["first_radius"]), int(row.get("image") or 0),
                                       int(row.get("workgroup") or 0)), cost
    except OSError:
        pass
    return best


def sweep_partial_bitonic(repeats=5, problem_size=1 << 30, query_counts=(64, 256, 1024, 4096),
                          k_values=(32, 64, 128, 256, 512, 1024, 2048), block_sizes=(64, 128, 256, 512),
                          seed=17, progress=None):
    """Time partial-bitonic-regs on cuda:0 over q x (problem_size / q) matrices."""
    import torch
    import bitsknn

    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    flat = torch.rand(problem_size, device=dev, generator=gen)
    for q in query_counts:
        rows = flat.view(q, problem_size // q)
        for k in k_values:
            out_d = torch.empty((q, k), dtype=torch.float32, device=dev)
            out_l = torch.empty((q, k), dtype=torch.int32, device=dev)
            for block in block_sizes:
                bitsknn.topk_partial_bitonic(rows, k, block, out_dist=out_d, out_label=out_l)
                start = torch.cuda.Event(enable_timing=True)
                end = torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(repeats):
                    bitsknn.topk_partial_bitonic(rows, k, block, out_dist=out_d, out_label=out_l)
                end.record()
                end.synchronize()
                yield {"algorithm": "partial-bitonic-regs", "point_count": problem_size // q,
                       "query_count": q, "k": k, "dim": 1, "block_size": block, "items_per_thread": 1,
                       "items_per_thread2": 1, "items_per_thread3": 1, "deg": 1,
                       "time": start.elapsed_time(end) / 1e3 / repeats}
            if progress is not None:
                progress(q, k)


def optima(rows):
    """Fastest row of every (algorithm, point_count, query_count, k, dim)."""
    best = {}
    for row in rows:
        key = (row["algorithm"], row["point_count"], row["query_count"], row["k"], row["dim"])
        if key not in best or row["time"] < best[key]["time"]:
            best[key] = row
    return [best[key] for key in sorted(best)]


def write_optima(rows, path, hostname="mi355x", gpu="MI355X"):
    with open(path, "w", newline="") as handle:
        writer = csv.writer(handle, lineterminator="\n")
        writer.writerow(OPTIMA_COLUMNS)
        for row in rows:
            full = dict(row, hostname=hostname, GPU=gpu)
            full["time"] = f"{row['time']:.10g}"
            writer.writerow([full[name] for name in OPTIMA_COLUMNS])


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--out", default=DEFAULT_OPTIMA, help="optima CSV to write")
    ap.add_argument("--all", default=None, help="also write every measurement to this CSV")
    ap.add_argument("--repeats", type=int, default=10)
    ap.add_argument("--hostname", default="mi355x")
    ap.add_argument("--only", choices=("bits", "bits-sq", "partial-bitonic-regs", "fused-cache", "fused-tuning"),
                    default=None, help="time one family only (bits covers bits and bits-prefetch; fused-tuning: the "
                                       "launch parameters of the fused kernels, into --fused-out)")
    ap.add_argument("--fused-out", default=DEFAULT_FUSED_TUNING, help="fused tuning CSV to write")
    args = ap.parse_args(argv)

    def progress(q, k):
        print(f"q={q} k={k} done", file=sys.stderr, flush=True)

    if args.only == "fused-tuning":
        measured = list(sweep_fused_tuning(progress=progress))
        if args.all:
            write_fused_tuning(measured, args.all, args.hostname)
        write_fused_tuning(fused_optima(measured), args.fused_out, args.hostname)
        return 0
    rows = []
    if args.only in (None, "bits"):
        rows += list(sweep(repeats=args.repeats, progress=progress))
        rows += list(sweep(repeats=args.repeats, point_count=SHORT_ROWS_POINT_COUNT,
                           query_counts=(SHORT_ROWS_QUERY_COUNT,), progress=progress))
    if args.only in (None, "bits-sq"):
        rows += list(sweep_bits_sq(repeats=args.repeats, progress=progress))
    if args.only in (None, "fused-cache"):
        rows += list(sweep_fused(progress=progress))
    if args.only in (None, "partial-bitonic-regs"):
        rows += list(sweep_partial_bitonic(repeats=max(1, args.repeats // 2), progress=progress))
    if args.all:
        write_optima(rows, args.all, args.hostname)
    write_optima(optima(rows), args.out, args.hostname)
    return 0


if __name__ == "__main__":
    sys.exit(main())
