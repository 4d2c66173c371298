"""Jain's fairness index over per-model slowdown factors, from the load generator's stats files.

Follows reference tools/calculate_jains_fairness_index.py:14-27: for every row of a sweep file (one row per
fairness threshold), slowdown_i = latency of model i in the mix / latency of model i served alone, and

    index = (sum_i slowdown_i)^2 / (n * sum_i slowdown_i^2)          (1 = all models slowed down equally, 1/n = one starved)

A stats row is what llis_app_client appends per run (reference app/client.cpp:479-494):
    x, num_jobs, elapsed_us, then 7 columns {mean, p50, p90, p95, p99, max, sd} for all requests and 7 per job type.

Column choice.  The reference script indexes the sweep file with `9::7` and a baseline file with `[2]`.  Against the
row layout above those are the standard-deviation columns and the elapsed time, so the script was evidently written
for an earlier row layout; `reference_columns=True` reproduces that indexing literally, the default takes the
per-type column of the chosen statistic (mean unless told otherwise) and the same statistic of the baseline's
all-requests block.
"""
import argparse

import numpy as np

STATS = ("mean", "p50", "p90", "p95", "p99", "max", "sd")
FIRST_STATS_COLUMN = 3


def jain_index(values):
    """(sum x)^2 / (n sum x^2) along the last axis."""
    v = np.asarray(values, dtype=np.float64)
    return v.sum(axis=-1) ** 2 / (v.shape[-1] * (v ** 2).sum(axis=-1))


def _rows(path):
    return np.atleast_2d(np.genfromtxt(path, delimiter=","))


def slowdown_table(sweep_rows, baseline_rows, stat="mean", reference_columns=False):
    """sweep_rows: 2-D array, one stats row per sweep point.  baseline_rows: one stats row per model, in job-type
    order.  Returns an array with columns [x, index, slowdown_0, slowdown_1, ...] -- the reference tool's output."""
    data = np.atleast_2d(np.asarray(sweep_rows, dtype=np.float64))
    base = [np.asarray(b, dtype=np.float64).reshape(-1) for b in baseline_rows]
    if reference_columns:
        mix = data[:, 9::7]
        alone = np.array([b[2] for b in base])
    else:
        k = STATS.index(stat)
        first = FIRST_STATS_COLUMN + len(STATS) + k
        mix = data[:, first::len(STATS)]
        alone = np.array([b[FIRST_STATS_COLUMN + k] for b in base])
    if mix.shape[1] != len(alone):
        raise ValueError("%d job types in the sweep file but %d baselines" % (mix.shape[1], len(alone)))
    slowdown = mix / alone
    return np.concatenate([data[:, 0:1], jain_index(slowdown)[:, None], slowdown], axis=1)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("-o", "--output_path", required=True)
    ap.add_argument("-b", "--input_baseline_path", dest="input_baseline_paths", action="append", required=True,
                    help="stats file of one model served alone; give one per job type, in job-type order")
    ap.add_argument("-i", "--input_path", required=True, help="stats file of the sweep (one row per threshold)")
    ap.add_argument("--stat", choices=STATS, default="mean")
    ap.add_argument("--reference-columns", action="store_true", help="index the files exactly as the reference script does")
    args = ap.parse_args(argv)
    table = slowdown_table(_rows(args.input_path), [_rows(p)[-1] for p in args.input_baseline_paths], args.stat, args.reference_columns)
    np.savetxt(args.output_path, table, delimiter=",")


if __name__ == "__main__":
    main()
