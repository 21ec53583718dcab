#!/usr/bin/env python3
"""Turns rocprofv3's rocpd databases into the short text summaries kept under profiles/.

rocprofv3 (ROCm 7) writes one SQLite database per run (`-d <dir> -o <name>` -> <dir>/**/<name>_results.db).
This script prints, for one or more such databases:

  kernels   per (kernel, grid): calls, mean / min duration in microseconds, registers, LDS
            (from a `--kernel-trace` run; the mean duration of the dominant kernel is the figure
            bench.py's `roofline.achieved` must agree with)
  counters  per (kernel, grid, counter): calls and mean value per dispatch (from a `--pmc` run)
  traffic   HBM bytes per launch of named kernels from a FETCH_SIZE pass and a WRITE_SIZE pass,
            each scaled by what the same counter reads for a plain device copy of known size in the
            same run (`bench.py --calibrate-copy` issues three 1 GiB copies), printed as
            `traffic <config> <tokens> <stage> <bytes>` lines that bench.py reads back from
            profiles/*hbm_counters*.txt for `roofline.traffic`

Examples (on the GPU box, from /tmp with TMPDIR=/tmp; every pass is its own run):
  rocprofv3 --kernel-trace --stats -d /tmp/kt -o b -- python3 bench.py --cpu-tokens 0
  rocprofv3 --pmc FETCH_SIZE --kernel-trace -d /tmp/pf -o b -- python3 bench.py --cpu-tokens 0 --host-steps 0 --steps 3 --warmup 1 --calibrate-copy
  rocprofv3 --pmc WRITE_SIZE --kernel-trace -d /tmp/pw -o b -- python3 bench.py --cpu-tokens 0 --host-steps 0 --steps 3 --warmup 1 --calibrate-copy
  python3 rocprof_summary.py kernels /tmp/kt
  python3 rocprof_summary.py counters /tmp/pf
  python3 rocprof_summary.py traffic /tmp/pf /tmp/pw --config mixtral_bf16 \\
      --map 4096:expert_gate_up='ffn_tiled_pipe_kernel<true>' --map 1:expert_gate_up='ffn_stream_kernel<1, false, true@229376,2,1'
"""
import argparse
import glob
import os
import sqlite3
import sys

COPY_KERNEL = "__amd_rocclr_copyBuffer"
ROOT = os.path.dirname(os.path.abspath(__file__))


def kernels_sha():
    """Short hash of the kernel sources this tree builds (csrc/*.hip, *.h, Makefile).  A counter
    summary records it, and bench.py quotes the summary's HBM traffic only while the hash still
    matches the sources it runs: after a kernel change the line says that the figure is stale."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "ateniaengine_amd", "csrc")
    for name in sorted(os.listdir(src)):
        if name.endswith((".hip", ".h")) or name == "Makefile":
            with open(os.path.join(src, name), "rb") as fh:
                h.update(name.encode() + b"\0" + fh.read())
    return h.hexdigest()[:16]


def find_db(path):
    if os.path.isfile(path):
        return path
    dbs = sorted(glob.glob(os.path.join(path, "**", "*.db"), recursive=True))
    if not dbs:
        sys.exit(f"no rocpd database under {path}")
    return dbs[0]


def short(name):
    return name.replace("atenia_moe::(anonymous namespace)::", "").replace("void ", "")


def kernels(db, limit):
    c = sqlite3.connect(db)
    print(f"{'kernel':74s} {'grid':>22s} {'calls':>6s} {'mean_us':>10s} {'min_us':>10s} "
          f"{'vgpr':>5s} {'agpr':>5s} {'lds':>7s}")
    q = ("select name, grid_x, grid_y, grid_z, count(*), avg(duration), min(duration), vgpr_count, "
         "accum_vgpr_count, lds_size from kernels group by name, grid_x, grid_y, grid_z "
         f"order by sum(duration) desc limit {int(limit)}")
    for r in c.execute(q):
        print(f"{short(r[0])[:74]:74s} {str(r[1:4]):>22s} {r[4]:6d} {r[5] / 1000:10.2f} "
              f"{r[6] / 1000:10.2f} {r[7]:5d} {r[8]:5d} {r[9]:7d}")


def counter_rows(db):
    c = sqlite3.connect(db)
    q = ("select p.name, k.grid_x, k.grid_y, k.grid_z, p.counter_name, count(*), avg(p.counter_value) "
         "from pmc_events p join kernels k on p.dispatch_id = k.dispatch_id "
         "group by p.name, k.grid_x, k.grid_y, k.grid_z, p.counter_name "
         "order by p.name, k.grid_x, p.counter_name")
    return list(c.execute(q))


def counters(db, only):
    print(f"{'kernel':74s} {'grid':>22s} {'counter':>32s} {'calls':>6s} {'mean per dispatch':>18s}")
    for r in counter_rows(db):
        if only and not any(o in r[0] for o in only):
            continue
        print(f"{short(r[0])[:74]:74s} {str(r[1:4]):>22s} {r[4]:>32s} {r[5]:6d} {r[6]:18.1f}")


def traffic(fetch_db, write_db, config, maps, copy_bytes):
    def per_kernel(db, counter):
        rows = [r for r in counter_rows(db) if r[4] == counter]
        copy = [r[6] for r in rows if COPY_KERNEL in r[0]]
        if not copy:
            sys.exit(f"{db}: no {COPY_KERNEL} dispatch to calibrate {counter} with "
                     "(run bench.py with --calibrate-copy)")
        unit = copy_bytes / max(copy)  # bytes per counter unit
        return rows, unit

    f_rows, f_unit = per_kernel(fetch_db, "FETCH_SIZE")
    w_rows, w_unit = per_kernel(write_db, "WRITE_SIZE")
    print(f"kernels_sha {kernels_sha()}")
    print(f"# calibration: a {copy_bytes} byte device copy reads FETCH_SIZE x {f_unit:.1f} B and "
          f"WRITE_SIZE x {w_unit:.1f} B per unit")
    def pick(rows, pattern):
        grid = None
        if "@" in pattern:  # <substring>@gx,gy,gz picks one launch shape of the kernel
            pattern, g = pattern.rsplit("@", 1)
            grid = tuple(int(v) for v in g.split(","))
        pattern = pattern.replace(",_", ", ")  # "<1,_false>" may be written for "<1, false>"
        hit = [r for r in rows if pattern in short(r[0]) and (grid is None or r[1:4] == grid)]
        if not hit:
            sys.exit(f"no dispatch matches {pattern!r} {grid or ''}")
        # several launch shapes of one kernel match a bare substring: the largest one is meant
        return max(hit, key=lambda r: r[6])

    for m in maps:
        tokens, rest = m.split(":", 1)
        stage, patterns = rest.split("=", 1)
        total = 0.0
        for pattern in patterns.split("+"):  # a stage of several launches: their sum
            f, w = pick(f_rows, pattern), pick(w_rows, pattern)
            print(f"# {short(f[0])[:70]} grid {f[1:4]}: read {f[6] * f_unit / 1e9:.3f} GB, "
                  f"written {w[6] * w_unit / 1e9:.3f} GB per launch")
            total += f[6] * f_unit + w[6] * w_unit
        print(f"traffic {config} {int(tokens)} {stage} {total:.1f}")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    k = sub.add_parser("kernels")
    k.add_argument("db")
    k.add_argument("--limit", type=int, default=30)
    c = sub.add_parser("counters")
    c.add_argument("db")
    c.add_argument("--only", action="append", default=[], help="substring of the kernel name")
    t = sub.add_parser("traffic")
    t.add_argument("fetch_db")
    t.add_argument("write_db")
    t.add_argument("--config", required=True)
    t.add_argument("--map", action="append", default=[], required=True,
                   help="<tokens>:<stage>=<substring of the kernel name>[@gx,gy,gz][+<another launch>...]")
    t.add_argument("--copy-bytes", type=float, default=float(1 << 30))
    a = ap.parse_args()
    if a.cmd == "kernels":
        kernels(find_db(a.db), a.limit)
    elif a.cmd == "counters":
        counters(find_db(a.db), a.only)
    else:
        traffic(find_db(a.fetch_db), find_db(a.write_db), a.config, a.map, a.copy_bytes)


if __name__ == "__main__":
    main()
