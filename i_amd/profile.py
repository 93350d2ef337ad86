"""Per-kernel report from a rocprofv3 run of a program that uses this backend.

rocprofv3 (ROCm 7) writes its results as a rocpd SQLite database; two of its views are all a kernel-level
report needs: ``kernels`` (one row per dispatch: name, start, end, duration in ns, grid, workgroup, LDS) and ``counters_collection`` (one row per dispatch and counter when the run had ``--pmc``).  Typical use::

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --kernel-trace --stats -d out -o run -- python3 my_script.py
    python3 -m i_amd.profile out/run_results.db              # every kernel of the run
    python3 -m i_amd.profile out/run_results.db --ours        # only this backend's kernels

The hand-written kernels keep their names in the trace (``attn_fwd_bf16_d128_bn64_direct_w8``,
``gemm_nt_bf16_256x256x64_direct``, ``row_softmax_wave_v16`` ...) and generated kernels are ``f<k>`` /
``f<k>_p<i>`` as in the plan that ``Component._code()`` prints, so a row of the report can be matched to a kernel
of the component by name.  The reference's only introspection tool is the printed source (core/src/lib.rs:124-139);
this is its counterpart for time.
"""
import argparse
import re
import sqlite3
from collections import namedtuple

KernelRow = namedtuple("KernelRow", "name calls total_us avg_us min_us max_us share lds_bytes workgroup")
CounterRow = namedtuple("CounterRow", "kernel counter dispatches avg min max")

# every name the backend can launch: the hand-written kernels (kernels/kernels.hip), the generated kernels f<k> in
# their forms (_w: a wavefront per iteration, _g / _gw: a loop in parts) and the helpers generated beside them
_OURS = re.compile(r"^(attn_fwd_|attn_kv_merge$|gemm_n[nt]_|splitk_reduce$|row_(softmax|shift|norm|exp|scaled_softmax)_|transpose_b(16|32)$|"
                   r"pad_rows_b(16|32)$|convert_|shader_clock_probe$|ilang_(fill|combine|combine_w)$|f\d+(_w|_g|_gw)?$)")


def is_backend_kernel(name):
    """True for the names this backend launches (hand-written kernels and generated ``f<k>`` kernels)."""
    return bool(_OURS.match(name.split("(")[0]))


def _columns(db, view):
    return {r[1] for r in db.execute(f"pragma table_info({view})")}


def kernel_rows(db_path, ours_only=False):
    """One KernelRow per kernel name, sorted by total time."""
    db = sqlite3.connect(f"file:{db_path}?mode=ro", uri=True)
    cols = _columns(db, "kernels")
    if not {"name", "duration"} <= cols:
        raise ValueError(f"{db_path}: no rocpd 'kernels' view with name and duration columns")
    extra = [c if c in cols else "null" for c in ("lds_size", "workgroup_x")]
    rows = db.execute(
        f"select name, count(*), sum(duration), avg(duration), min(duration), max(duration), "
        f"max({extra[0]}), max({extra[1]}) from kernels group by name order by sum(duration) desc").fetchall()
    if ours_only:
        rows = [r for r in rows if is_backend_kernel(r[0])]
    total = sum(r[2] for r in rows) or 1
    return [KernelRow(r[0], r[1], r[2] / 1e3, r[3] / 1e3, r[4] / 1e3, r[5] / 1e3, r[2] / total, r[6], r[7]) for r in rows]


def dispatch_durations_us(db_path, kernel):
    """Durations of one kernel's dispatches in start order (warm-up, timed steps ... as the program issued them)."""
    db = sqlite3.connect(f"file:{db_path}?mode=ro", uri=True)
    return [r[0] / 1e3 for r in db.execute("select duration from kernels where name = ? order by start", (kernel,))]


def counter_rows(db_path, ours_only=False):
    """One CounterRow per (kernel, counter) of a ``--pmc`` run; empty when the run collected no counters."""
    db = sqlite3.connect(f"file:{db_path}?mode=ro", uri=True)
    if not {"kernel_name", "counter_name", "value"} <= _columns(db, "counters_collection"):
        return []
    rows = db.execute("select kernel_name, counter_name, count(*), avg(value), min(value), max(value) "
                      "from counters_collection group by kernel_name, counter_name order by kernel_name, counter_name").fetchall()
    if ours_only:
        rows = [r for r in rows if is_backend_kernel(r[0])]
    return [CounterRow(*r) for r in rows]


def _short(name, width=64):
    name = name.split("(")[0]
    return name if len(name) <= width else name[: width - 3] + "..."


def format_report(db_path, ours_only=False, top=20):
    """Markdown tables: kernels by total time, then counters per kernel if there are any."""
    out = ["| kernel | calls | avg us | min us | max us | % of GPU time | LDS bytes | workgroup |", "|---|---|---|---|---|---|---|---|"]
    for r in kernel_rows(db_path, ours_only)[:top]:
        out.append(f"| {_short(r.name)} | {r.calls} | {r.avg_us:.1f} | {r.min_us:.1f} | {r.max_us:.1f} | {100 * r.share:.1f} | "
                   f"{r.lds_bytes if r.lds_bytes is not None else ''} | "
                   f"{r.workgroup if r.workgroup is not None else ''} |")
    counters = counter_rows(db_path, ours_only)
    if counters:
        out += ["", "| kernel | counter | dispatches | avg | min | max |", "|---|---|---|---|---|---|"]
        out += [f"| {_short(c.kernel)} | {c.counter} | {c.dispatches} | {c.avg:.0f} | {c.min:.0f} | {c.max:.0f} |" for c in counters]
    return "\n".join(out)


def main(argv=None):
    ap = argparse.ArgumentParser(description="per-kernel report from a rocprofv3 (rocpd SQLite) result file")
    ap.add_argument("database", help="<dir>/<name>_results.db written by rocprofv3 -d <dir> -o <name>")
    ap.add_argument("--ours", action="store_true", help="only the kernels this backend launches")
    ap.add_argument("--top", type=int, default=20)
    args = ap.parse_args(argv)
    print(format_report(args.database, args.ours, args.top))


if __name__ == "__main__":
    main()
