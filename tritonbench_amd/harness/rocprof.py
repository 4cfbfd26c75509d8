"""`rocprof` metric: per-kernel device time (and optionally hardware counters) of ONE
(backend, input) pair, collected by re-launching the benchmark in a fresh child process under
rocprofv3.

Upstream's counterpart re-launches `sys.argv` with `--only <backend> --input-id <i>
--num-inputs 1 --metrics <in-task metric>` under a profiler and returns where the trace went
(tritonbench/utils/triton_op.py:1599-1623, 1749-1753; the AMD flavour is the ATT tracer of
tritonbench/components/att/att_trace.py:36-64, which needs rocprofv2's ATT plugin). Here the
child runs under `rocprofv3 --kernel-trace --stats` (or one `--pmc` pass) and the CSV summary
is parsed into the result table, so the figure that counts, average microseconds per kernel, is
in the table itself.

Rules of the road for the child process:
  * it is spawned with subprocess (a new process), never exec'ed over a process that has
    touched the GPU;
  * the interpreter comes directly after `--`: no `env`, no shell, no launcher script;
  * counter passes are their own runs (`--pmc` is never combined with a trace option), and
    a pass must fit the hardware's counter blocks (checked before anything is launched).
"""
import csv
import os
import shutil
import subprocess
import sys
import tempfile
from typing import Dict, Iterable, List, Optional, Sequence

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
RUN_PY = os.path.join(ROOT, "run.py")
IN_TASK_METRIC = "_rocprof_in_task"  # what the child is asked for: run the backend a few times, no timing loops
OUTPUT_NAME = "run"

# counters one rocprofv3 pass can hold, by hardware block (a derived counter may use several:
# FETCH_SIZE takes three TCC counters, WRITE_SIZE two); asking for more makes rocprofv3 print
# "Request exceeds the capabilities of the hardware to collect" and hang
PMC_BLOCK_LIMITS = {"SQ_": 8, "TCC_": 4, "TCP_": 4, "TA_": 2, "TD_": 2, "GRBM_": 2}
DERIVED_COST = {"FETCH_SIZE": ("TCC_", 3), "WRITE_SIZE": ("TCC_", 2)}


def find_rocprofv3() -> str:
    path = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(path):
        raise NotImplementedError("rocprofv3 not found (looked on PATH and in /opt/rocm/bin)")
    return path


def check_pmc_fits(counters: Sequence[str]) -> None:
    """Raises ValueError when the counters cannot be collected in one pass."""
    used: Dict[str, int] = {}
    seen = set()
    for c in counters:
        base = c
        for suffix in ("_sum", "_avr", "_min", "_max"):  # reductions of one counter count once
            if base.endswith(suffix):
                base = base[: -len(suffix)]
        if base in seen:
            continue
        seen.add(base)
        if base in DERIVED_COST:
            block, cost = DERIVED_COST[base]
        else:
            block = next((b for b in PMC_BLOCK_LIMITS if base.startswith(b)), None)
            cost = 1
        if block is not None:
            used[block] = used.get(block, 0) + cost
    for block, n in used.items():
        if n > PMC_BLOCK_LIMITS[block]:
            raise ValueError(
                f"{n} {block}* counters in one pass, the hardware collects {PMC_BLOCK_LIMITS[block]}: "
                "split them over separate runs"
            )


def child_argv(op_name: str, fn_name: str, input_id: int, tb_args=None, extra_args: Optional[Iterable[str]] = None,
               python: Optional[str] = None) -> List[str]:
    """Command line of the child: this repository's run.py restricted to one backend and one
    input, asked for the in-task metric. Harness flags that change the inputs or the backend
    are carried over; everything the operator's own parser reads is passed through."""
    argv = [python or sys.executable, RUN_PY, "--op", op_name, "--only", fn_name, "--input-id", str(input_id),
            "--num-inputs", "1", "--metrics", IN_TASK_METRIC]
    if tb_args is not None:
        if getattr(tb_args, "device", None):
            argv += ["--device", tb_args.device]
        precision = getattr(tb_args, "precision", None)
        if precision and precision != "bypass":
            argv += ["--precision", precision]
    argv += list(extra_args or [])
    return argv


def profiler_argv(child: Sequence[str], out_dir: str, pmc: Optional[Sequence[str]] = None) -> List[str]:
    """rocprofv3 command line around `child`: kernel trace with statistics, or one counter pass."""
    if pmc:
        check_pmc_fits(pmc)
        mode = ["--pmc", *pmc]
    else:
        mode = ["--kernel-trace", "--stats"]
    first = os.path.basename(child[0])
    if not first.startswith("python"):
        raise ValueError(f"the program after `--` must be the interpreter itself, not {child[0]!r}")
    return [find_rocprofv3(), *mode, "-f", "csv", "-d", out_dir, "-o", OUTPUT_NAME, "--", *child]


def _find(out_dir: str, suffix: str) -> str:
    for base, _, files in os.walk(out_dir):
        for f in files:
            if f.endswith(suffix):
                return os.path.join(base, f)
    raise FileNotFoundError(f"no *{suffix} under {out_dir}")


def parse_kernel_stats(path: str) -> List[dict]:
    """Rows of a rocprofv3 `*_kernel_stats.csv`: name, calls, average / min / max microseconds
    and share of the device time, in the file's order (largest total first)."""
    rows = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            rows.append({
                "name": r["Name"],
                "calls": int(r["Calls"]),
                "avg_us": float(r["AverageNs"]) / 1e3,
                "min_us": float(r["MinNs"]) / 1e3,
                "max_us": float(r["MaxNs"]) / 1e3,
                "total_us": float(r["TotalDurationNs"]) / 1e3,
                "percent": float(r["Percentage"]),
            })
    return rows


def parse_counters(path: str) -> Dict[str, Dict[str, dict]]:
    """`*_counter_collection.csv` -> {kernel name: {counter: {"mean", "min", "max", "dispatches"}}}."""
    acc: Dict[str, Dict[str, List[float]]] = {}
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            acc.setdefault(r["Kernel_Name"], {}).setdefault(r["Counter_Name"], []).append(float(r["Counter_Value"]))
    return {
        k: {c: {"mean": sum(v) / len(v), "min": min(v), "max": max(v), "dispatches": len(v)} for c, v in per.items()}
        for k, per in acc.items()
    }


MARKER_KERNEL = "FillFunctor<short>"  # the child brackets its timed calls with fills of an int16 tensor
IN_TASK_WARMUP = 2
IN_TASK_CALLS = 5


def run_in_task(fn) -> int:
    """What the child does for IN_TASK_METRIC: a few untimed calls, then IN_TASK_CALLS calls
    between two marker kernels the parent finds in the kernel trace."""
    import torch

    marker = torch.empty(3, dtype=torch.int16, device="cuda")
    for _ in range(IN_TASK_WARMUP):
        fn()
    torch.cuda.synchronize()
    marker.fill_(7)
    for _ in range(IN_TASK_CALLS):
        fn()
    marker.fill_(9)
    torch.cuda.synchronize()
    return IN_TASK_CALLS


def parse_kernel_trace(path: str) -> List[dict]:
    """Dispatches of a rocprofv3 `*_kernel_trace.csv` in start order: name, start_ns, dur_us."""
    rows = []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            a, b = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
            rows.append({"name": r["Kernel_Name"], "start_ns": a, "dur_us": (b - a) / 1e3})
    rows.sort(key=lambda r: r["start_ns"])
    return rows


def window_stats(dispatches: Sequence[dict], calls: int = IN_TASK_CALLS, marker: str = MARKER_KERNEL) -> List[dict]:
    """Per-kernel statistics of the dispatches between the last two marker kernels:
    launches per call, average / min / max microseconds, microseconds per call."""
    marks = [i for i, d in enumerate(dispatches) if marker in d["name"]]
    if len(marks) < 2:
        raise RuntimeError(f"kernel trace holds {len(marks)} marker kernels ({marker}), expected two")
    inside = dispatches[marks[-2] + 1: marks[-1]]
    by_name: Dict[str, List[float]] = {}
    for d in inside:
        by_name.setdefault(d["name"], []).append(d["dur_us"])
    rows = []
    for name, durs in by_name.items():
        rows.append({
            "name": name, "kernel": short_kernel_name(name), "launches_per_call": len(durs) / calls,
            "avg_us": sum(durs) / len(durs), "min_us": min(durs), "max_us": max(durs),
            "us_per_call": sum(durs) / calls,
        })
    rows.sort(key=lambda r: -r["us_per_call"])
    return rows


def format_rows(rows: Sequence[dict]) -> str:
    """One table cell: `kernel: avg us x launches per call; ...`, largest first."""
    return "; ".join(f"{r['kernel']}: {r['avg_us']:.1f} us x{r['launches_per_call']:g}" for r in rows)


def short_kernel_name(name: str) -> str:
    """`void (anonymous namespace)::gemm_tiled_kernel<256, ...>(...)` -> `gemm_tiled_kernel<256, ...>`."""
    s = name.strip()
    if s.startswith("void "):
        s = s[5:]
    depth, cut = 0, len(s)
    for i, ch in enumerate(s):  # drop the argument list: the first '(' outside template brackets ...
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0 and not s.startswith("(anonymous namespace)", i):
            cut = i
            break
    s = s[:cut]
    return s.replace("(anonymous namespace)::", "")


def matching(rows: Iterable[dict], substrings: Sequence[str]) -> List[dict]:
    return [r for r in rows if any(sub in r["name"] for sub in substrings)]


def run_profiler(child: Sequence[str], pmc: Optional[Sequence[str]] = None, out_dir: Optional[str] = None,
                 timeout_s: float = 300.0) -> str:
    """Runs the child under rocprofv3 in a new process; returns the output directory."""
    out_dir = out_dir or tempfile.mkdtemp(prefix="rocprof_")
    os.makedirs(out_dir, exist_ok=True)
    cmd = profiler_argv(child, out_dir, pmc)
    env = dict(os.environ)
    env.setdefault("TMPDIR", "/tmp")
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout_s,
                          cwd=tempfile.gettempdir(), env=env)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)} failed with status {proc.returncode}:\n{proc.stdout[-2000:]}")
    return out_dir


def profile_backend(op_name: str, fn_name: str, input_id: int, tb_args=None, extra_args=None,
                    out_dir: Optional[str] = None) -> List[dict]:
    """The metric: per-kernel device time of one backend on one input, measured in a child
    process (its IN_TASK_CALLS calls between the two marker kernels)."""
    child = child_argv(op_name, fn_name, input_id, tb_args, extra_args)
    where = run_profiler(child, out_dir=out_dir)
    return window_stats(parse_kernel_trace(_find(where, "_kernel_trace.csv")))


def profile_backend_counters(op_name: str, fn_name: str, input_id: int, counters: Sequence[str], tb_args=None,
                             extra_args=None, kernels: Optional[Sequence[str]] = None,
                             out_dir: Optional[str] = None) -> Dict[str, Dict[str, float]]:
    """One counter pass over the same child: {short kernel name: {counter: mean per dispatch}} for the
    kernels whose full names are in `kernels` (all of the child's kernels when None). The means are
    over every dispatch of a kernel in the child, its warm-up calls included."""
    check_pmc_fits(counters)
    child = child_argv(op_name, fn_name, input_id, tb_args, extra_args)
    where = run_profiler(child, pmc=list(counters), out_dir=out_dir)
    table = parse_counters(_find(where, "_counter_collection.csv"))
    keep = None if kernels is None else set(kernels)
    return {short_kernel_name(name): {c: v["mean"] for c, v in per.items()}
            for name, per in table.items() if keep is None or name in keep}


def format_counters(per_kernel: Dict[str, Dict[str, float]]) -> str:
    """One table cell: `kernel: COUNTER=mean, ...; ...`."""
    return "; ".join(f"{k}: " + ", ".join(f"{c}={v:.6g}" for c, v in sorted(per.items()))
                     for k, per in per_kernel.items())


# ---- traffic summary for bench.py -----------------------------------------------------------

def traffic_summary(fetch_csv: str, write_csv: str, kernel: str, copy_kernel: str, copy_read_bytes: int,
                    copy_write_bytes: int) -> dict:
    """HBM-side bytes per launch of the kernel whose name contains `kernel`, from two counter
    passes (FETCH_SIZE, then WRITE_SIZE; both count KiB per dispatch), each scaled by what the
    same counter reads for a copy kernel of known size in the same run (`copy_kernel`)."""
    fetch, write = parse_counters(fetch_csv), parse_counters(write_csv)

    def pick(table, sub, counter):
        hits = [(k, v[counter]) for k, v in table.items() if sub in k and counter in v]
        if not hits:
            raise KeyError(f"no kernel matching {sub!r} with {counter} in the counter file")
        return max(hits, key=lambda kv: kv[1]["dispatches"])

    _, cal_f = pick(fetch, copy_kernel, "FETCH_SIZE")
    _, cal_w = pick(write, copy_kernel, "WRITE_SIZE")
    fetch_factor = copy_read_bytes / (cal_f["mean"] * 1024.0)
    write_factor = copy_write_bytes / (cal_w["mean"] * 1024.0)
    name, f = pick(fetch, kernel, "FETCH_SIZE")
    _, w = pick(write, kernel, "WRITE_SIZE")
    fetched = f["mean"] * 1024.0 * fetch_factor
    written = w["mean"] * 1024.0 * write_factor
    return {
        "kernel": short_kernel_name(name),
        "dispatches": f["dispatches"],
        "fetch_kib_raw": f["mean"],
        "write_kib_raw": w["mean"],
        "fetch_factor": fetch_factor,
        "write_factor": write_factor,
        "fetch_bytes": int(round(fetched)),
        "write_bytes": int(round(written)),
        "traffic_bytes": int(round(fetched + written)),
    }
