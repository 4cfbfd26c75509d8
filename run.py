"""`python run.py --op fp8_gemm_rowwise [--m M --n N --k K] [--bias] [--metrics ...]`

Entry point with the same command line shape as tritonbench's run.py: harness flags are
parsed here, everything unknown is handed to the operator's own parser.
"""
import sys
from typing import List, Optional

from tritonbench_amd.harness.loader import list_operators, load_opbench_by_name
from tritonbench_amd.harness.parser import get_parser
from tritonbench_amd.harness.registry import REGISTERED_BENCHMARKS


def _run(args, extra_args):
    Opbench = load_opbench_by_name(args.op)
    opbench = Opbench(tb_args=args, extra_args=extra_args)
    if args.list_backends:
        for name, cfg in REGISTERED_BENCHMARKS[opbench.name].items():
            print(f"{name}\tlabel={cfg.label}\tbaseline={cfg.baseline}\tenabled={cfg.enabled}")
        return None
    if args.test_only:
        opbench.run(0, 1)
    else:
        opbench.run(args.warmup, args.iter)
    out = opbench.output
    if args.output_dir:
        print(f"[run.py] wrote {out.write_csv(args.output_dir)}")
    if args.output:
        with open(args.output, "w", newline="") as f:
            out.write_csv_to_file(f)
    if args.output_json:
        with open(args.output_json, "w") as f:
            out.write_json_to_file(f)
    if args.csv:
        out.write_csv_to_file(sys.stdout)
    else:
        print(out)
    return out


def run(argv: Optional[List[str]] = None):
    parser = get_parser()
    args, extra_args = parser.parse_known_args(argv)
    if not args.op:
        print("available operators: " + ", ".join(list_operators()))
        return None
    ops = [o for o in args.op.split(",") if o]
    result = None
    for op in ops:
        args.op = op
        result = _run(args, extra_args)
    return result


if __name__ == "__main__":
    run()
