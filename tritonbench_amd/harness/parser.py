"""Harness-level command line (the subset of tritonbench/utils/parser.py:7-322 a single
operator run reads). Unknown flags are left for the operator's own parser, as upstream's
parse_known_args split does (run.py:112-113)."""
import argparse


def get_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(allow_abbrev=False)
    p.add_argument("--op", type=str, required=False, help="operator to benchmark")
    p.add_argument("--mode", choices=["fwd", "bwd", "fwd_bwd", "fwd_no_grad"], default="fwd")
    p.add_argument("--precision", "--dtype", default="bypass")
    p.add_argument("--device", default="cuda", choices=["cuda", "cpu"])
    p.add_argument("--warmup", type=int, default=25, help="warm-up time (ms)")
    p.add_argument("--iter", type=int, default=100, help="measurement time (ms)")
    p.add_argument("--csv", action="store_true", help="print the table as ';'-separated values")
    p.add_argument("--output", default=None, help="write CSV to this file")
    p.add_argument("--output-json", default=None, help="write the flat JSON dict to this file")
    p.add_argument("--output-dir", default=None, help="write a uniquely named CSV into this directory")
    p.add_argument("--simple-output", action="store_true")
    p.add_argument("--benchmark-name", default=None)
    p.add_argument("--metrics", default=None, help="comma separated metric names")
    p.add_argument("--only", default=None, help="comma separated backend names to run")
    p.add_argument("--skip", default=None, help="comma separated backend names to leave out")
    p.add_argument("--only-match-mode", choices=["exact", "prefix-with-baseline"], default="exact")
    p.add_argument("--baseline", default=None, help="backend to compare the others against")
    p.add_argument("--num-inputs", type=int, default=None)
    p.add_argument("--input-id", type=int, default=0)
    p.add_argument("--keep-going", action="store_true", help="record a backend's exception instead of raising")
    p.add_argument("--bypass-fail", action="store_true")
    p.add_argument("--cudagraph", action="store_true", help="time a captured graph of repeated calls")
    p.add_argument("--test-only", action="store_true", help="run each backend once, no timing loops")
    p.add_argument("--rtol", type=float, default=None)
    p.add_argument("--atol", type=float, default=None)
    p.add_argument("--export", choices=["input", "output", "both"], default=None,
                   help="dump the inputs and/or every backend's output as .pt files")
    p.add_argument("--export-dir", default=None, help="existing directory for --export")
    p.add_argument("--rocprof-pmc", default=None,
                   help="with --metrics rocprof: hardware counters (comma separated, one rocprofv3 pass) collected "
                        "in a second child run and shown per kernel")
    p.add_argument("--list-backends", action="store_true")
    return p
