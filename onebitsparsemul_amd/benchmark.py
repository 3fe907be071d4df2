"""Command-line benchmark with the flag spellings of the reference's `a.out` (tests/kernel_test.cu:121-216,
README.md:23-26, script/cuda_run_test.sh):

    python -m onebitsparsemul_amd.benchmark --a_rows=8192 --n=8192 --a_cols=8192 --reference-check=false
    python -m onebitsparsemul_amd.benchmark --sweep            # 512 ... 12800 squares, 30 iterations each
    python -m onebitsparsemul_amd.benchmark --sweep --json sweep.json --csv sweep.csv
    python -m onebitsparsemul_amd.benchmark --layer --a_rows=11008 --n=16 --a_cols=4096   # BinaryLinear_2_4's kernel call

Prints the reference's table columns (a_rows, n, a_cols, GFLOPs = 2*M*N*K / t, runtime in ms). Timing mirrors
tests/kernel_test.cu:619-691: one warm-up, then `iterations` back-to-back launches between two events. Output
dtype fp32 and alpha = beta = 1 by default, as in the reference benchmark (tests/kernel_test.cu:563-564,
csrc/kernel.h:17). --reference-check compares with a dense fp32 matmul of the decompressed weight on the GPU
(the reference's check is a host GEMM on the decompressed weight, tests/kernel_test.cu:410-505).
--layer times the form the linear layer uses instead: y (n tokens x a_rows) = x (n x a_cols) @ W.T + bias, x and y
token-major, fp16 result (no alpha / beta).
"""
import argparse
import sys

import torch

from . import _native, dequant_desparse_tile, synthetic

SWEEP = (512, 1024, 2048, 4096, 8192, 10240, 12800)  # script/cuda_run_test.sh:4


def _bool(text):
    return str(text).lower() in ("1", "true", "yes", "on")


def run_layer(a_rows, n, a_cols, iterations, reference_check, seed=3080):
    m, k = a_rows, a_cols
    a, meta = synthetic.make_weight(m, k, seed, device="cuda")
    x = synthetic.make_b(n, k, seed, kind="int" if reference_check else "normal", device="cuda")
    bias = torch.randint(-8, 9, (m,), device="cuda").to(torch.float16)
    prep = _native.prepare(a, meta, m, k)
    y = torch.empty((n, m), dtype=torch.float16, device="cuda")
    _native.linear_prepared(prep, x, y, m, k, bias=bias)
    torch.cuda.synchronize()
    passed = None
    if reference_check:
        ref = x.to(torch.float32) @ dequant_desparse_tile(a, meta).to(torch.float32).T + bias.to(torch.float32)
        passed = bool(torch.equal(y.to(torch.float32), ref.to(torch.float16).to(torch.float32)))
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iterations):
        _native.linear_prepared(prep, x, y, m, k, bias=bias)
    stop.record()
    torch.cuda.synchronize()
    runtime_ms = start.elapsed_time(stop) / iterations
    return runtime_ms, 2.0 * m * n * k / (runtime_ms * 1e-3) / 1e9, passed


def run(a_rows, n, a_cols, alpha, beta, iterations, reference_check, out_dtype=torch.float32, seed=3080):
    m, k = a_rows, a_cols
    a, meta = synthetic.make_weight(m, k, seed, device="cuda")
    b = synthetic.make_b(k, n, seed, kind="int" if reference_check else "normal", device="cuda")
    c = torch.randint(-8, 9, (m, n), device="cuda").to(out_dtype) if beta != 0 else None
    prep = _native.prepare(a, meta, m, k)
    d = torch.empty((m, n), dtype=out_dtype, device="cuda")
    _native.matmul_prepared(prep, b, d, m, n, k, c=c, alpha=alpha, beta=beta)
    torch.cuda.synchronize()
    passed = None
    if reference_check:
        dense = dequant_desparse_tile(a, meta).to(torch.float32)
        ref = alpha * (dense @ b.to(torch.float32))
        if c is not None:
            ref = ref + beta * c.to(torch.float32)
        passed = bool(torch.equal(d.to(torch.float32), ref.to(out_dtype).to(torch.float32)))
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iterations):
        _native.matmul_prepared(prep, b, d, m, n, k, c=c, alpha=alpha, beta=beta)
    stop.record()
    torch.cuda.synchronize()
    runtime_ms = start.elapsed_time(stop) / iterations
    gflops = 2.0 * m * n * k / (runtime_ms * 1e-3) / 1e9
    return runtime_ms, gflops, passed


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--a_rows", type=int, default=1024)
    ap.add_argument("--n", type=int, default=1024)
    ap.add_argument("--a_cols", type=int, default=1024)
    ap.add_argument("--alpha", type=float, default=1.0)
    ap.add_argument("--beta", type=float, default=1.0)
    ap.add_argument("--iterations", type=int, default=20)
    ap.add_argument("--reference-check", dest="reference_check", type=_bool, default=False)
    ap.add_argument("--fp16-out", action="store_true", help="fp16 C/D instead of the reference's fp32")
    ap.add_argument("--sweep", action="store_true", help="the reference's square sweep, 30 iterations each")
    ap.add_argument("--layer", action="store_true", help="time the linear layer's form (token-major x and y, bias) instead")
    ap.add_argument("--json", default=None, metavar="PATH", help="also write the rows as a JSON list to PATH")
    ap.add_argument("--csv", default=None, metavar="PATH", help="also write the rows as CSV to PATH")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("this benchmark needs a GPU")
    dtype = torch.float16 if args.fp16_out else torch.float32
    shapes = [(s, s, s) for s in SWEEP] if args.sweep else [(args.a_rows, args.n, args.a_cols)]
    iterations = 30 if args.sweep else args.iterations
    print("| a_rows |   n   | a_cols |    GFLOPs    | Runtime (ms) |" + (" check |" if args.reference_check else ""))
    print("|--------|-------|--------|--------------|--------------|" + ("-------|" if args.reference_check else ""))
    ok = True
    rows = []
    for (m, n, k) in shapes:
        if args.layer:
            ms, gflops, passed = run_layer(m, n, k, iterations, args.reference_check)
        else:
            ms, gflops, passed = run(m, n, k, args.alpha, args.beta, iterations, args.reference_check, dtype)
        line = f"| {m:6d} | {n:5d} | {k:6d} | {gflops:12.1f} | {ms:12.6f} |"
        if passed is not None:
            line += " Passed |" if passed else " FAILED |"
            ok = ok and passed
        print(line, flush=True)
        rows.append(dict(a_rows=m, n=n, a_cols=k, gflops=gflops, runtime_ms=ms, alpha=args.alpha, beta=args.beta,
                         iterations=iterations, out_dtype="fp16" if args.fp16_out or args.layer else "fp32", check=passed,
                         form="layer" if args.layer else "gemm"))
    if args.json:
        import json
        with open(args.json, "w") as fh:
            json.dump(rows, fh, indent=1)
    if args.csv:
        import csv
        with open(args.csv, "w", newline="") as fh:
            writer = csv.DictWriter(fh, fieldnames=list(rows[0].keys()))
            writer.writeheader()
            writer.writerows(rows)
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
