"""ek-benchmark's batch scan for the HIP backend.

Mirrors ek-benchmark (the reference's only perf harness on this path): build N experts with
random weights (ek-benchmark/src/main.rs:88-101), time `exp.forward(exp.rand_input(batch))`
for every batch size (Benchmarker::scan_batch, ek-benchmark/src/bench.rs:36-52,75-107) and
write one row per call with the reference's columns (bench.rs:109-118) as parquet.  Defaults
are the reference's (hidden 7168, intermediate 2048, 8 experts, batches 1..256).

`--backend torch` runs the reference's own four ops (ffn/expert_torch.rs:81-84) with libtorch on
the host cores, for a number beside it on the same machine.

    python -m ek_hip.scan_batch --iterations 4            # from expert-kit_amd/
"""
from __future__ import annotations

import argparse
import os
import time

import torch

from . import EKInstance, ExpertWeight, HipFFN

COLUMNS = ["experiment_id", "iteration", "batch_size", "expert_id", "elapsed_micros", "input_dim", "hidden_dim",
           "backend"]


class TorchCpuFFN:
    """TorchFFN's closure on the host (ffn/expert_torch.rs:58-91): weights cast to bf16 once."""

    def __init__(self, hidden, inter, w: ExpertWeight):
        self.hidden, self.inter = hidden, inter
        self.w1, self.w3, self.w2 = (t.to(torch.bfloat16) for t in (w.up_w, w.gate_w, w.down_w))

    def backend(self):
        return "torch"

    def rand_input(self, batch):
        return torch.rand(batch, self.hidden, dtype=torch.bfloat16)

    def forward(self, x):
        up, gate = x @ self.w1.t(), x @ self.w3.t()
        return (up * torch.nn.functional.silu(gate)) @ self.w2.t()


def scan_batch(experts, batch_sizes, iterations, repeats, device_input):
    rows = []
    for exp in experts:                                       # warm up all experts (bench.rs:81-84)
        exp.forward(exp.rand_input(1))
    for experiment_id in range(repeats):
        for it in range(iterations):
            for batch in batch_sizes:
                for eidx, exp in enumerate(experts):
                    x = exp.rand_input(batch)
                    if device_input:
                        x = x.cuda()
                        torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    y = exp.forward(x)
                    if y.is_cuda:
                        torch.cuda.synchronize()
                    us = (time.perf_counter() - t0) * 1e6
                    rows.append((experiment_id, it, batch, eidx, int(us), exp.hidden, exp.inter, exp.backend()))
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--backend", choices=["hip", "torch"], default="hip")
    ap.add_argument("--batch-sizes", default="1,2,4,8,16,32,64,128,256")
    ap.add_argument("-i", "--intermediate-dim", type=int, default=2048)
    ap.add_argument("--hidden-dim", type=int, default=7168)
    ap.add_argument("-e", "--experts", type=int, default=8)
    ap.add_argument("--iterations", type=int, default=4)
    ap.add_argument("-r", "--repeats", type=int, default=1)
    ap.add_argument("-o", "--output-dir", default="./data")
    ap.add_argument("--device-input", action="store_true",
                    help="hand the expert device-resident rows (no PCIe in the timed call)")
    args = ap.parse_args(argv)
    batch_sizes = [int(b) for b in args.batch_sizes.split(",")]
    experts = []
    for _ in range(args.experts):
        w = ExpertWeight.from_rand_linear(args.hidden_dim, args.intermediate_dim, torch.bfloat16)
        if args.backend == "hip":
            f = HipFFN.construct(EKInstance(args.hidden_dim, args.intermediate_dim), w, max_rows=max(batch_sizes))
            f.hidden, f.inter = args.hidden_dim, args.intermediate_dim
        else:
            f = TorchCpuFFN(args.hidden_dim, args.intermediate_dim, w)
        experts.append(f)
    rows = scan_batch(experts, batch_sizes, args.iterations, args.repeats, args.device_input and args.backend == "hip")
    os.makedirs(args.output_dir, exist_ok=True)
    name = f"{args.backend}_{args.intermediate_dim}_{args.hidden_dim}_{args.experts}_{int(time.time())}"
    cols = {c: [r[i] for r in rows] for i, c in enumerate(COLUMNS)}
    try:
        import pyarrow as pa
        import pyarrow.parquet as pq
        path = os.path.join(args.output_dir, name + ".parquet")
        pq.write_table(pa.table(cols), path, compression="snappy")
    except ImportError:
        path = os.path.join(args.output_dir, name + ".csv")
        with open(path, "w") as fh:
            fh.write(",".join(COLUMNS) + "\n")
            for r in rows:
                fh.write(",".join(str(v) for v in r) + "\n")
    print(f"wrote {len(rows)} rows to {path}")
    print(f"{'batch':>6} {'mean us':>10} {'min us':>10}   ({args.backend}, hidden {args.hidden_dim}, "
          f"intermediate {args.intermediate_dim}, {args.experts} experts)")
    for b in batch_sizes:
        v = [r[4] for r in rows if r[2] == b]
        print(f"{b:>6} {sum(v) / len(v):>10.1f} {min(v):>10.1f}")
    for f in experts:
        if hasattr(f, "close"):
            f.close()


if __name__ == "__main__":
    main()
