"""Writes the GEMM kernel-selection table that recurrent_drafting_amd.gemm_tuning loads.

    python ml-recurrent-drafter_amd/tune_gemms.py [--out FILE] [--hidden 4096] [--intermediate 11008]
        [--heads 32] [--kv-heads 32] [--vocab 32000] [--drafter-exit 8192]
        [--rows 32:1536:32,4000] [--draft-rows 360,8]

For every row count it runs the model's GEMMs (fused QKV, attention output, fused gate/up, down,
lm_head; the drafter's two recurrent projections, its ResBlock and its head) once under torch's
TunableOp with tuning switched on: torch times every kernel hipBLASLt and rocBLAS offer for the
problem, with rotating buffers so that the weights always come from HBM as they do in the model,
and records the fastest.  Takes about a second per problem on an MI355X.  Needs a GPU.
"""

from __future__ import annotations

import argparse
import os
import sys
import time

import torch


def _rows(spec: str):
    out = []
    for part in spec.split(","):
        if ":" in part:
            lo, hi, step = (int(v) for v in part.split(":"))
            out += list(range(lo, hi + 1, step))
        elif part:
            out.append(int(part))
    return sorted(set(out))


def main() -> int:
    here = os.path.dirname(os.path.abspath(__file__))
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(here, "recurrent_drafting_amd", "gemm_tuning_gfx950.csv"))
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--intermediate", type=int, default=11008)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--kv-heads", type=int, default=32)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--drafter-exit", type=int, default=8192)
    ap.add_argument("--rows", default="32:1536:32,4000")
    ap.add_argument("--draft-rows", default="360,8")
    ap.add_argument("--rotating-mb", type=int, default=1024)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("tune_gemms.py: no GPU", file=sys.stderr)
        return 2
    import torch.cuda.tunable as tunable

    dev, dt = "cuda", torch.bfloat16
    head_dim = args.hidden // args.heads
    llm = [  # (out features, in features, bias)
        ((args.heads + 2 * args.kv_heads) * head_dim, args.hidden, False),
        (args.hidden, args.hidden, False),
        (2 * args.intermediate, args.hidden, False),
        (args.hidden, args.intermediate, False),
        (args.vocab, args.hidden, False),
    ]
    drafter = [
        (args.hidden, args.hidden, False), (args.hidden, args.hidden, True),
        (args.drafter_exit, args.drafter_exit, True), (args.vocab, args.drafter_exit, False),
    ]
    if os.path.exists(args.out):
        os.remove(args.out)
    tunable.enable(True)
    tunable.tuning_enable(True)
    tunable.set_filename(args.out)
    tunable.set_rotating_buffer_size(args.rotating_mb)
    t0 = time.time()
    done = 0
    for shapes, rows in ((llm, _rows(args.rows)), (drafter, _rows(args.draft_rows))):
        for n, k, bias in shapes:
            w = torch.randn(n, k, device=dev, dtype=dt) * 0.02
            b = torch.zeros(n, device=dev, dtype=dt) if bias else None
            for m in rows:
                x = torch.randn(m, k, device=dev, dtype=dt)
                torch.nn.functional.linear(x, w, b)
                torch.cuda.synchronize()
                done += 1
                if done % 20 == 0:
                    print(f"[tune_gemms] {done} problems, {time.time() - t0:.0f}s", flush=True)
            del w
    tunable.tuning_enable(False)
    results = tunable.get_results()
    print(f"[tune_gemms] {len(results)} entries in {time.time() - t0:.0f}s -> {args.out}", flush=True)
    return 0  # torch writes the file when the process ends


if __name__ == "__main__":
    sys.exit(main())
