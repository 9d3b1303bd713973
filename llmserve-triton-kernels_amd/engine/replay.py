"""Trace replay: feeds given token ids through a model step by step and writes logits.
It samples nothing and has no forward pass, cache or loader of its own: it drives the
`ModelRunner` that generation uses.

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
All entries of a step run as one batch.  For a step in which something is wanted the logits
at the wanted places, in the order of the entries and of `want`, are written to
`<out>/<step>.f32` as little-endian 32-bit floats [wanted, vocab].  After every step a line
`done <step>` is printed and flushed.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


class Replayer:
    """Applies trace records to a `ModelRunner`; `run` returns the wanted logits of one step."""

    def __init__(self, runner):
        self.runner = runner

    def run(self, record: dict):
        from .runner import StepEntry

        entries = []
        for e in record.get("entries", []):
            if not self.runner.manager.has_sequence(e["id"]):
                self.runner.add_sequence(e["id"])
            entries.append(StepEntry(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = self.runner.step(entries)
        for seq_id in record.get("end", []):
            if self.runner.manager.has_sequence(seq_id):
                self.runner.free_sequence(seq_id)
        return logits


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--block-size", type=int, default=16, help="tokens in a cache page")
    ap.add_argument("--max-seqs", type=int, default=8, help="most requests alive at once")
    args = ap.parse_args(argv)

    import numpy as np

    from ..config.engine_config import EngineConfig
    from .runner import ModelRunner

    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    if args.max_tokens < 1:
        ap.error("--max-tokens must be positive")
    num_blocks = -(-args.max_tokens // args.block_size)
    engine_config = EngineConfig(dtype=args.dtype, block_size=args.block_size, num_blocks=num_blocks,
                                 max_num_seqs=args.max_seqs)
    replayer = Replayer(ModelRunner.from_folder(args.model, engine_config))

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        logits = replayer.run(record)
        if logits.shape[0] > 0:
            np.ascontiguousarray(logits.cpu().numpy().astype("<f4")).tofile(out_dir / f"{record['step']}.f32")
        print(f"done {record['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
