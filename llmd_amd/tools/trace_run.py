"""Replay a trace of given token ids through the engine, step by step, and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object per line,
    {"step": 7, "entries": [{"id": "r1", "tokens": [11, 4, 90, 2], "want": [3]}, {"id": "r2", "tokens": [8], "want": []}],
     "end": ["r2"]}
(on one line)
``entries`` bring each request's next tokens (a request is admitted at its first entry and may
skip steps); ``want`` are the places among them whose logits are written; ``end`` lists the
requests finished after the step. All entries of a step run as one batch of the engine's own
step (LLMEngine.forced_step): prompt portions beside single tokens, through the scheduler's
admission, the block manager's pages and the state slots. Nothing is sampled.

For a step with wanted places it writes DIR/<step>.f32: little-endian fp32 [wanted, vocab] in
the order of the entries and their ``want``. After every step it prints ``done <step>``.

The page pool holds --max-tokens tokens (in pages of 64) and there are four state slots / live
requests, so pages and slots are reused. float32 runs every matrix product and kernel in true
32-bit. Exit code 3: float32 asked of a model class that runs in bfloat16 only.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-seqs", type=int, default=4, help="live requests / state slots")
    ap.add_argument("--device", default="cuda")
    a = ap.parse_args(argv)

    import torch

    from llmd_amd.engine.config import EngineConfig, ModelConfig
    from llmd_amd.models import model_class

    mc = ModelConfig.from_hf(a.model)
    if a.dtype == "float32" and not getattr(model_class(mc), "supports_float32", False):
        print(f"{mc.model_type} runs in bfloat16 only", file=sys.stderr)
        return 3
    if a.device.startswith("cuda") and not torch.cuda.is_available():
        print("no GPU visible (pass --device cpu for the reference ops)", file=sys.stderr)
        return 2
    from llmd_amd.engine.engine import LLMEngine

    bs = 64
    cfg = EngineConfig.create(
        a.model, model_config=mc, device=a.device, dtype=a.dtype, load_format="safetensors",
        weights_path=a.model, block_size=bs, num_gpu_blocks=max(1, -(-a.max_tokens // bs)),
        max_num_seqs=a.max_seqs, max_model_len=a.max_tokens + 1, max_num_batched_tokens=max(a.max_tokens, bs),
        enable_prefix_caching=False, async_scheduling=False, enforce_eager=True, prefill_token_align=0)
    eng = LLMEngine(cfg, capture_graphs=False)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st.get("entries", [])]
        logits = eng.forced_step(entries, st.get("end") or [])
        if logits is not None and logits.shape[0]:
            data = logits.to(torch.float32).contiguous().cpu().numpy().astype("<f4")
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
