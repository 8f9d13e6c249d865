"""Replay a trace of token steps through a served language model and write the logits that are asked for.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N  < steps.jsonl

Each input line is one step: {"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}], "end": [ids]}.  An entry
continues the request `id` (or starts it) with its next tokens on the cache and state earlier steps left; `want` lists the places
among these tokens whose logits are written, for all entries in order, to OUT/<n>.f32 (little-endian fp32 [wanted, vocab]).
Requests named in `end` give their cache sequence back after the step.  `done <n>` is printed after every step.

The model class comes from config.json through the framework's registry (`infer.load_model`); the step runs the served path:
`decoder.forward_spans` (mn_seq_step, mn_pmix_step, mn_hyb_step or mn_pn_step), the decoder's arenas and states and `sequences.SequenceSlots`.  Nothing is sampled.
--dtype bfloat16 is the serving arithmetic (bf16 MFMA products above 8 rows, fp32 elsewhere), float32 is fp32 FMA everywhere.
"""
import argparse
import json
import os
import sys

import numpy as np


def replay(model, out_dir, lines, emit):
    import torch
    dec, slots = model.dec, model.slots
    live = {}                                              # request id -> cache sequence
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        spans, toks, want = [], [], []
        r0 = 0
        for e in step.get("entries", []):
            n = len(e["tokens"])
            if n == 0:
                continue
            if e["id"] not in live:
                live[e["id"]] = slots.alloc()
            seq = live[e["id"]]
            past = slots.length[seq]
            if past + n > dec.t_max:
                raise ValueError(f"request {e['id']}: {past + n} tokens exceed the cache (t_max = {dec.t_max}; raise --max-tokens)")
            spans.append((seq, n, past))
            toks += [int(t) for t in e["tokens"]]
            want += [r0 + int(w) for w in e.get("want", [])]
            slots.length[seq] = past + n
            r0 += n
        if spans:
            ids = torch.tensor(toks, dtype=torch.long, device=dec.device)
            hidden = dec.forward_spans(dec.embed(ids), spans, tokens=ids)
            if want:
                rows = hidden[torch.tensor(want, dtype=torch.long, device=dec.device)]
                logits = dec.logits(rows).cpu().numpy().astype("<f4")
                tmp = os.path.join(out_dir, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(logits).tobytes())
                os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
            else:
                torch.cuda.synchronize()
        for rid in step.get("end", []):
            if rid in live:
                slots.release(live.pop(rid))
        emit(f"done {step['step']}")


def main(argv=None):
    ap = argparse.ArgumentParser(description="feed token steps through a served model and write the requested logits")
    ap.add_argument("--model", required=True, help="directory with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True, help="directory for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, default=4096, help="most tokens that live requests hold at any time")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    from .infer import load_model
    model = load_model(a.model, dtype={"bfloat16": "bf16", "float32": "f32"}[a.dtype], t_max=max(1, a.max_tokens))
    if not hasattr(model, "slots"):
        print("this model has no token-step interface", file=sys.stderr)
        return 4

    def emit(s):
        sys.stdout.write(s + "\n")
        sys.stdout.flush()

    replay(model, a.out, sys.stdin, emit)
    return 0


if __name__ == "__main__":
    sys.exit(main())
