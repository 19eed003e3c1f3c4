"""Trace replay: feeds given token ids through the engine's model runner step by step and writes
the logits asked for.  The steps come from standard input instead of from the scheduler; the
cache manager, the runner's step function, the model and its kernels are the engine's.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--max-seqs 4]

One JSON object a line:  {"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}],
"end": [ids]}.  A step with wanted positions writes OUT/<n>.f32 (fp32 little-endian
[wanted, vocab], in the order of entries and of `want`); every step answers `done <n>`.
"""
import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the live requests hold at most (each rounded up to 64)")
    ap.add_argument("--max-seqs", type=int, default=4, help="requests live at any time")
    ap.add_argument("--block-size", type=int, default=16)
    a = ap.parse_args(argv)
    if 64 % a.block_size != 0:
        ap.error("--block-size must divide 64")

    import torch

    from vllm_legacy_amd import _lib
    from vllm_legacy_amd.engine.cache_manager import CacheManager
    from vllm_legacy_amd.engine.model_runner import ModelRunner
    from vllm_legacy_amd.model.registry import load_model

    _lib.seq_lib()      # compiles the kernels on a first call in a fresh checkout
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    torch.backends.cuda.matmul.allow_tf32 = False
    torch.set_float32_matmul_precision("highest")
    device = torch.device("cuda", 0)
    model = load_model(a.model, dtype, device)
    num_blocks = (a.max_tokens + a.block_size - 1) // a.block_size
    cache = CacheManager(num_blocks, a.block_size, a.max_seqs)
    runner = ModelRunner(model, cache, device)
    os.makedirs(a.out, exist_ok=True)
    computed = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries, want = [], []
        for e in step["entries"]:
            sid, tokens = e["id"], list(e["tokens"])
            if not cache.is_live(sid):
                cache.admit(sid)
                computed[sid] = 0
            cache.grow(sid, computed[sid] + len(tokens))
            entries.append((sid, tokens, computed[sid]))
            want.append(list(e.get("want", [])))
        if entries:
            logits = runner.execute(entries, want)
            for sid, tokens, _ in entries:
                computed[sid] += len(tokens)
            if logits is not None:
                data = logits.to(torch.float32).contiguous().cpu().numpy().astype("<f4")
                tmp = os.path.join(a.out, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(data.tobytes())
                os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
            else:
                torch.cuda.synchronize()
        for sid in step.get("end", []):
            if cache.is_live(sid):
                cache.free(sid)
                computed.pop(sid, None)
        sys.stdout.write(f"done {step['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
