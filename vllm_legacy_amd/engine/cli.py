"""Command line of the engine.

    python -m vllm_legacy_amd.engine.cli generate --model DIR --prompt 5,17,3 [--prompt ...]
        [--max-tokens 16] [--temperature 0] [--top-k 0] [--top-p 1] [--seed N] [--dtype bfloat16]
    python -m vllm_legacy_amd.engine.cli models
    python -m vllm_legacy_amd.engine.cli trace --model DIR --dtype ... --out DIR --max-tokens N

Prompts are token ids (no tokenizer ships with the engine); `generate` prints one JSON line per
request with the generated ids.
"""
import argparse
import json
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="vllm_legacy_amd.engine.cli")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate from token-id prompts")
    g.add_argument("--model", required=True)
    g.add_argument("--prompt", action="append", required=True, help="comma-separated token ids")
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int)
    g.add_argument("--block-size", type=int, default=16)
    g.add_argument("--num-blocks", type=int, default=4096)
    g.add_argument("--max-num-seqs", type=int, default=64)
    g.add_argument("--max-num-batched-tokens", type=int, default=2048)
    sub.add_parser("models", help="list the supported architectures")
    t = sub.add_parser("trace", help="replay steps from standard input (see engine/trace_replay.py)",
                       add_help=False)
    t.add_argument("rest", nargs=argparse.REMAINDER)
    a = ap.parse_args(argv)
    if a.cmd == "models":
        from vllm_legacy_amd.model.registry import supported_architectures
        print("\n".join(supported_architectures()))
        return 0
    if a.cmd == "trace":
        from vllm_legacy_amd.engine.trace_replay import main as trace_main
        return trace_main(a.rest)
    import torch

    from vllm_legacy_amd.engine import EngineConfig, LLMEngine, SamplingParams
    dtype = torch.bfloat16 if a.dtype == "bfloat16" else torch.float32
    engine = LLMEngine.from_pretrained(
        a.model, dtype, EngineConfig(a.block_size, a.num_blocks, a.max_num_seqs, a.max_num_batched_tokens))
    prompts = [[int(x) for x in p.split(",") if x.strip()] for p in a.prompt]
    params = SamplingParams(a.max_tokens, a.temperature, a.top_k, a.top_p, a.seed)
    for out in engine.generate(prompts, params):
        print(json.dumps({"request_id": out.request_id, "token_ids": out.token_ids,
                          "finish_reason": out.finish_reason}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
