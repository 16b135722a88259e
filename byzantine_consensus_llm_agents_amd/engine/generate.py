"""Command line of the id-level generation path: prompts of token ids in, generated ids out.

    python -m byzantine_consensus_llm_agents_amd.engine.generate --weights DIR \
        --prompt "5 17 3" --prompt "9 9 2 40" --max-tokens 16 [--temperature 0.8] [--dtype float32]

For checkpoints that ship no tokenizer (the model class comes from the directory's config.json).
Every prompt goes through the engine's scheduler: admission, paged prefill, batched decode
(captured HIP graphs on the hip backend) and the sampler.  One line of ids per prompt is printed.
"""
import argparse
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--weights", required=True, help="model directory (config.json + safetensors)")
    ap.add_argument("--prompt", action="append", required=True, help="whitespace-separated token ids (repeatable)")
    ap.add_argument("--max-tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--backend", choices=("hip", "torch"), default="hip")
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--seed", type=int, default=0)
    a = ap.parse_args(argv)
    import torch
    from ..utils.build import build_kernels, build_runtime
    build_runtime()
    if a.backend == "hip":
        build_kernels()
    from .engine import EngineArgs, InferenceEngine
    prompts = [[int(t) for t in p.split()] for p in a.prompt]
    args = EngineArgs.from_configs(a.weights, backend=a.backend, weights=a.weights, seed=a.seed,
                                   dtype=getattr(torch, a.dtype), max_model_len=a.max_model_len,
                                   max_batch_seqs=max(4, min(len(prompts), 512)),
                                   kv_pool_tokens=min(len(prompts), 512) * a.max_model_len)
    engine = InferenceEngine(args)
    try:
        for out in engine.generate_ids(prompts, a.max_tokens, a.temperature):
            print(" ".join(map(str, out)))
    finally:
        engine.shutdown()
    return 0


if __name__ == "__main__":
    sys.exit(main())
