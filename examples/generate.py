"""Generate with a model folder and show prefix-cache reuse. Short on purpose.

    python examples/generate.py --model DIR [--max-tokens 32] [--dtype bfloat16] [--prompt-ids 1,2,3 ...]
    python examples/generate.py --random Qwen3ForCausalLM:hidden_size=256,num_hidden_layers=2,... --seed 1 \
        --random-prompts 4x50

The command line of the reference (``examples/generate.py:26-49``) with its two options kept
(``--device``, ``--max-tokens``) and what a local folder needs added. The engine sees token ids only.
Prompts are given as ids (``--prompt-ids``, repeatable), or as text (``--prompt``) when the folder
holds a ``tokenizer.json``; without either, a shared "system" prefix and three tails of seeded random
ids stand in (``--random-prompts NxLEN``: N prompts of LEN seeded random ids, the first half of each
shared). ``--random ARCH:key=value,...`` stands for ``--model``: the architecture's config.json keys
and weights drawn from ``--seed`` (the seed of the sampling draws as well). As in the reference, the first prompt runs alone and warms the prefix cache, the rest
run batched and reuse it.
"""

from __future__ import annotations

import argparse
import os
import random
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams  # noqa: E402


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    source = parser.add_mutually_exclusive_group(required=True)
    source.add_argument("--model", help="folder with config.json and *.safetensors")
    source.add_argument("--random", metavar="ARCH:key=value,...",
                        help="instead of a folder: an architecture name and its config.json keys; weights are drawn from --seed")
    parser.add_argument("--device", default="cuda", help="only 'cuda' (the one GPU) is supported")
    parser.add_argument("--max-tokens", type=int, default=32)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--num-blocks", type=int, default=128)
    parser.add_argument("--kv-memory-fraction", type=float, default=None,
                        help="size the KV pool by memory instead: the engine stays within this share of the GPU's memory")
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--max-num-seqs", type=int, default=16)
    parser.add_argument("--max-num-batched-tokens", type=int, default=2048)
    parser.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeatable")
    parser.add_argument("--prompt", action="append", default=[], help="text; needs tokenizer.json in the folder")
    parser.add_argument("--random-prompts", metavar="NxLEN", help="N prompts of LEN seeded random ids whose first half is shared")
    args = parser.parse_args()
    if args.device != "cuda":
        parser.error("this engine runs on the GPU only: --device cuda")

    if args.random:
        from mini_engine_amd.weights import random_model_folder

        args.model = random_model_folder(args.random, args.seed, args.dtype)
    tok = None
    tok_path = os.path.join(args.model, "tokenizer.json")
    if args.prompt:
        if not os.path.exists(tok_path):
            parser.error("--prompt needs tokenizer.json in the model folder; use --prompt-ids")
        from tokenizers import Tokenizer

        tok = Tokenizer.from_file(tok_path)

    engine = LLMEngine.from_pretrained(
        args.model,
        EngineConfig(dtype=args.dtype, num_blocks=args.num_blocks, kv_memory_fraction=args.kv_memory_fraction,
                     block_size=args.block_size, seed=args.seed, max_num_seqs=args.max_num_seqs,
                     max_num_batched_tokens=args.max_num_batched_tokens),
    )
    vocab = engine.model.plan.vocab_size
    if args.prompt:
        prompts = [tok.encode(p).ids for p in args.prompt]
        labels = args.prompt
    elif args.prompt_ids:
        prompts = [[int(t) for t in p.split(",")] for p in args.prompt_ids]
        labels = [" ".join(map(str, p)) for p in prompts]
    else:
        rng = random.Random(args.seed)
        count, length = 3, 0
        if args.random_prompts:
            try:
                count, length = (int(v) for v in args.random_prompts.lower().split("x"))
            except ValueError:
                parser.error("--random-prompts takes NxLEN, for instance 4x50")
            if count < 1 or length < 1:
                parser.error("--random-prompts needs at least one prompt of at least one id")
        shared = length // 2 if length else 3 * args.block_size + 5
        system = [rng.randrange(1, vocab) for _ in range(shared)]
        prompts = [system + [rng.randrange(1, vocab) for _ in range(length - shared if length else 4 + i)] for i in range(count)]
        labels = [f"<{len(system)} shared ids> + {len(p) - len(system)} ids" for p in prompts]
    params = SamplingParams(max_tokens=args.max_tokens, temperature=args.temperature)

    start = time.perf_counter()
    # The first request warms the prefix cache; the rest are batched and reuse it.
    outputs = engine.generate(prompts[:1], params) + (engine.generate(prompts[1:], params) if prompts[1:] else [])
    elapsed = time.perf_counter() - start

    for label, out in zip(labels, outputs):
        answer = tok.decode(out, skip_special_tokens=True).strip() if tok else " ".join(map(str, out))
        print(f"Q: {label}\nA: {answer}\n")
    s = engine.stats
    print(
        f"{s.generated_tokens} tokens in {elapsed:.1f}s over {s.steps} steps | "
        f"prompt tokens {s.prompt_tokens}, served from prefix cache {engine.scheduler.num_cached_tokens}"
    )


if __name__ == "__main__":
    main()
