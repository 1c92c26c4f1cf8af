"""Decode and prefill throughput of the engine on the Qwen3-0.6B shape with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line. ``value`` is decoded tokens a second at batch 8 with every sequence at the
benchmark context length; a step is one decode step of the whole engine (schedule, step function
from the cache, greedy sampling, postprocess). The same line carries the 2,048-token prefill, the
HBM roofline of the decode step, and under ``points`` decode at batch 1 and 64 and the reference's own
throughput workload (64 requests of 256 prompt and 128 output tokens through ``generate``).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def model_config():
    """Layer sizes of the Qwen3-0.6B shape (28 layers, hidden 1024, 16/8 heads of 128, 3072, 151936, tied)."""
    from mini_engine_amd.models.qwen3 import Qwen3Config

    return Qwen3Config(vocab_size=151936, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28,
                       num_attention_heads=16, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-6,
                       rope_theta=1e6, max_position_embeddings=40960, tie_word_embeddings=True)


def prefill_flops(cfg, tokens: int) -> float:
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * cfg.hidden_size
    o = cfg.num_attention_heads * cfg.head_dim * cfg.hidden_size
    mlp = 3 * cfg.hidden_size * cfg.intermediate_size
    linear = 2.0 * tokens * cfg.num_hidden_layers * (qkv + o + mlp)
    attention = cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * tokens * tokens / 2
    head = 2.0 * cfg.vocab_size * cfg.hidden_size
    return linear + attention + head


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--skip-prefill", action="store_true", help="profiling aid: do not measure the prefill")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on one GPU)")
        return 2

    import torch

    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.sequence import Sequence

    cfg = model_config()
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    block = 16
    ctx, k, w = args.context, args.steps, args.warmup
    budget = 8192

    def prompt_len_for(batch):
        """Prompts are sized so that every sequence is still decoding, and within the context
        length, when the timed steps end: the first sequences decode while the later ones are still
        being prefilled under the token budget."""
        prefill_steps = -(-batch * ctx // budget) + 1
        n = ctx - (k + w + prefill_steps) - 2
        if n < 1:
            raise SystemExit("context is too short for this many steps")
        return n, prefill_steps
    blocks_per_seq = -(-ctx // block)
    econf = EngineConfig(block_size=block, num_blocks=max_batch * blocks_per_seq + 256, max_num_seqs=max_batch,
                         max_num_batched_tokens=budget, max_model_len=ctx, enable_prefix_caching=False,
                         dtype=args.dtype, seed=0, cuda_graphs=True)
    engine = LLMEngine.from_random("Qwen3ForCausalLM", cfg, econf, seed=0)
    gen = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(100, cfg.vocab_size, (n,), generator=gen).tolist()

    # ---- prefill of one whole prompt through the step function
    def prefill_once(n):
        seq = Sequence(prompt(n))
        assert engine.block_manager.try_allocate(seq, n)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.runner.step([StepItem(seq, seq.token_ids, 0, [n - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.block_manager.free(seq)
        return dt

    prefill = None
    if not args.skip_prefill:
        prefill_once(args.prefill_tokens)
        prefill_s = min(prefill_once(args.prefill_tokens) for _ in range(3))
        pf = prefill_flops(cfg, args.prefill_tokens)
        prefill = {"value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens,
                   "ms": round(prefill_s * 1e3, 3), "frac": round(pf / prefill_s / PEAK_FLOPS[args.dtype], 4)}

    # ---- decode: B sequences at the benchmark context, K timed engine steps
    kv_per_token = engine.runner.storage.kv_bytes_per_token()
    weight_bytes = engine.model.weight_bytes()

    def decode(batch):
        prompt_len, prefill_steps = prompt_len_for(batch)
        params = SamplingParams(max_tokens=k + w + prefill_steps + 2, temperature=0.0, ignore_eos=True)
        seqs = [engine.add_request(prompt(prompt_len), params) for _ in range(batch)]
        while any(s.num_output_tokens == 0 for s in seqs):
            engine.step()
        for _ in range(w - 1):
            engine.step()
        torch.cuda.synchronize()
        tokens_before = sum(len(s) for s in seqs)
        t0 = time.perf_counter()
        for _ in range(k):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens_after = sum(len(s) for s in seqs)
        live = sum(not s.is_finished for s in seqs)
        if live != batch or tokens_after - tokens_before != batch * k:
            raise SystemExit(f"batch {batch}: only {live} sequences were decoding through the timed steps "
                             f"({tokens_after - tokens_before} tokens instead of {batch * k})")
        while engine.scheduler.has_unfinished():
            engine.step()
        ms = dt / k * 1e3
        step_bytes = weight_bytes + (tokens_before + tokens_after) / 2 * kv_per_token
        return (tokens_after - tokens_before) / dt, ms, step_bytes / (dt / k) / 1e9

    def reference_workloads():
        """The reference's own two serving workloads, with its engine options (benchmarks/bench.py:52-62,
        :86-93, :113-123: pages of 16, 2,048 pages, 64 sequences, 8,192 tokens a step, prefix cache on).
        Throughput: 64 requests of 256 random prompt ids and 128 greedy output tokens, all submitted at
        once. Shared prefix: 64 requests of a common 512-token prefix and 32 tokens of their own, 64
        output tokens, the first request run alone so that the others find its pages. Output tokens
        over the wall time of the whole run, prefill and scheduling included."""
        ref = LLMEngine.from_random("Qwen3ForCausalLM", cfg, EngineConfig(
            block_size=16, num_blocks=2048, max_num_seqs=64, max_num_batched_tokens=8192, max_model_len=2048,
            enable_prefix_caching=True, dtype=args.dtype, seed=0, cuda_graphs=True), seed=0)
        ref.runner.capture_all()

        def timed(run):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = run()
            torch.cuda.synchronize()
            return sum(len(o) for o in outs) / (time.perf_counter() - t0)

        params = SamplingParams(max_tokens=128, temperature=0.0, ignore_eos=True)
        ref.generate([prompt(256) for _ in range(2)], params)  # code objects, the GEMM library's plans
        prompts = [prompt(256) for _ in range(64)]
        throughput = timed(lambda: ref.generate(prompts, params))
        ref.block_manager.reset_prefix_cache()
        shared = prompt(512)
        prompts = [shared + prompt(32) for _ in range(64)]
        params = SamplingParams(max_tokens=64, temperature=0.0, ignore_eos=True)
        cached_before = ref.scheduler.num_cached_tokens
        prefix = timed(lambda: ref.generate(prompts[:1], params) + ref.generate(prompts[1:], params))
        assert ref.scheduler.num_cached_tokens - cached_before == 63 * 512, "the shared prefix was not served from the cache"
        return throughput, prefix

    tok_s, ms_per_step, gbs = decode(args.batch)
    measured = {b: decode(b) for b in points}
    pts = {f"decode_b{b}": round(m[0], 1) for b, m in measured.items()}
    # the same bound as `roofline`, for the other batch sizes: bytes a step must read / its time / the HBM peak
    pts_frac = {f"decode_b{b}": round(m[2] / HBM_PEAK_GBS, 4) for b, m in measured.items()}
    if max_batch >= 64:
        throughput, prefix = reference_workloads()
        pts["throughput_64x256in_128out"] = round(throughput, 1)
        pts["shared_prefix_64x544in_64out"] = round(prefix, 1)
    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-0.6B shape)", "value": round(tok_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": k, "warmup": w, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, random N(0, 0.02) weights",
        "config": {"model": "Qwen3-0.6B shape", "layers": cfg.num_hidden_layers, "layers_of_config": 28,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                   "tied_head": cfg.tie_word_embeddings, "global_batch": args.batch, "seq_len": ctx,
                   "block_size": block, "graphs": econf.cuda_graphs, "parallelism": "single GPU"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4)},
        "points": pts,
        "points_roofline_frac": pts_frac,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
