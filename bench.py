"""Decode and prefill throughput of the engine with random weights, one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 0.6b|8b|32b]

Prints ONE JSON line. With the default shape (Qwen3-0.6B layer sizes) ``value`` is decoded tokens a
second at batch 8 with every sequence at the benchmark context length; a step is one decode step of
the whole engine (schedule, step function from the cache, greedy sampling, postprocess). The same
line carries the 2,048-token prefill, the HBM roofline of the decode step, the host's phases of a
step, the rates a probe kernel measures on this GPU, and under ``points``: decode at batch 1 and 64
at that context, decode at batch 1/8/64 behind 2,048-token prompts with 256 generated tokens each,
decode at batch 8 behind 16,384 and 32,768 tokens, prompts of 8,192 and 32,704 tokens, one float32 point, the reference's
own two serving workloads, the serving workloads of the 8B and 32B shapes, and decode steps (batch 1/8/64) and a prefill of
the 1.7B, 8B and 32B shapes. ``--shape 8b`` / ``--shape 32b`` print that shape's workload as a line of its own,
with its prefill and the roofline of its decode step.
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Published MI355X peaks: HBM3E bandwidth, dense matrix-core rates.
HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

SHAPES = {
    "0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, intermediate_size=3072,
                 tie_word_embeddings=True, max_position_embeddings=40960),
    "8b": dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=12288,
               tie_word_embeddings=False, max_position_embeddings=40960),
    "32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, intermediate_size=25600,
                tie_word_embeddings=False, max_position_embeddings=40960),
    # a shape between the measured ones (Qwen3-1.7B's layer sizes): its products fall between the thresholds of the kernel choice
    "1.7b": dict(num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, num_key_value_heads=8, intermediate_size=6144,
                 tie_word_embeddings=True, max_position_embeddings=40960),
}
SHAPE_NAMES = {"0.6b": "Qwen3-0.6B shape", "1.7b": "Qwen3-1.7B shape", "8b": "Qwen3-8B shape", "32b": "Qwen3-32B shape"}
SHAPE_CONTEXT = {"1.7b": 2304, "8b": 2304, "32b": 640}  # near the context of the shape's serving workload


def model_config(shape: str = "0.6b"):
    """Layer sizes of the Qwen3 dense shapes (head size 128, vocabulary 151,936, rope theta 1e6, eps 1e-6)."""
    from mini_engine_amd.models.qwen3 import Qwen3Config

    return Qwen3Config(vocab_size=151936, head_dim=128, rms_norm_eps=1e-6, rope_theta=1e6, **SHAPES[shape])


def prefill_flops(cfg, tokens: int) -> float:
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim * cfg.hidden_size
    o = cfg.num_attention_heads * cfg.head_dim * cfg.hidden_size
    mlp = 3 * cfg.hidden_size * cfg.intermediate_size
    linear = 2.0 * tokens * cfg.num_hidden_layers * (qkv + o + mlp)
    attention = cfg.num_hidden_layers * 4.0 * cfg.num_attention_heads * cfg.head_dim * tokens * tokens / 2
    head = 2.0 * cfg.vocab_size * cfg.hidden_size
    return linear + attention + head


def flat_config(cfg, name: str, **extra) -> dict:
    return {"model": name, "layers": cfg.num_hidden_layers, "layers_of_config": cfg.num_hidden_layers,
            "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "tied_head": cfg.tie_word_embeddings, **extra}


def synchronize():
    import torch

    torch.cuda.synchronize()


def release() -> None:
    """Give the memory of engines that are no longer referenced back to the device."""
    import torch

    gc.collect()
    torch.cuda.empty_cache()


def measured_peaks() -> dict:
    """What probe kernels reach on this GPU: GB/s of a kernel that streams 4 GiB once, TFLOP/s of the
    bfloat16 16x16x32 matrix-core instruction issued from registers on every compute unit."""
    import torch

    from mini_engine_amd.ops import kernels as K

    buf = torch.empty(1 << 30, dtype=torch.int32, device="cuda").fill_(1)
    word, fword = torch.zeros(1, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.float32, device="cuda")
    best_read = best_mfma = 0.0
    for _ in range(4):
        synchronize()
        t0 = time.perf_counter()
        K.probe_read(buf, word)
        synchronize()
        best_read = max(best_read, buf.numel() * 4 / (time.perf_counter() - t0) / 1e9)
    for _ in range(4):
        synchronize()
        t0 = time.perf_counter()
        flops = K.probe_mfma(2048, 20000, fword)
        synchronize()
        best_mfma = max(best_mfma, flops / (time.perf_counter() - t0) / 1e12)
    del buf
    return {"hbm_read_GBs": round(best_read, 1), "mfma_bf16_TFs": round(best_mfma, 1)}


class DecodeBench:
    """An engine of one shape and dtype at a fixed context length, for decode steps at several batch
    sizes and whole-prompt prefills."""

    def __init__(self, cfg, dtype: str, ctx: int, max_batch: int, budget: int = 8192, block: int = 16, seed: int = 0):
        import torch

        from mini_engine_amd import EngineConfig, LLMEngine

        self.cfg, self.dtype, self.ctx, self.budget, self.block = cfg, dtype, ctx, budget, block
        blocks_per_seq = -(-ctx // block)
        self.econf = EngineConfig(block_size=block, num_blocks=max_batch * blocks_per_seq + 256, max_num_seqs=max_batch,
                                  max_num_batched_tokens=budget, max_model_len=ctx, enable_prefix_caching=False,
                                  dtype=dtype, seed=0, cuda_graphs=True)
        self.engine = LLMEngine.from_random("Qwen3ForCausalLM", cfg, self.econf, seed=seed)
        self.gen = torch.Generator().manual_seed(0)
        self.kv_per_token = self.engine.runner.storage.kv_bytes_per_token()
        self.weight_bytes = self.engine.model.weight_bytes()

    def prompt(self, n: int) -> list[int]:
        import torch

        return torch.randint(100, self.cfg.vocab_size, (n,), generator=self.gen).tolist()

    def prefill(self, tokens: int) -> dict:
        """One whole prompt through the step function: best of three after a warm-up."""
        from mini_engine_amd.engine.batch import StepItem
        from mini_engine_amd.engine.sequence import Sequence

        engine = self.engine

        def once():
            seq = Sequence(self.prompt(tokens))
            assert engine.block_manager.try_allocate(seq, tokens)
            synchronize()
            t0 = time.perf_counter()
            engine.runner.step([StepItem(seq, seq.token_ids, 0, [tokens - 1])])
            synchronize()
            dt = time.perf_counter() - t0
            engine.block_manager.free(seq)
            return dt

        once()
        s = min(once() for _ in range(3))
        return {"value": round(tokens / s, 1), "tokens": tokens, "ms": round(s * 1e3, 3),
                "frac": round(prefill_flops(self.cfg, tokens) / s / PEAK_FLOPS[self.dtype], 4)}

    def decode(self, batch: int, steps: int, warmup: int, prompt_len: int | None = None, phases: bool = False):
        """``steps`` timed decode steps of ``batch`` sequences. Without ``prompt_len`` the prompts are
        sized so that every sequence sits just below the context length through the timed steps (the
        first sequences decode while the later ones are still being prefilled under the token budget).
        Returns (tokens/s, ms per step, GB/s of the bytes a step must read, phases in ms per step)."""
        from mini_engine_amd import SamplingParams

        engine, k, w = self.engine, steps, warmup
        prefill_steps = -(-batch * (prompt_len or self.ctx) // self.budget) + 1
        if prompt_len is None:
            prompt_len = self.ctx - (k + w + prefill_steps) - 4
            if prompt_len < 1:
                raise SystemExit("context is too short for this many steps")
        params = SamplingParams(max_tokens=k + w + prefill_steps + 4, temperature=0.0, ignore_eos=True)
        seqs = [engine.add_request(self.prompt(prompt_len), params) for _ in range(batch)]
        while any(s.num_output_tokens == 0 for s in seqs):
            engine.step()
        for _ in range(w - 1):
            engine.step()
        synchronize()
        tokens_before = sum(len(s) for s in seqs)
        engine.time_phases = phases
        if phases:
            engine.step()  # settles a step that was launched ahead, untimed
            synchronize()
            tokens_before = sum(len(s) for s in seqs)
        before = dict(engine.stats.phase_seconds)
        t0 = time.perf_counter()
        for _ in range(k):
            engine.step()
        synchronize()
        dt = time.perf_counter() - t0
        engine.time_phases = False
        tokens_after = sum(len(s) for s in seqs)
        live = sum(not s.is_finished for s in seqs)
        if live != batch or tokens_after - tokens_before != batch * k:
            raise SystemExit(f"batch {batch}: only {live} sequences were decoding through the timed steps "
                             f"({tokens_after - tokens_before} tokens instead of {batch * k})")
        while engine.scheduler.has_unfinished():
            engine.step()
        step_bytes = self.weight_bytes + (tokens_before + tokens_after) / 2 * self.kv_per_token
        spent = {p: round((v - before[p]) / k * 1e3, 4) for p, v in engine.stats.phase_seconds.items()}
        return (tokens_after - tokens_before) / dt, dt / k * 1e3, step_bytes / (dt / k) / 1e9, spent


def reference_workloads(cfg, dtype: str, prompt) -> tuple[float, float]:
    """The reference's own two serving workloads, with its engine options (benchmarks/bench.py:52-62,
    :86-93, :113-123: pages of 16, 2,048 pages, 64 sequences, 8,192 tokens a step, prefix cache on).
    Throughput: 64 requests of 256 random prompt ids and 128 greedy output tokens, all submitted at
    once. Shared prefix: 64 requests of a common 512-token prefix and 32 tokens of their own, 64
    output tokens, the first request run alone so that the others find its pages. Output tokens
    over the wall time of the whole run, prefill and scheduling included."""
    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    ref = LLMEngine.from_random("Qwen3ForCausalLM", cfg, EngineConfig(
        block_size=16, num_blocks=2048, max_num_seqs=64, max_num_batched_tokens=8192, max_model_len=2048,
        enable_prefix_caching=True, dtype=dtype, seed=0, cuda_graphs=True), seed=0)
    ref.runner.capture_all()

    def timed(run):
        synchronize()
        t0 = time.perf_counter()
        outs = run()
        synchronize()
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


def serving_workload(shape: str, dtype: str = "bfloat16") -> dict:
    """The serving workload of a larger shape, through ``generate``.

    8b: 64 requests with prompt lengths uniform in [128, 2048] and 128 greedy output tokens each,
    continuous batching with chunked prefill under an 8,192-token step budget (the workload of the
    reference's ``benchmarks/bench.py:56-62, 113-123`` at this shape). 32b: 64 requests of a shared
    512-token prefix and 32 tokens of their own, 64 greedy output tokens, the first request run alone
    so that the prefix cache is warm (``benchmarks/bench.py:86-93``), at a 4,096-token context limit.
    Output tokens over the wall time of the whole run, prefill and scheduling included."""
    import torch

    from mini_engine_amd import EngineConfig, LLMEngine, SamplingParams

    cfg = model_config(shape)
    rng = random.Random(0)
    gen = torch.Generator().manual_seed(1)

    def prompt(n):
        return torch.randint(100, cfg.vocab_size, (n,), generator=gen).tolist()

    if shape == "8b":
        lengths = [rng.randint(128, 2048) for _ in range(64)]
        out_tokens, max_len, caching = 128, 2048 + 128, False
        pages = sum(-(-(n + out_tokens) // 16) for n in lengths) + 64
    else:
        lengths = [544] * 64
        out_tokens, max_len, caching = 64, 4096, True
        pages = 64 * -(-(544 + out_tokens) // 16) + 64
    engine = LLMEngine.from_random("Qwen3ForCausalLM", cfg, EngineConfig(
        block_size=16, num_blocks=pages, max_num_seqs=64, max_num_batched_tokens=8192, max_model_len=max_len,
        enable_prefix_caching=caching, dtype=dtype, seed=0, cuda_graphs=True), seed=0)
    engine.runner.capture_all()
    params = SamplingParams(max_tokens=out_tokens, temperature=0.0, ignore_eos=True)
    engine.generate([prompt(300), prompt(40)], SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True))  # warm-up
    engine.block_manager.reset_prefix_cache()
    if shape == "8b":
        prompts = [prompt(n) for n in lengths]
        run = lambda: engine.generate(prompts, params)
    else:
        shared = prompt(512)
        prompts = [shared + prompt(32) for _ in range(64)]
        run = lambda: engine.generate(prompts[:1], params) + engine.generate(prompts[1:], params)
    steps0, pre0, cached0 = engine.stats.steps, engine.scheduler.num_preemptions, engine.scheduler.num_cached_tokens
    synchronize()
    t0 = time.perf_counter()
    outs = run()
    synchronize()
    dt = time.perf_counter() - t0
    result = {"tok_s": round(sum(len(o) for o in outs) / dt, 1), "seconds": round(dt, 3), "steps": engine.stats.steps - steps0,
              "preemptions": engine.scheduler.num_preemptions - pre0,
              "cached_tokens": engine.scheduler.num_cached_tokens - cached0, "prompt_tokens": sum(lengths)}
    if shape == "32b":
        assert result["cached_tokens"] == 63 * 512, "the shared prefix was not served from the cache"
    del engine, run
    release()
    return result


def shape_points(shape: str, dtype: str, steps: int, warmup: int, prefill_tokens: int = 2048) -> dict:
    """Decode steps at batch 64, 1 and 8 near the context of the shape's serving workload, and one prefill: what a
    shape other than the headline's adds to a line. Returns the numbers of the batch-64 step beside the points."""
    cfg = model_config(shape)
    ctx = SHAPE_CONTEXT[shape]
    bench = DecodeBench(cfg, dtype, max(ctx, prefill_tokens + 16), 64)
    prefill = bench.prefill(prefill_tokens)

    def decode(batch):  # the sequences reach `ctx` at the end of the timed steps, whatever the engine's limit is
        return bench.decode(batch, steps, warmup, prompt_len=ctx - (steps + warmup + -(-batch * ctx // bench.budget) + 5))

    tok_s, ms, gbs, _ = decode(64)
    points, fracs = {"decode_b64": round(tok_s, 1)}, {"decode_b64": round(gbs / HBM_PEAK_GBS, 4)}
    for b in (1, 8):
        m = decode(b)
        points[f"decode_b{b}"], fracs[f"decode_b{b}"] = round(m[0], 1), round(m[2] / HBM_PEAK_GBS, 4)
    bench.engine = None
    del bench
    release()
    return {"cfg": cfg, "ctx": ctx, "prefill": prefill, "ms": ms, "gbs": gbs, "points": points, "fracs": fracs}


def shape_line(shape: str, args) -> dict:
    """The line of ``--shape 8b|32b``: the shape's serving workload as ``value``, plus the 2,048-token
    prefill and the HBM roofline of a decode step at batch 64 near that workload's context."""
    work = serving_workload(shape, args.dtype)
    sp = shape_points(shape, args.dtype, args.steps, args.warmup, args.prefill_tokens)
    cfg, ctx, prefill, ms, gbs, points, fracs = (sp[k] for k in ("cfg", "ctx", "prefill", "ms", "gbs", "points", "fracs"))
    name = SHAPE_NAMES[shape]
    what = {"8b": "64 requests, prompts uniform in [128, 2048], 128 output tokens, 8,192-token step budget",
            "32b": "64 requests of a shared 512-token prefix + 32 tokens, 64 output tokens, prefix cache warm"}[shape]
    return {
        "metric": f"output tok/s, {what} ({name})", "value": work["tok_s"], "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, random N(0, 0.02) weights",
        "config": flat_config(cfg, name, global_batch=64, seq_len=ctx, block_size=16, graphs=True, parallelism="single GPU"),
        "workload": work, "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4)},
        "points": points, "points_roofline_frac": fracs,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", default="0.6b", choices=["0.6b", "8b", "32b"])
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--points", default="1,64", help="other batch sizes to measure, comma separated ('' for none)")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--skip-prefill", action="store_true", help="profiling aid: do not measure the prefill")
    ap.add_argument("--skip-extras", action="store_true",
                    help="profiling aid: only the decode steps and the prefill (no serving workloads, no float32 point, no probes)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on one GPU)")
        return 2
    if args.shape != "0.6b":
        print(json.dumps(shape_line(args.shape, args)))
        return 0

    cfg = model_config()
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    k, w = args.steps, args.warmup
    bench = DecodeBench(cfg, args.dtype, args.context, max_batch)
    prefill = None if args.skip_prefill else bench.prefill(args.prefill_tokens)
    tok_s, ms_per_step, gbs, _ = bench.decode(args.batch, k, w)
    measured = {b: bench.decode(b, k, w) for b in points}
    pts = {f"decode_b{b}": round(m[0], 1) for b, m in measured.items()}
    # the same bound as `roofline`, for the other points: bytes a step must read / its time / the HBM peak
    pts_frac = {f"decode_b{b}": round(m[2] / HBM_PEAK_GBS, 4) for b, m in measured.items()}
    extras = {}
    if not args.skip_extras:
        # the host's share of a step: each phase ends with a wait for the device, so they add up to more than a step
        *_, phases = bench.decode(args.batch, min(k, 32), 2, phases=True)
        extras["phases_ms_per_step"] = phases
        # decode behind 2,048-token prompts, 256 generated tokens per sequence: the timed steps are the last 247
        # (contexts of about 2,060 to 2,310; at batch 64 the first sequences decode while the last are prefilled)
        for b in sorted({1, args.batch, max_batch}):
            m = bench.decode(b, 247, 8, prompt_len=2048)
            pts[f"decode_b{b}_2048in_256out"] = round(m[0], 1)
            pts_frac[f"decode_b{b}_2048in_256out"] = round(m[2] / HBM_PEAK_GBS, 4)
        if max_batch >= 64:
            throughput, prefix = reference_workloads(cfg, args.dtype, bench.prompt)
            release()
            pts["throughput_64x256in_128out"] = round(throughput, 1)
            pts["shared_prefix_64x544in_64out"] = round(prefix, 1)
        bench.engine = None
        release()
        # further contexts and prompt lengths of the headline shape: decode at batch 8 behind 16,384 and 32,768 tokens,
        # whole prompts of 8,192 and 32,768 tokens
        for ctx in (16384, 32768):
            far = DecodeBench(cfg, args.dtype, ctx, args.batch)
            m = far.decode(args.batch, 32, 4)
            pts[f"decode_b{args.batch}_ctx{ctx}"] = round(m[0], 1)
            pts_frac[f"decode_b{args.batch}_ctx{ctx}"] = round(m[2] / HBM_PEAK_GBS, 4)
            if ctx == 32768:
                for tokens in (8192, 32768 - 64):
                    pf = far.prefill(tokens)
                    pts[f"prefill_{tokens}_tok_s"], pts_frac[f"prefill_{tokens}"] = pf["value"], pf["frac"]
            far.engine = None
            del far
            release()
        if args.dtype == "bfloat16":
            f32 = DecodeBench(cfg, "float32", args.context, args.batch)
            m = f32.decode(args.batch, 8, 2)
            pts[f"decode_b{args.batch}_float32"] = round(m[0], 1)
            pf = f32.prefill(args.prefill_tokens)
            pts["prefill_float32_tok_s"], pts_frac["prefill_float32"] = pf["value"], pf["frac"]
            del f32
            release()
        for shape in ("8b", "32b"):
            work = serving_workload(shape, args.dtype)
            pts[f"serving_{shape}_out_tok_s"] = work["tok_s"]
            pts[f"serving_{shape}_steps"] = work["steps"]
            pts[f"serving_{shape}_preemptions"] = work["preemptions"]
            pts[f"serving_{shape}_cached_tokens"] = work["cached_tokens"]
        # the decode steps and the prefill of the other shapes (the in-between one, whose products fall between the
        # thresholds of the kernel choice, and the two wide ones), near the contexts of their serving workloads
        for shape in ("1.7b", "8b", "32b"):
            sp = shape_points(shape, args.dtype, 32, 4, args.prefill_tokens)
            for key, value in sp["points"].items():
                pts[f"{key}_{shape}_ctx{sp['ctx']}"] = value
                pts_frac[f"{key}_{shape}_ctx{sp['ctx']}"] = sp["fracs"][key]
            pts[f"prefill_{sp['prefill']['tokens']}_{shape}_tok_s"] = sp["prefill"]["value"]
            pts_frac[f"prefill_{sp['prefill']['tokens']}_{shape}"] = sp["prefill"]["frac"]
        extras["measured_peaks"] = measured_peaks()
    line = {
        "metric": f"decode tok/s at batch {args.batch} (Qwen3-0.6B shape)", "value": round(tok_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": k, "warmup": w, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded uniform-random token ids, random N(0, 0.02) weights",
        "config": flat_config(cfg, "Qwen3-0.6B shape", global_batch=args.batch, seq_len=args.context, block_size=bench.block,
                              graphs=bench.econf.cuda_graphs, parallelism="single GPU"),
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4)},
        "points": pts,
        "points_roofline_frac": pts_frac,
        **extras,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
