"""A toy mixer with state of its own, defined here, is registered, built into a model and stepped
without a change to the framework's files. It keeps, per request, the running sum of its inputs
(a fixed-size state in a slot) and returns the running mean through a projection:

    s_t = s_{t-1} + h_t;   y_t = W (s_t / (t + 1))

The state must be carried from portion to portion, start from zero for a new request in a used slot,
and not leak between requests that share a batch. A toy feed-forward with routing (two experts, top-1
by a float32 router) and no position encoding on that layer (the mixer is order-aware by itself) show the
other registries; a second test registers a toy position encoding (angles that grow with the square
root of the position, over the first half of each head) for the framework's own attention mixer. None
of this is a model of anyone's."""

from __future__ import annotations

from dataclasses import dataclass

import pytest
import torch

pytestmark = pytest.mark.gpu


@dataclass(frozen=True)
class RunningMeanSpec:
    hidden_size: int
    kind: str = "toy_running_mean"


@dataclass(frozen=True)
class Top1ExpertsSpec:
    hidden_size: int
    num_experts: int
    kind: str = "toy_top1_experts"


def register_toys():
    from mini_engine_amd.parts import FEED_FORWARDS, MIXERS, FeedForward, Mixer, StateNeed
    from mini_engine_amd.weights import TensorWant

    class RunningMean(Mixer):
        def weight_wants(self, prefix):
            h = self.spec.hidden_size
            return {f"{prefix}.out.weight": TensorWant((h, h))}

        def load(self, tensors, prefix):
            self.w = tensors[f"{prefix}.out.weight"]

        def cache_need(self):
            return StateNeed((self.spec.hidden_size,), torch.float32)

        def forward(self, h, batch, cache=None):
            out = torch.empty_like(h)
            cursor = 0
            for start, n, slot in zip(batch.starts, batch.qlens, batch.slots_host):
                seg = h[cursor : cursor + n].float()
                running = cache.state[slot] + seg.cumsum(0)
                counts = torch.arange(start + 1, start + n + 1, device=h.device, dtype=torch.float32)[:, None]
                out[cursor : cursor + n] = ((running / counts) @ self.w.float().T).to(h.dtype)
                cache.state[slot] = running[-1]
                cursor += n
            return out

    class Top1Experts(FeedForward):
        def weight_wants(self, prefix):
            h, e = self.spec.hidden_size, self.spec.num_experts
            wants = {f"{prefix}.router.weight": TensorWant((e, h), "vector")}  # kept in float32
            for i in range(e):
                wants[f"{prefix}.experts.{i}.weight"] = TensorWant((h, h))
            return wants

        def load(self, tensors, prefix):
            self.router = tensors[f"{prefix}.router.weight"]
            self.experts = [tensors[f"{prefix}.experts.{i}.weight"] for i in range(self.spec.num_experts)]

        def forward(self, h, batch=None):
            choice = (h.float() @ self.router.T).argmax(-1)  # router logits in float32
            out = torch.zeros_like(h)
            for i, w in enumerate(self.experts):
                rows = (choice == i).nonzero()[:, 0]
                if rows.numel():
                    out[rows] = (h[rows].float() @ w.float().T).to(h.dtype)
            return out

    MIXERS.register("toy_running_mean", RunningMean)
    FEED_FORWARDS.register("toy_top1_experts", Top1Experts)


def toy_plan():
    """Layer 0: the toy mixer + routed toy feed-forward. Layer 1: attention + dense gated MLP."""
    from mini_engine_amd.config import AttentionSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec, RotarySpec

    h = 48
    norm = NormSpec(dim=h, eps=1e-5)
    layers = (
        LayerSpec(mixer=RunningMeanSpec(h), ffn=Top1ExpertsSpec(h, 2), mixer_norm=norm, ffn_norm=norm,
                  mixer_prefix="toy.0.mix", ffn_prefix="toy.0.moe", mixer_norm_name="toy.0.n1", ffn_norm_name="toy.0.n2"),
        LayerSpec(mixer=AttentionSpec(hidden_size=h, num_heads=3, num_kv_heads=1, head_dim=16, scale=0.25,
                                      qk_norm_eps=None, position=RotarySpec(16, 1e4)),
                  ffn=GatedMlpSpec(hidden_size=h, intermediate_size=80), mixer_norm=norm, ffn_norm=norm,
                  mixer_prefix="toy.1.attn", ffn_prefix="toy.1.mlp", mixer_norm_name="toy.1.n1", ffn_norm_name="toy.1.n2"),
    )
    return ModelPlan(architecture="ToyForTests", vocab_size=97, hidden_size=h, layers=layers, order=(0, 1),
                     final_norm=norm, embed_name="toy.embed", final_norm_name="toy.norm", head_name="toy.head",
                     tie_word_embeddings=False, max_position_embeddings=256)


def plain_toy(w, tokens):
    import plain_qwen3 as plain

    x = w["toy.embed"][torch.tensor(tokens)]
    t = len(tokens)
    h = plain.rms_norm(x, w["toy.0.n1"], 1e-5)
    x = x + (h.cumsum(0) / torch.arange(1, t + 1)[:, None]) @ w["toy.0.mix.out.weight"].T
    h = plain.rms_norm(x, w["toy.0.n2"], 1e-5)
    choice = (h @ w["toy.0.moe.router.weight"].T).argmax(-1)
    moe = torch.stack([h[i] @ w[f"toy.0.moe.experts.{int(choice[i])}.weight"].T for i in range(t)])
    x = x + moe
    h = plain.rms_norm(x, w["toy.1.n1"], 1e-5)
    q = (h @ w["toy.1.attn.q_proj.weight"].T).view(t, 3, 16)
    k = (h @ w["toy.1.attn.k_proj.weight"].T).view(t, 1, 16)
    v = (h @ w["toy.1.attn.v_proj.weight"].T).view(t, 1, 16)
    cos, sin = plain.rope_tables(torch.arange(t), 16, 1e4)
    a = plain.grouped_causal_attention(plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin), v, 0.25)
    x = x + a.reshape(t, -1) @ w["toy.1.attn.o_proj.weight"].T
    h = plain.rms_norm(x, w["toy.1.n2"], 1e-5)
    x = x + plain.swiglu_mlp(h, w, "toy.1.mlp")
    return plain.rms_norm(x, w["toy.norm"], 1e-5) @ w["toy.head"].T


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    from mini_engine_amd import EngineConfig
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.runner import ModelRunner
    from mini_engine_amd.engine.sequence import Sequence
    from mini_engine_amd.parts import Decoder
    from mini_engine_amd.weights import RandomSource

    register_toys()
    plan = toy_plan()
    dec = Decoder(plan, torch.float32, "cuda")
    wants = dec.weight_wants()
    assert "toy.0.mix.out.weight" in wants and "toy.0.moe.experts.1.weight" in wants
    src = RandomSource(wants, seed=2, std=0.2, norm_std=0.1, device="cpu")
    weights = {n: src.get(n) for n in wants}
    weights["toy.0.moe.router.weight"] = torch.randn(2, 48, generator=torch.Generator().manual_seed(8))

    class Source:
        def shapes(self):
            return {n: tuple(t.shape) for n, t in weights.items()}

        def get(self, n):
            return weights[n]

    dec.load(Source())
    runner = ModelRunner(dec, EngineConfig(block_size=8, num_blocks=32, max_num_seqs=2, dtype="float32",
                                           max_model_len=128))
    assert runner.layout.has_state and list(runner.layout.state_layers) == [0] and runner.program is not None
    bm = runner.new_block_manager()
    assert not bm.enable_prefix_caching  # state cannot be rebuilt from shared pages

    g = torch.Generator().manual_seed(1)
    reqs = {k: torch.randint(0, 97, (n,), generator=g).tolist() for k, n in (("a", 37), ("b", 21), ("c", 30))}
    want = {k: plain_toy(weights, v) for k, v in reqs.items()}
    assert len({int(c) for c in (want["a"].argmax(-1))}) > 1

    def feed(schedule):
        """schedule: list of steps, each a list of (request, number of tokens)."""
        seqs, got = {}, {k: [] for k in reqs}
        for step in schedule:
            items = []
            for k, n in step:
                seq = seqs.setdefault(k, Sequence(reqs[k]))
                lo = seq.num_computed_tokens
                assert bm.try_allocate(seq, lo + n)
                items.append((k, StepItem(seq, reqs[k][lo : lo + n], lo, list(range(n)))))
            out = runner.step([it for _, it in items]).cpu()
            r = 0
            for k, it in items:
                got[k].append(out[r : r + len(it.tokens)].clone())
                r += len(it.tokens)
                seqs[k].num_computed_tokens += len(it.tokens)
                if seqs[k].num_computed_tokens == len(reqs[k]):
                    bm.free(seqs.pop(k))
        return {k: torch.cat(v) for k, v in got.items() if v}

    # whole requests one after another: the second and third reuse a slot whose state is not zero
    whole = feed([[("a", 37)], [("b", 21)], [("c", 30)]])
    for k in reqs:
        torch.testing.assert_close(whole[k], want[k], rtol=1e-4, atol=1e-4)
    # portions and single tokens, two requests side by side, the third admitted when a slot frees
    mixed = feed([[("a", 10), ("b", 1)], [("b", 19), ("a", 2)], [("a", 1)], [("a", 24), ("b", 1)], [("c", 29)], [("c", 1)]])
    for k in reqs:
        torch.testing.assert_close(mixed[k], want[k], rtol=1e-4, atol=1e-4)
    assert bm.slots.in_use == set() and all(len(p.free_pool) == p.num_blocks for p in bm.pools)


@dataclass(frozen=True)
class SqrtAnglesSpec:
    rotary_dim: int
    rate: float
    kind: str = "toy_sqrt_angles"


def register_toy_position():
    from mini_engine_amd.parts import POSITION_ENCODINGS, PositionEncoding

    class SqrtAngles(PositionEncoding):
        """angle[p, j] = rate * sqrt(p) / (j + 1): not a function of distances alone, so a table
        read at a wrong row or a portion that restarts at zero changes the logits."""

        def tables(self, num_positions=1):
            rd = self.spec.rotary_dim
            p = torch.arange(max(num_positions, 256), dtype=torch.float32, device=self.device)
            angle = self.spec.rate * p.sqrt()[:, None] / torch.arange(1, rd // 2 + 1, device=self.device)
            return torch.stack((angle.cos(), angle.sin()), dim=1).contiguous()

    POSITION_ENCODINGS.register("toy_sqrt_angles", SqrtAngles)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_position_encoding_is_registered_and_used_by_the_attention_mixer(dtype):
    import plain_qwen3 as plain
    from mini_engine_amd import EngineConfig
    from mini_engine_amd.config import AttentionSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.runner import ModelRunner
    from mini_engine_amd.engine.sequence import Sequence
    from mini_engine_amd.parts import Decoder
    from mini_engine_amd.weights import RandomSource

    register_toy_position()
    h, nh, nkv, d, rd = 64, 4, 2, 32, 16
    norm = NormSpec(dim=h, eps=1e-5)
    layer = LayerSpec(mixer=AttentionSpec(hidden_size=h, num_heads=nh, num_kv_heads=nkv, head_dim=d, scale=0.3,
                                          qk_norm_eps=None, position=SqrtAnglesSpec(rd, 1.7)),
                      ffn=GatedMlpSpec(hidden_size=h, intermediate_size=96), mixer_norm=norm, ffn_norm=norm,
                      mixer_prefix="t.attn", ffn_prefix="t.mlp", mixer_norm_name="t.n1", ffn_norm_name="t.n2")
    plan = ModelPlan(architecture="ToyPositionForTests", vocab_size=113, hidden_size=h, layers=(layer,), order=(0,),
                     final_norm=norm, embed_name="t.embed", final_norm_name="t.norm", head_name="t.head",
                     tie_word_embeddings=False, max_position_embeddings=256)
    dec = Decoder(plan, dtype, "cuda")
    wants = dec.weight_wants()
    src = RandomSource(wants, seed=5, std=0.2, norm_std=0.1, device="cpu")
    # matrices rounded to bfloat16, so that both dtypes and the plain implementation see the same values
    weights = {n: (src.get(n).to(torch.bfloat16).float() if w.role == "matrix" else src.get(n))
               for n, w in wants.items()}

    class Source:
        def shapes(self):
            return {n: tuple(t.shape) for n, t in weights.items()}

        def get(self, n):
            return weights[n]

    dec.load(Source())
    runner = ModelRunner(dec, EngineConfig(block_size=16, num_blocks=16, max_num_seqs=2, dtype=str(dtype)[6:],
                                           max_model_len=128))
    bm = runner.new_block_manager()
    tokens = torch.randint(0, 113, (70,), generator=torch.Generator().manual_seed(3)).tolist()

    def rotate(x, cos, sin):  # the first rd elements of each head, pairs (j, j + rd/2)
        return torch.cat((plain.apply_rope(x[..., :rd], cos, sin), x[..., rd:]), dim=-1)

    w = {n: t.float() for n, t in weights.items()}
    t = len(tokens)
    x = w["t.embed"][torch.tensor(tokens)]
    hn = plain.rms_norm(x, w["t.n1"], 1e-5)
    q = (hn @ w["t.attn.q_proj.weight"].T).view(t, nh, d)
    k = (hn @ w["t.attn.k_proj.weight"].T).view(t, nkv, d)
    v = (hn @ w["t.attn.v_proj.weight"].T).view(t, nkv, d)
    angle = 1.7 * torch.arange(t, dtype=torch.float32).sqrt()[:, None] / torch.arange(1, rd // 2 + 1)
    cos, sin = torch.cat((angle, angle), -1).cos(), torch.cat((angle, angle), -1).sin()
    a = plain.grouped_causal_attention(rotate(q, cos, sin), rotate(k, cos, sin), v, 0.3)
    x = x + a.reshape(t, -1) @ w["t.attn.o_proj.weight"].T
    x = x + plain.swiglu_mlp(plain.rms_norm(x, w["t.n2"], 1e-5), w, "t.mlp")
    want = plain.rms_norm(x, w["t.norm"], 1e-5) @ w["t.head"].T
    no_rotation = plain.grouped_causal_attention(q, k, v, 0.3)
    assert (a - no_rotation).abs().max() > 0.05  # the encoding matters at these sizes

    seq, got = Sequence(tokens), []
    for n in (33, 2, 19, 1, 1, 14):  # portions and single tokens
        lo = seq.num_computed_tokens
        assert bm.try_allocate(seq, lo + n)
        got.append(runner.step([StepItem(seq, tokens[lo : lo + n], lo, list(range(n)))]).float().cpu())
        seq.num_computed_tokens += n
    bm.free(seq)
    got = torch.cat(got)
    if dtype is torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-4)
    else:
        assert (got - want).abs().max() < 0.04 * want.abs().max()


# ------------------------------------------------------------------------------------------------
# Toy parts that can be captured into a graph, a norm that is not RMS-shaped, and the plan's scales


@dataclass(frozen=True)
class CenteredNormSpec:
    dim: int
    eps: float
    kind: str = "toy_centered_norm"


@dataclass(frozen=True)
class BlendedExpertsSpec:
    hidden_size: int
    kind: str = "toy_blended_experts"


def register_capturable_toys():
    from mini_engine_amd.parts import FEED_FORWARDS, MIXERS, NORMS, FeedForward, Mixer, Norm, StateNeed
    from mini_engine_amd.weights import TensorWant

    class CenteredNorm(Norm):
        """Mean subtraction, variance norm, weight and bias: nothing the RMS kernels could compute."""

        graph_safe = True

        def weight_wants(self, name):
            return {name: TensorWant((self.spec.dim,), "vector"), name + ".bias": TensorWant((self.spec.dim,), "vector")}

        def load(self, tensors, name):
            self.weight, self.bias = tensors[name], tensors[name + ".bias"]

        def forward(self, x):
            centered = x - x.mean(-1, keepdim=True)
            y = centered * torch.rsqrt(centered.pow(2).mean(-1, keepdim=True) + self.spec.eps)
            return (y * self.weight + self.bias).to(self.dtype)

    class RunningMeanOnDevice(Mixer):
        """The running mean of the first test; a decode step reads its slots and positions from the
        batch's device tensors, so the launches can be captured once and replayed."""

        graph_safe = True

        def weight_wants(self, prefix):
            return {f"{prefix}.out.weight": TensorWant((self.spec.hidden_size, self.spec.hidden_size))}

        def load(self, tensors, prefix):
            self.w = tensors[f"{prefix}.out.weight"]

        def cache_need(self):
            return StateNeed((self.spec.hidden_size,), torch.float32)

        def forward(self, h, batch, cache=None):
            if batch.decode_only:
                slots = batch.state_slots.long()
                running = cache.state[slots] + h.float()
                cache.state[slots] = running  # rows that pad the batch all write the spare slot, which nobody reads
                counts = (batch.positions + 1).float()[:, None]
                return ((running / counts) @ self.w.float().T).to(h.dtype)
            out = torch.empty_like(h)
            cursor = 0
            for start, n, slot in zip(batch.starts, batch.qlens, batch.slots_host):
                running = cache.state[slot] + h[cursor : cursor + n].float().cumsum(0)
                counts = torch.arange(start + 1, start + n + 1, device=h.device, dtype=torch.float32)[:, None]
                out[cursor : cursor + n] = ((running / counts) @ self.w.float().T).to(h.dtype)
                cache.state[slot] = running[-1]
                cursor += n
            return out

    class BlendedExperts(FeedForward):
        """Two experts, the better one by a float32 router; both are computed and one is kept, so
        nothing waits for the device."""

        graph_safe = True

        def weight_wants(self, prefix):
            h = self.spec.hidden_size
            return {f"{prefix}.router.weight": TensorWant((2, h), "vector"),
                    f"{prefix}.experts.0.weight": TensorWant((h, h)), f"{prefix}.experts.1.weight": TensorWant((h, h))}

        def load(self, tensors, prefix):
            self.router = tensors[f"{prefix}.router.weight"]
            self.experts = [tensors[f"{prefix}.experts.{i}.weight"] for i in range(2)]

        def forward(self, h, batch=None):
            score = h.float() @ self.router.T
            both = [h.float() @ w.float().T for w in self.experts]
            return torch.where((score[:, 1] > score[:, 0])[:, None], both[1], both[0]).to(h.dtype)

    NORMS.register("toy_centered_norm", CenteredNorm)
    MIXERS.register("toy_running_mean_on_device", RunningMeanOnDevice)
    FEED_FORWARDS.register("toy_blended_experts", BlendedExperts)


def capturable_plan():
    from mini_engine_amd.config import AttentionSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec, RotarySpec

    h = 48
    rms, centered = NormSpec(dim=h, eps=1e-5), CenteredNormSpec(dim=h, eps=1e-3)
    layers = (
        LayerSpec(mixer=RunningMeanSpec(h, kind="toy_running_mean_on_device"), ffn=BlendedExpertsSpec(h),
                  mixer_norm=centered, ffn_norm=rms, mixer_prefix="toy.0.mix", ffn_prefix="toy.0.moe",
                  mixer_norm_name="toy.0.n1", ffn_norm_name="toy.0.n2"),
        LayerSpec(mixer=AttentionSpec(hidden_size=h, num_heads=3, num_kv_heads=1, head_dim=16, scale=0.25,
                                      qk_norm_eps=None, position=RotarySpec(16, 1e4)),
                  ffn=GatedMlpSpec(hidden_size=h, intermediate_size=80), mixer_norm=rms, ffn_norm=centered,
                  mixer_prefix="toy.1.attn", ffn_prefix="toy.1.mlp", mixer_norm_name="toy.1.n1", ffn_norm_name="toy.1.n2"),
    )
    return ModelPlan(architecture="CapturableToyForTests", vocab_size=97, hidden_size=h, layers=layers, order=(0, 1),
                     final_norm=centered, embed_name="toy.embed", final_norm_name="toy.norm", head_name="toy.head",
                     tie_word_embeddings=False, max_position_embeddings=256, embedding_multiplier=1.5, logit_scale=0.25)


def plain_capturable(w, tokens):
    import plain_qwen3 as plain

    def centered(x, name):
        c = x - x.mean(-1, keepdim=True)
        return c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-3) * w[name] + w[name + ".bias"]

    t = len(tokens)
    x = 1.5 * w["toy.embed"][torch.tensor(tokens)]
    h = centered(x, "toy.0.n1")
    x = x + (h.cumsum(0) / torch.arange(1, t + 1)[:, None]) @ w["toy.0.mix.out.weight"].T
    h = plain.rms_norm(x, w["toy.0.n2"], 1e-5)
    choice = (h @ w["toy.0.moe.router.weight"].T).argmax(-1)
    x = x + torch.stack([h[i] @ w[f"toy.0.moe.experts.{int(choice[i])}.weight"].T for i in range(t)])
    h = plain.rms_norm(x, w["toy.1.n1"], 1e-5)
    q = (h @ w["toy.1.attn.q_proj.weight"].T).view(t, 3, 16)
    k = (h @ w["toy.1.attn.k_proj.weight"].T).view(t, 1, 16)
    v = (h @ w["toy.1.attn.v_proj.weight"].T).view(t, 1, 16)
    cos, sin = plain.rope_tables(torch.arange(t), 16, 1e4)
    a = plain.grouped_causal_attention(plain.apply_rope(q, cos, sin), plain.apply_rope(k, cos, sin), v, 0.25)
    x = x + a.reshape(t, -1) @ w["toy.1.attn.o_proj.weight"].T
    x = x + plain.swiglu_mlp(centered(x, "toy.1.n2"), w, "toy.1.mlp")
    return 0.25 * (centered(x, "toy.norm") @ w["toy.head"].T)


@pytest.mark.parametrize("kernel_by_kernel", [False, True])
@pytest.mark.parametrize("graphs", [True, False])
def test_capturable_toy_parts_replay_from_graphs(graphs, kernel_by_kernel):
    """A model of toy parts that say they can be captured: a mixer with state, a routed
    feed-forward, a norm with mean subtraction and bias (before a mixer, before a feed-forward and as
    the final norm), an embedding multiplier and a logit scale. Decode steps replay a graph; rows that
    pad the batch write the spare state slot; a request whose one-token prompt arrives in a decode
    step starts from a zero state in a slot that another request has used. The parts run as calls inside
    the engine's step program; the same parts launched kernel by kernel from Python give the same."""
    from mini_engine_amd import EngineConfig
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.runner import ModelRunner
    from mini_engine_amd.engine.sequence import Sequence
    from mini_engine_amd.parts import Decoder
    from mini_engine_amd.weights import RandomSource

    register_capturable_toys()
    dec = Decoder(capturable_plan(), torch.float32, "cuda")
    wants = dec.weight_wants()
    src = RandomSource(wants, seed=9, std=0.2, norm_std=0.3, device="cpu")
    weights = {n: src.get(n) for n in wants}
    weights["toy.0.moe.router.weight"] = torch.randn(2, 48, generator=torch.Generator().manual_seed(8))

    class Source:
        def shapes(self):
            return {n: tuple(t.shape) for n, t in weights.items()}

        def get(self, n):
            return weights[n]

    dec.load(Source())
    if kernel_by_kernel:
        from kernel_by_kernel import KernelByKernelRunner as ModelRunner  # noqa: F811
    runner = ModelRunner(dec, EngineConfig(block_size=8, num_blocks=32, max_num_seqs=3, dtype="float32", max_model_len=128,
                                           cuda_graphs=graphs))
    # the model steps through the native program like any other: its own parts are calls in it
    assert runner.layout.has_state and runner.graph_safe and runner.program is not None
    bm = runner.new_block_manager()
    g = torch.Generator().manual_seed(4)
    reqs = {k: torch.randint(0, 97, (n,), generator=g).tolist() for k, n in (("a", 20), ("b", 9), ("c", 7))}
    want = {k: plain_capturable(weights, v) for k, v in reqs.items()}
    assert len({int(c) for c in want["a"].argmax(-1)}) > 1
    schedule = [[("a", 14), ("b", 3)]] + [[("a", 1), ("b", 1)]] * 6 + [[("c", 1)]] * 7
    seqs, got = {}, {k: [] for k in reqs}
    for step in schedule:
        items = []
        for k, n in step:
            seq = seqs.setdefault(k, Sequence(reqs[k]))
            lo = seq.num_computed_tokens
            assert bm.try_allocate(seq, lo + n)
            items.append((k, StepItem(seq, reqs[k][lo : lo + n], lo, list(range(n)))))
        out = runner.step([it for _, it in items]).cpu()
        r = 0
        for k, it in items:
            got[k].append(out[r : r + len(it.tokens)].clone())
            r += len(it.tokens)
            seqs[k].num_computed_tokens += len(it.tokens)
            if seqs[k].num_computed_tokens == len(reqs[k]):
                bm.free(seqs.pop(k))
    for k in reqs:
        torch.testing.assert_close(torch.cat(got[k]), want[k], rtol=1e-4, atol=1e-4)
    assert runner.graph_replays == (13 if graphs else 0)
    assert bm.slots.in_use == set()


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_plan_scales_and_gate_activation_in_the_native_step(tiny_folders, activation, monkeypatch):
    """The plan's two scales and the feed-forward's other activation through the native step program, in
    both dtypes, against the plain implementation with a scaled embedding table, scaled logits and the
    activation swapped (B's head is not tied). Portions of 33 and 5 tokens and single tokens: the gate is the
    epilogue of the small and of the streaming product, and follows a library product."""
    import dataclasses

    import plain_qwen3 as plain
    import trace_helpers as th
    from conftest import random_prompt
    from mini_engine_amd import EngineConfig, LLMEngine
    from mini_engine_amd.config.registry import plan_from_folder
    from mini_engine_amd.engine.batch import StepItem
    from mini_engine_amd.engine.runner import TORCH_DTYPES
    from mini_engine_amd.engine.sequence import Sequence
    from mini_engine_amd.parts import Decoder
    from mini_engine_amd.weights.loader import FolderSource

    folder = tiny_folders["B"]
    _, plan = plan_from_folder(folder)
    layers = tuple(dataclasses.replace(l, ffn=dataclasses.replace(l.ffn, activation=activation)) for l in plan.layers)
    plan = dataclasses.replace(plan, layers=layers, embedding_multiplier=3.0, logit_scale=0.5)
    pcfg, w = plain.read_config(folder), plain.read_weights(folder)
    w["model.embed_tokens.weight"] = 3.0 * w["model.embed_tokens.weight"]
    tokens = random_prompt(40, pcfg.vocab_size, seed=12)
    if activation == "gelu_tanh":
        monkeypatch.setattr(plain, "silu", lambda z: torch.nn.functional.gelu(z, approximate="tanh"))
    want = 0.5 * plain.forward_logits(w, pcfg, tokens)
    for dtype in ("float32", "bfloat16"):
        model = Decoder(plan, TORCH_DTYPES[dtype], "cuda")
        model.load(FolderSource(folder))
        engine = LLMEngine(model, EngineConfig(block_size=8, num_blocks=16, dtype=dtype, max_model_len=64))
        assert engine.runner.program is not None
        seq, got = Sequence(tokens, core=engine.core), []
        for n in (33, 1, 1, 5):
            lo = seq.num_computed_tokens
            assert engine.block_manager.try_allocate(seq, lo + n)
            got.append(engine.runner.step([StepItem(seq, tokens[lo : lo + n], lo, list(range(n)))]).float().cpu())
            seq.num_computed_tokens += n
        engine.block_manager.free(seq)
        th.assert_logits_close(torch.cat(got), want, dtype, f"scaled embedding and logits, {activation}, {dtype}")
