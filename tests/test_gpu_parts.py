"""Each part alone against its plain function, and a toy architecture defined here that the engine
has never seen: a mixer with state of its own, a windowed attention layer in a cache group of its
own, a layer that runs twice, and a layer that reads another layer's cache."""
import json
import math
import os

import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


def dev(x, dtype=torch.float32):
    return torch.as_tensor(np.asarray(x)).to(DEV).to(dtype).contiguous()


class PartHarness:
    """Runs one part on a batch of sequences through the engine's own cache manager and batch builder."""

    def __init__(self, cache_specs, dtype, page_size=8, pages=64):
        from sprout_lm_amd.cache import CacheManager
        from sprout_lm_amd.engine.batch import DescriptorStager, Workspace
        self.dtype = dtype
        self.cache = CacheManager(cache_specs, page_size, pages, 8, prefix_caching=False)
        self.cache.attach_storage(dtype, DEV)
        self.workspace, self.stager = Workspace(DEV), DescriptorStager(DEV)

    def context(self, seqs_and_counts):
        from sprout_lm_amd.engine.batch import StepEntry, build_context
        entries = []
        for seq, n in seqs_and_counts:
            assert self.cache.reserve(seq, seq.length + n)
            entries.append(StepEntry(seq, [0] * n, []))
        return build_context(entries, self.cache, self.stager, self.workspace, self.dtype,
                             1 if self.dtype == torch.float32 else 0), entries

    def slot_view(self, ctx, slot, writes=True):
        from sprout_lm_amd.engine.batch import CacheSlotView
        kind, g, index = self.cache.slot_location[slot]
        group = self.cache.groups[g]
        return CacheSlotView(writes, k=group.k[index], v=group.v[index], block_tables=ctx.group_tables[g],
                             slot_mapping=ctx.group_slots[g], page_size=self.cache.block_size)

    def commit(self, entries):
        for e in entries:
            self.cache.commit(e.seq, e.seq.length + len(e.tokens))


def rounded(x, dtype):
    return P.bf16_round(x) if dtype == torch.bfloat16 else np.asarray(x, np.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_embedding_head_parts(dtype):
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(0)
    Hd, V = 72, 131
    norm = make_part("norm", "rmsnorm", size=Hd, eps=1e-4)
    w = rounded(rng.uniform(0.5, 1.5, Hd), dtype)
    norm.bind({"weight": dev(w, dtype)})
    x = rng.standard_normal((5, Hd)).astype(np.float32)
    out = torch.empty(5, Hd, dtype=dtype, device=DEV)
    norm.forward(None, dev(x), out)
    tol = 2e-6 if dtype == torch.float32 else 2 ** -8
    assert np.abs(out.float().cpu().numpy() - P.rms_norm(x, w, 1e-4)).max() <= tol * 4
    table = rounded(rng.standard_normal((V, Hd)), dtype)
    emb = make_part("embedding", "token_embedding", vocab=V, hidden=Hd)
    emb.bind({"weight": dev(table, dtype)})
    res = torch.empty(3, Hd, device=DEV)
    emb.forward(None, torch.tensor([130, 0, 7], dtype=torch.int32, device=DEV), res)
    assert np.array_equal(res.cpu().numpy(), table[[130, 0, 7]])
    head = make_part("head", "linear_head", vocab=V, hidden=Hd, tied=True)
    head.bind({})
    head.tie(emb.w["weight"])
    hrows = rounded(rng.standard_normal((3, Hd)), dtype)
    logits = torch.empty(3, V, device=DEV)
    head.forward(None, dev(hrows, dtype), logits)
    assert np.abs(logits.cpu().numpy() - P.linear(hrows, table)).max() <= 1e-4
    assert make_part("head", "linear_head", vocab=V, hidden=Hd, tied=False).tensors()["weight"].shape == (V, Hd)


def attention_weights(rng, hidden, heads, kv_heads, hd, dtype, own_kv=True):
    names = [("q_proj", heads * hd)] + ([("k_proj", kv_heads * hd), ("v_proj", kv_heads * hd)] if own_kv else [])
    w = {}
    for name, rows in names:
        w[f"{name}.weight"] = rounded(rng.standard_normal((rows, hidden)) * 0.2, dtype)
        w[f"{name}.bias"] = rounded(rng.uniform(-0.3, 0.3, rows), dtype)
    w["o_proj.weight"] = rounded(rng.standard_normal((hidden, heads * hd)) * 0.2, dtype)
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,window", [(4, 2, 16, None), (3, 1, 32, None), (6, 2, 48, 7), (2, 2, 64, 20)])
def test_attention_part_alone_in_portions(dtype, heads, kv_heads, hd, window):
    """One attention part, two sequences fed in uneven portions beside each other, against the plain function."""
    from sprout_lm_amd.models.plan import PartPlan
    rng = np.random.default_rng(heads * 10 + hd)
    hidden, theta = 40, 5000.0
    part = PartPlan("mixer", "attention", {"hidden": hidden, "heads": heads, "kv_heads": kv_heads, "head_dim": hd,
                                           "position": PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": theta}),
                                           "window": window}).make()
    w = attention_weights(rng, hidden, heads, kv_heads, hd, dtype)
    part.bind({k: dev(v, dtype) for k, v in w.items()})
    part.prepare(DEV, dtype)
    harness = PartHarness([part.cache_spec()], dtype)
    lengths = [37, 22]
    hs = [rounded(rng.standard_normal((n, hidden)), dtype) for n in lengths]
    store = P.bf16_round if dtype == torch.bfloat16 else P.f32
    want = []
    for h in hs:   # the plain mixer: projections, rotation, attention, output projection
        pos = np.arange(len(h))
        q = store(P.rope_neox(store(P.linear(h, w["q_proj.weight"], w["q_proj.bias"])), pos, hd, theta))
        k = store(P.rope_neox(store(P.linear(h, w["k_proj.weight"], w["k_proj.bias"])), pos, hd, theta))
        v = store(P.linear(h, w["v_proj.weight"], w["v_proj.bias"]))
        a = store(P.causal_gqa_attention(q, k, v, heads, kv_heads, hd, window=window))
        want.append(P.linear(a, w["o_proj.weight"]))
    seqs = [harness.cache.create() for _ in lengths]
    fed = [0, 0]
    got = [np.zeros((n, hidden), np.float32) for n in lengths]
    portions = [(16, 1), (5, 9), (1, 1), (2, 3), (13, 8)]
    for step in portions:
        batch = [(s, min(n, lengths[i] - fed[i])) for i, (s, n) in enumerate(zip(seqs, step)) if fed[i] < lengths[i]]
        index = [i for i in range(2) if fed[i] < lengths[i]]
        ctx, entries = harness.context(batch)
        h = torch.cat([dev(hs[i][fed[i]:fed[i] + n], dtype) for i, (_, n) in zip(index, batch)])
        residual = torch.zeros(h.shape[0], hidden, device=DEV)
        part.forward(ctx, h, residual, harness.slot_view(ctx, 0))
        out = residual.cpu().numpy()
        harness.commit(entries)
        row = 0
        for i, (_, n) in zip(index, batch):
            got[i][fed[i]:fed[i] + n] = out[row:row + n]
            fed[i] += n
            row += n
    assert fed == lengths
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for g, wnt in zip(got, want):
        assert np.abs(g - wnt).max() <= tol * (1 + np.abs(wnt).max())
    if window:   # pages that the window has passed came back
        assert any(p == -1 for p in seqs[0].blocks[0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 7, 40, 150])
def test_feed_forward_and_block_parts(dtype, T):
    from sprout_lm_amd.models.plan import PartPlan
    rng = np.random.default_rng(T)
    hidden, inner = 56, 104
    cfg = dict(hidden_size=hidden, num_attention_heads=1, num_key_value_heads=1, rms_norm_eps=1e-5, rope_theta=1e4)
    w = {"model.layers.0.mlp.gate_proj.weight": rounded(rng.standard_normal((inner, hidden)) * 0.2, dtype),
         "model.layers.0.mlp.up_proj.weight": rounded(rng.standard_normal((inner, hidden)) * 0.2, dtype),
         "model.layers.0.mlp.down_proj.weight": rounded(rng.standard_normal((hidden, inner)) * 0.2, dtype),
         "model.layers.0.post_attention_layernorm.weight": rounded(rng.uniform(0.7, 1.3, hidden), dtype)}
    ffn = PartPlan("feed_forward", "gated_mlp", {"hidden": hidden, "inner": inner}).make()
    ffn.bind({k.split("mlp.")[1]: dev(v, dtype) for k, v in w.items() if "mlp." in k})
    harness = PartHarness([], dtype)
    ctx, _ = harness.context([])
    h = rounded(rng.standard_normal((T, hidden)), dtype)
    base = rng.standard_normal((T, hidden)).astype(np.float32)
    residual = dev(base)
    ffn.forward(ctx, dev(h, dtype), residual)
    store = P.bf16_round if dtype == torch.bfloat16 else P.f32
    gate = store(P.linear(h, w["model.layers.0.mlp.gate_proj.weight"]))
    up = store(P.linear(h, w["model.layers.0.mlp.up_proj.weight"]))
    want = base + P.linear(store(P.swiglu(gate, up)), w["model.layers.0.mlp.down_proj.weight"])
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(residual.cpu().numpy() - want).max() <= tol * (1 + np.abs(want).max())
    with pytest.raises(ValueError, match="silu"):
        PartPlan("feed_forward", "gated_mlp", {"hidden": 8, "inner": 8, "activation": "gelu"}).make()


# ----------------------------------------------------------------------------------------------------
# A toy architecture, registered here and nowhere in the engine.

def register_toy():
    from dataclasses import dataclass
    from typing import ClassVar

    import sprout_lm_amd as S
    from sprout_lm_amd.cache import StateSpec
    from sprout_lm_amd.config.base import ModelConfig
    from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
    from sprout_lm_amd.parts import Mixer, register_part, registered_parts
    from sprout_lm_amd.weights import TensorSpec

    if "toy_running_mean" in registered_parts("mixer"):
        return

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = W . mean(h_0 .. h_t): the state per request is the running sum and the count.

        A step in which every request brings one token is computed from device-resident values alone (state
        slots and rows are indexed on the device), so the part may be recorded into a graph; portions of
        prompts are cut on the host."""

        graph_safe = True

        def __init__(self, hidden):
            self.hidden = hidden

        def cache_spec(self):
            return StateSpec((self.hidden + 1,), "float32")

        def tensors(self):
            return {"proj.weight": TensorSpec((self.hidden, self.hidden))}

        def forward(self, ctx, h, residual, cache):
            from sprout_lm_amd import ops
            if ctx.max_q_len == 1:
                # row i is request i's one token; padded rows of a recorded step point at the spare state slot
                slots = ctx.state_slots.long()
                state = cache.state.index_select(0, slots)
                sums = state[:, :-1] + h.float()
                counts = state[:, -1] + 1
                mean = (sums / counts[:, None]).to(h.dtype).contiguous()
                ops.gemm(mean, self.w["proj.weight"], residual, accumulate=True)
                cache.state.index_copy_(0, slots, torch.cat([sums, counts[:, None]], dim=1))
                return
            for start, n, slot in zip(ctx.host["q_start"], ctx.host["q_len"], ctx.host["state_slots"]):
                state = cache.state[slot]
                sums = torch.cumsum(h[start:start + n].float(), 0) + state[:-1]
                counts = state[-1] + torch.arange(1, n + 1, device=h.device)
                mean = (sums / counts[:, None]).to(h.dtype).float()
                residual[start:start + n] += mean @ self.w["proj.weight"].float().T
                state[:-1] = sums[-1]
                state[-1] = counts[-1]

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyMeanForCausalLM"
        model_types: ClassVar[tuple] = ("toy_mean",)
        hidden: int = 0
        inner: int = 0
        vocab: int = 0
        heads: int = 0
        kv_heads: int = 0
        window: int = 0
        eps: float = 0.0
        theta: float = 0.0

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "window", "eps", "theta")})

        def to_dict(self):
            return {"architectures": [self.architecture], "model_type": "toy_mean", "hidden": self.hidden,
                    "inner": self.inner, "vocab": self.vocab, "heads": self.heads, "kv_heads": self.kv_heads,
                    "window": self.window, "eps": self.eps, "theta": self.theta}

    def build_toy(cfg):
        hd = cfg.hidden // cfg.heads
        norm = lambda prefix: PartPlan("norm", "rmsnorm", {"size": cfg.hidden, "eps": cfg.eps}, prefix)
        rotary = lambda: PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": cfg.theta})
        attention = lambda prefix, **extra: PartPlan("mixer", "attention", {
            "hidden": cfg.hidden, "heads": cfg.heads, "kv_heads": cfg.kv_heads, "head_dim": hd, "position": rotary(),
            **extra}, prefix)
        mlp = lambda prefix: PartPlan("feed_forward", "gated_mlp", {"hidden": cfg.hidden, "inner": cfg.inner}, prefix)
        mixers = [attention("l0.attn."), PartPlan("mixer", "toy_running_mean", {"hidden": cfg.hidden}, "l1.mean."),
                  attention("l2.attn.", window=cfg.window), attention("l3.attn.", own_kv=False)]
        layers = [LayerPlan("pre_norm", {"mixer_norm": norm(f"l{i}.n1."), "mixer": m, "ffn_norm": norm(f"l{i}.n2."),
                                         "ffn": mlp(f"l{i}.mlp.")}) for i, m in enumerate(mixers)]
        # layer 0 runs twice (slots 0 and 3); layer 3 reads what layer 0's first run cached
        schedule = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2), LayerCall(3, 0, writes=False), LayerCall(0, 3)]
        return ModelPlan("ToyMeanForCausalLM", cfg, cfg.hidden, cfg.vocab, 512, (0,),
                         PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.hidden}, "embed."),
                         layers, schedule, norm("final."),
                         PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.hidden, "tied": True}, "head."))

    S.register_architecture("ToyMeanForCausalLM", ToyConfig, build_toy, model_types=("toy_mean",))


TOY = dict(model_type="toy_mean", hidden=48, inner=80, vocab=97, heads=3, kv_heads=1, window=6, eps=1e-5, theta=1e4)


def plain_toy_logits(w, tokens, store):
    c = TOY
    hd = c["hidden"] // c["heads"]
    pos = np.arange(len(tokens))
    x = P.f32(w["embed.weight"][np.asarray(tokens)])

    def mlp(x, i):
        n = store(P.rms_norm(x, w[f"l{i}.n2.weight"], c["eps"]))
        gate, up = store(P.linear(n, w[f"l{i}.mlp.gate_proj.weight"])), store(P.linear(n, w[f"l{i}.mlp.up_proj.weight"]))
        return P.f32(x + P.linear(store(P.swiglu(gate, up)), w[f"l{i}.mlp.down_proj.weight"]))

    def attn(x, i, window=None, kv=None):
        n = store(P.rms_norm(x, w[f"l{i}.n1.weight"], c["eps"]))
        p = f"l{i}.attn."
        q = store(P.rope_neox(store(P.linear(n, w[p + "q_proj.weight"], w[p + "q_proj.bias"])), pos, hd, c["theta"]))
        if kv is None:
            k = store(P.rope_neox(store(P.linear(n, w[p + "k_proj.weight"], w[p + "k_proj.bias"])), pos, hd, c["theta"]))
            v = store(P.linear(n, w[p + "v_proj.weight"], w[p + "v_proj.bias"]))
        else:
            k, v = kv
        a = store(P.causal_gqa_attention(q, k, v, c["heads"], c["kv_heads"], hd, window=window))
        return P.f32(x + P.linear(a, w[p + "o_proj.weight"])), (k, v)

    x, kv0 = attn(x, 0)
    x = mlp(x, 0)
    n = store(P.rms_norm(x, w["l1.n1.weight"], c["eps"])).astype(np.float64)
    mean = store(np.cumsum(n, 0) / np.arange(1, len(tokens) + 1)[:, None])
    x = mlp(P.f32(x + P.linear(mean, w["l1.mean.proj.weight"])), 1)
    x, _ = attn(x, 2, window=c["window"])
    x = mlp(x, 2)
    x, _ = attn(x, 3, kv=kv0)
    x = mlp(x, 3)
    x, _ = attn(x, 0)
    x = mlp(x, 0)
    return P.linear(store(P.rms_norm(x, w["final.weight"], c["eps"])), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_registers_builds_and_steps(tmp_path, dtype):
    register_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    folder = str(tmp_path / "toy")
    write_model_folder(folder, S.config_from_dict(TOY), seed=3, dtype=torch.bfloat16, std=0.15)
    assert json.load(open(os.path.join(folder, "config.json")))["architectures"] == ["ToyMeanForCausalLM"]
    runner = ModelRunner.from_folder(folder, dtype, block_size=4, num_blocks=40, max_sequences=3)
    assert runner.parts.graph_safe                           # every part says so, the toy mixer included
    kinds = [(g.spec.window, g.slots) for g in runner.cache.groups]
    assert kinds == [(None, [0, 3]), (6, [2])] and runner.cache.state_groups[0].slots == [1]
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    requests = {"a": H.random_tokens(97, 41, 1), "b": H.random_tokens(97, 23, 2), "c": H.random_tokens(97, 30, 3)}
    want = {k: plain_toy_logits(w, t, store) for k, t in requests.items()}
    tol = 3e-5 if dtype == "float32" else 4e-2
    # a and b run beside each other in uneven portions; c starts when b has ended, in b's state slot and pages
    seqs = {"a": runner.cache.create(), "b": runner.cache.create()}
    fed = {k: 0 for k in requests}
    plan = [{"a": 9, "b": 2}, {"a": 1, "b": 13}, {"a": 5, "b": 8}, {"a": 1}, {"a": 3, "c": 11}, {"a": 1, "c": 1},
            {"a": 21, "c": 2}, {"c": 16}]
    worst = 0.0
    for step in plan:
        if "c" in step and "c" not in seqs:
            seqs.pop("b").release()
            seqs["c"] = runner.cache.create()
        entries, rows = [], []
        for rid, n in step.items():
            n = min(n, len(requests[rid]) - fed[rid])
            assert runner.cache.reserve(seqs[rid], fed[rid] + n)
            entries.append(StepEntry(seqs[rid], requests[rid][fed[rid]:fed[rid] + n], list(range(n))))
            rows += [(rid, fed[rid] + i) for i in range(n)]
            fed[rid] += n
        got = runner.step(entries).cpu().numpy()
        for row, (rid, pos) in zip(got, rows):
            err = np.abs(row - want[rid][pos]).max()
            worst = max(worst, err)
            assert err <= tol * (1 + np.abs(want[rid][pos]).max()), f"{rid} position {pos}: {err:.3e}"
    assert fed == {k: len(v) for k, v in requests.items()}
    for s in seqs.values():
        s.release()
    assert runner.cache.free_pages() == [40, 40]
    print(f"toy {dtype}: worst error {worst:.3e}")


def test_toy_architecture_decodes_through_recorded_graphs(tmp_path):
    """What decides whether steps of single tokens are replayed from recorded graphs is the parts' own word
    (`graph_safe`), not the kind of cache a model has: the toy model, with per-request state and a windowed
    group that gives pages back under way, replays, and every replay's logits are the plain side's.  Three
    requests make a step of four rows: the padded row keeps its state in the spare slot."""
    register_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.cache import FREED
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.sampling import SamplingParams
    from sprout_lm_amd.weights import write_model_folder
    folder = str(tmp_path / "toy")
    write_model_folder(folder, S.config_from_dict(TOY), seed=3, dtype=torch.bfloat16, std=0.15)
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_folder(folder, dtype, block_size=4, num_blocks=40, max_sequences=3)
        store = P.bf16_round if dtype == "bfloat16" else P.f32
        requests = {"a": H.random_tokens(97, 30, 11), "b": H.random_tokens(97, 19, 12), "c": H.random_tokens(97, 25, 13)}
        want = {k: plain_toy_logits(w, t, store) for k, t in requests.items()}
        tol = 3e-5 if dtype == "float32" else 4e-2
        seqs = {k: runner.cache.create() for k in requests}
        fed = {"a": 9, "b": 2, "c": 14}
        for k, n in fed.items():                                # the prompts' first portions, eagerly
            assert runner.cache.reserve(seqs[k], n)
            runner.step([StepEntry(seqs[k], requests[k][:n], [])])
        spare = runner.cache.spare_state_slot
        state_before = runner.cache.state_groups[0].data[0, spare].clone()
        steps = 0
        while seqs:
            names = list(seqs)
            entries = []
            for k in names:
                assert runner.cache.reserve(seqs[k], fed[k] + 1)
                entries.append(StepEntry(seqs[k], [requests[k][fed[k]]], [0]))
            pending = runner.launch_decode(entries, [SamplingParams()] * len(names), [0] * len(names))
            assert pending is not None
            runner.finish_decode(pending)
            got = pending.logits[:len(names)].cpu().numpy()
            for row, k in zip(got, names):
                err = np.abs(row - want[k][fed[k]]).max()
                assert err <= tol * (1 + np.abs(want[k][fed[k]]).max()), f"{dtype} {k} position {fed[k]}: {err:.3e}"
                fed[k] += 1
                if fed[k] == len(requests[k]):
                    seqs.pop(k).release()
            steps += 1
            if steps == 5:
                assert FREED in seqs["a"].blocks[1]             # the window has given pages back under way
        assert runner._graphs.replays == steps and steps == 21
        # the padded row of the first steps ran like any other row; what it added up lies in the spare slot
        assert not torch.equal(runner.cache.state_groups[0].data[0, spare], state_before)
        assert runner.cache.free_pages() == [40, 40]


# A second toy architecture: a feed-forward with routing and a position encoding of its own, both
# registered here and nowhere in the engine.

def register_routed_toy():
    from dataclasses import dataclass
    from typing import ClassVar

    import sprout_lm_amd as S
    from sprout_lm_amd import ops
    from sprout_lm_amd.config.base import ModelConfig
    from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
    from sprout_lm_amd.parts import FeedForward, PositionEncoding, register_part, registered_parts
    from sprout_lm_amd.weights import TensorSpec

    if "toy_top1_experts" in registered_parts("feed_forward"):
        return

    @register_part("position", "toy_stretched_rotary")
    class StretchedRotary(PositionEncoding):
        """Rotation of the first `rotary_dim` dims of a head only, with positions divided by `stretch`."""

        graph_safe = True

        def __init__(self, head_dim, theta, rotary_dim, stretch):
            self.head_dim, self.theta, self.rotary_dim, self.stretch = head_dim, theta, rotary_dim, stretch
            self.inv_freq = None

        def prepare(self, device, dtype):
            d = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
            self.inv_freq = (float(self.theta) ** (-d / self.rotary_dim) / self.stretch).to(torch.float32).to(device)

    @register_part("feed_forward", "toy_top1_experts")
    class Top1Experts(FeedForward):
        """Every token goes to the expert with the largest router logit; its SwiGLU output is weighted with
        that expert's softmax probability.  Router logits and probabilities are float32."""

        def __init__(self, hidden, inner, experts):
            self.hidden, self.inner, self.experts = hidden, inner, experts

        def tensors(self):
            out = {"router.weight": TensorSpec((self.experts, self.hidden))}
            for e in range(self.experts):
                out[f"experts.{e}.gate_up.weight"] = TensorSpec((2 * self.inner, self.hidden))
                out[f"experts.{e}.down.weight"] = TensorSpec((self.hidden, self.inner))
            return out

        def forward(self, ctx, h, residual):
            T = h.shape[0]
            logits = torch.empty(T, self.experts, dtype=torch.float32, device=h.device)
            ops.gemm(h, self.w["router.weight"], logits)
            prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
            for e in range(self.experts):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel() == 0:
                    continue
                x = h[rows].contiguous()
                gu = torch.empty(x.shape[0], 2 * self.inner, dtype=h.dtype, device=h.device)
                ops.gemm(x, self.w[f"experts.{e}.gate_up.weight"], gu)
                act = torch.empty(x.shape[0], self.inner, dtype=h.dtype, device=h.device)
                ops.silu_mul(gu, act)
                y = torch.empty(x.shape[0], self.hidden, dtype=torch.float32, device=h.device)
                ops.gemm(act, self.w[f"experts.{e}.down.weight"], y)
                residual.index_add_(0, rows, y * prob[rows, None])

    @dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyRoutedForCausalLM"
        model_types: ClassVar[tuple] = ("toy_routed",)
        hidden: int = 0
        inner: int = 0
        vocab: int = 0
        heads: int = 0
        kv_heads: int = 0
        experts: int = 0
        rotary_dim: int = 0
        stretch: float = 0.0
        eps: float = 0.0
        theta: float = 0.0

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "experts", "rotary_dim",
                                               "stretch", "eps", "theta")})

        def to_dict(self):
            return {"architectures": [self.architecture], "model_type": "toy_routed",
                    **{k: getattr(self, k) for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "experts",
                                                      "rotary_dim", "stretch", "eps", "theta")}}

    def build(cfg):
        hd = cfg.hidden // cfg.heads
        norm = lambda prefix: PartPlan("norm", "rmsnorm", {"size": cfg.hidden, "eps": cfg.eps}, prefix)
        attention = lambda prefix, position: PartPlan("mixer", "attention", {
            "hidden": cfg.hidden, "heads": cfg.heads, "kv_heads": cfg.kv_heads, "head_dim": hd, "position": position,
            "qkv_bias": False}, prefix)
        stretched = PartPlan("position", "toy_stretched_rotary", {"head_dim": hd, "theta": cfg.theta,
                                                                   "rotary_dim": cfg.rotary_dim, "stretch": cfg.stretch})
        layers = [
            LayerPlan("pre_norm", {"mixer_norm": norm("l0.n1."), "mixer": attention("l0.attn.", stretched),
                                   "ffn_norm": norm("l0.n2."),
                                   "ffn": PartPlan("feed_forward", "toy_top1_experts",
                                                   {"hidden": cfg.hidden, "inner": cfg.inner, "experts": cfg.experts},
                                                   "l0.moe.")}),
            LayerPlan("pre_norm", {"mixer_norm": norm("l1.n1."),
                                   "mixer": attention("l1.attn.", PartPlan("position", "none", {"head_dim": hd})),
                                   "ffn_norm": norm("l1.n2."),
                                   "ffn": PartPlan("feed_forward", "gated_mlp", {"hidden": cfg.hidden, "inner": cfg.inner},
                                                   "l1.mlp.")}),
        ]
        return ModelPlan("ToyRoutedForCausalLM", cfg, cfg.hidden, cfg.vocab, 512, (0,),
                         PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.hidden}, "embed."),
                         layers, [LayerCall(0, 0), LayerCall(1, 1)], norm("final."),
                         PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.hidden, "tied": False}, "head."))

    S.register_architecture("ToyRoutedForCausalLM", RoutedConfig, build, model_types=("toy_routed",))


ROUTED = dict(model_type="toy_routed", hidden=64, inner=48, vocab=101, heads=2, kv_heads=2, experts=3, rotary_dim=16,
              stretch=4.0, eps=1e-6, theta=5e3)


def plain_routed_logits(w, tokens, store):
    """The routed toy, whole sequence.  Returns the logits and, per token, the gap between the two largest
    router logits (a token on the edge between two experts may go either way in bfloat16)."""
    c = ROUTED
    hd = c["hidden"] // c["heads"]
    pos = np.arange(len(tokens), dtype=np.float64)
    x = P.f32(w["embed.weight"][np.asarray(tokens)])

    def stretched_rope(t):
        t = np.asarray(t, dtype=np.float64).reshape(len(tokens), c["heads"], hd).copy()
        half = c["rotary_dim"] // 2
        d = np.arange(half, dtype=np.float64)
        angle = (pos / c["stretch"])[:, None] / c["theta"] ** (2.0 * d / c["rotary_dim"])
        cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
        a, b = t[..., :half].copy(), t[..., half:2 * half].copy()
        t[..., :half] = a * cos - b * sin
        t[..., half:2 * half] = b * cos + a * sin
        return P.f32(t.reshape(len(tokens), -1))

    def attn(x, i, rotate):
        n = store(P.rms_norm(x, w[f"l{i}.n1.weight"], c["eps"]))
        p = f"l{i}.attn."
        q, k, v = (store(P.linear(n, w[p + f"{name}_proj.weight"])) for name in "qkv")
        if rotate:
            q, k = store(stretched_rope(q)), store(stretched_rope(k))
        a = store(P.causal_gqa_attention(q, k, v, c["heads"], c["kv_heads"], hd))
        return P.f32(x + P.linear(a, w[p + "o_proj.weight"]))

    x = attn(x, 0, True)
    n = store(P.rms_norm(x, w["l0.n2.weight"], c["eps"]))
    logits = np.asarray(P.linear(n, w["l0.moe.router.weight"]), dtype=np.float64)
    top = np.sort(logits, axis=-1)
    gap = top[:, -1] - top[:, -2]
    prob = np.exp(logits - logits.max(-1, keepdims=True))
    prob /= prob.sum(-1, keepdims=True)
    choice = logits.argmax(-1)
    out = np.zeros_like(x, dtype=np.float64)
    for e in range(c["experts"]):
        rows = np.nonzero(choice == e)[0]
        if len(rows) == 0:
            continue
        gu = store(P.linear(n[rows], w[f"l0.moe.experts.{e}.gate_up.weight"]))
        act = store(P.swiglu(gu[:, :c["inner"]], gu[:, c["inner"]:]))
        out[rows] = np.asarray(P.linear(act, w[f"l0.moe.experts.{e}.down.weight"]), dtype=np.float64) * prob[rows, e, None]
    x = P.f32(x + out)
    x = attn(x, 1, False)
    n = store(P.rms_norm(x, w["l1.n2.weight"], c["eps"]))
    gate, up = store(P.linear(n, w["l1.mlp.gate_proj.weight"])), store(P.linear(n, w["l1.mlp.up_proj.weight"]))
    x = P.f32(x + P.linear(store(P.swiglu(gate, up)), w["l1.mlp.down_proj.weight"]))
    return P.linear(store(P.rms_norm(x, w["final.weight"], c["eps"])), w["head.weight"]), gap


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_another_position_encoding(tmp_path, dtype):
    """A feed-forward with routing (router logits and probabilities in float32) and a position encoding that the
    engine does not have, defined and registered in this file, built from a model folder and stepped in portions
    beside another request."""
    register_routed_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    folder = str(tmp_path / "routed")
    write_model_folder(folder, S.config_from_dict(ROUTED), seed=5, dtype=torch.bfloat16, std=0.2)
    runner = ModelRunner.from_folder(folder, dtype, block_size=8, num_blocks=24, max_sequences=2)
    assert not runner.parts.graph_safe                        # the routed feed-forward decides on the host
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    requests = {"a": H.random_tokens(101, 37, 7), "b": H.random_tokens(101, 20, 8)}
    want = {k: plain_routed_logits(w, t, store) for k, t in requests.items()}
    tol = 3e-5 if dtype == "float32" else 4e-2
    seqs = {k: runner.cache.create() for k in requests}
    fed = {k: 0 for k in requests}
    used = set()
    checked = 0
    for step in [{"a": 11, "b": 3}, {"a": 1, "b": 9}, {"a": 2, "b": 1}, {"a": 23, "b": 7}]:
        entries, rows = [], []
        for rid, n in step.items():
            assert runner.cache.reserve(seqs[rid], fed[rid] + n)
            entries.append(StepEntry(seqs[rid], requests[rid][fed[rid]:fed[rid] + n], list(range(n))))
            rows += [(rid, fed[rid] + i) for i in range(n)]
            fed[rid] += n
        got = runner.step(entries).cpu().numpy()
        for row, (rid, pos) in zip(got, rows):
            logits, gap = want[rid]
            # a token's own routing must be clear of ties, and so must that of every earlier token it attends to
            if gap[:pos + 1].min() < 0.05:
                continue
            checked += 1
            err = np.abs(row - logits[pos]).max()
            assert err <= tol * (1 + np.abs(logits[pos]).max()), f"{rid} position {pos}: {err:.3e}"
    assert fed == {k: len(v) for k, v in requests.items()} and checked >= 20
    for s in seqs.values():
        s.release()
    assert runner.cache.free_pages() == [24]             # both layers have the same needs: one group of pages


def register_windowed_toy():
    """Two layers of the engine's own parts, the second with a window: two cache groups and no state."""
    from dataclasses import dataclass
    from typing import ClassVar

    import sprout_lm_amd as S
    from sprout_lm_amd.config.base import ModelConfig
    from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
    from sprout_lm_amd.registry import registered_architectures

    if "ToyWindowForCausalLM" in registered_architectures():
        return

    @dataclass(frozen=True)
    class WindowConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyWindowForCausalLM"
        model_types: ClassVar[tuple] = ("toy_window",)
        hidden: int = 0
        inner: int = 0
        vocab: int = 0
        heads: int = 0
        kv_heads: int = 0
        window: int = 0
        window_page: int = 0       # tokens in a page of the windowed layer's cache
        eps: float = 0.0
        theta: float = 0.0

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "window", "window_page",
                                              "eps", "theta")})

        def to_dict(self):
            return {"architectures": [self.architecture], "model_type": "toy_window", "hidden": self.hidden,
                    "inner": self.inner, "vocab": self.vocab, "heads": self.heads, "kv_heads": self.kv_heads,
                    "window": self.window, "window_page": self.window_page, "eps": self.eps, "theta": self.theta}

    def build(cfg):
        hd = cfg.hidden // cfg.heads
        norm = lambda prefix: PartPlan("norm", "rmsnorm", {"size": cfg.hidden, "eps": cfg.eps}, prefix)
        attention = lambda prefix, **extra: PartPlan("mixer", "attention", {
            "hidden": cfg.hidden, "heads": cfg.heads, "kv_heads": cfg.kv_heads, "head_dim": hd,
            "position": PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": cfg.theta}), **extra}, prefix)
        mlp = lambda prefix: PartPlan("feed_forward", "gated_mlp", {"hidden": cfg.hidden, "inner": cfg.inner}, prefix)
        mixers = [attention("l0.attn."), attention("l1.attn.", window=cfg.window, page_tokens=cfg.window_page)]
        layers = [LayerPlan("pre_norm", {"mixer_norm": norm(f"l{i}.n1."), "mixer": m, "ffn_norm": norm(f"l{i}.n2."),
                                         "ffn": mlp(f"l{i}.mlp.")}) for i, m in enumerate(mixers)]
        return ModelPlan("ToyWindowForCausalLM", cfg, cfg.hidden, cfg.vocab, 512, (0,),
                         PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.hidden}, "embed."),
                         layers, [LayerCall(0, 0), LayerCall(1, 1)], norm("final."),
                         PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.hidden, "tied": True}, "head."))

    S.register_architecture("ToyWindowForCausalLM", WindowConfig, build, model_types=("toy_window",))


WINDOWED = dict(model_type="toy_window", hidden=64, inner=96, vocab=89, heads=4, kv_heads=2, window=10, window_page=4,
                eps=1e-6, theta=1e4)


def plain_windowed_logits(w, tokens, store):
    c = WINDOWED
    hd = c["hidden"] // c["heads"]
    pos = np.arange(len(tokens))
    x = P.f32(w["embed.weight"][np.asarray(tokens)])
    for i, window in enumerate([None, c["window"]]):
        p = f"l{i}.attn."
        n = store(P.rms_norm(x, w[f"l{i}.n1.weight"], c["eps"]))
        q = store(P.rope_neox(store(P.linear(n, w[p + "q_proj.weight"], w[p + "q_proj.bias"])), pos, hd, c["theta"]))
        k = store(P.rope_neox(store(P.linear(n, w[p + "k_proj.weight"], w[p + "k_proj.bias"])), pos, hd, c["theta"]))
        v = store(P.linear(n, w[p + "v_proj.weight"], w[p + "v_proj.bias"]))
        a = store(P.causal_gqa_attention(q, k, v, c["heads"], c["kv_heads"], hd, window=window))
        x = P.f32(x + P.linear(a, w[p + "o_proj.weight"]))
        n = store(P.rms_norm(x, w[f"l{i}.n2.weight"], c["eps"]))
        gate, up = store(P.linear(n, w[f"l{i}.mlp.gate_proj.weight"])), store(P.linear(n, w[f"l{i}.mlp.up_proj.weight"]))
        x = P.f32(x + P.linear(store(P.swiglu(gate, up)), w[f"l{i}.mlp.down_proj.weight"]))
    return P.linear(store(P.rms_norm(x, w["final.weight"], c["eps"])), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window_page", [4, 2])
def test_a_windowed_layer_shares_prefix_pages(tmp_path, dtype, window_page):
    """A model with a layer that keeps every key and one with a window of 10 (pages of 4; the windowed layer's own
    pages of 4 or of 2 tokens): a second request takes over the pages of a shared prefix in both cache groups, in
    the windowed one only those its window still covers (the earlier places of its block table say `given back`),
    and computes on from there; a third one after the first two have ended finds the pages in the cache alone.
    Every logit row of the later requests against the plain implementation, which knows no cache."""
    register_windowed_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.cache import FREED
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    folder = str(tmp_path / "windowed")
    write_model_folder(folder, S.config_from_dict(dict(WINDOWED, window_page=window_page)), seed=17, dtype=torch.bfloat16,
                       std=0.15)
    runner = ModelRunner.from_folder(folder, dtype, block_size=4, num_blocks=40, max_sequences=3, prefix_caching=True)
    cache = runner.cache
    per = 4 // window_page                                # the windowed group's pages in four tokens
    assert cache.prefix_caching and [(g.spec.window, g.page_tokens) for g in cache.groups] == [(None, 4), (10, window_page)]
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    tol = 3e-5 if dtype == "float32" else 4e-2
    shared = H.random_tokens(89, 30, 5)
    requests = {"a": shared + H.random_tokens(89, 9, 6), "b": shared[:26] + H.random_tokens(89, 15, 7),
                "c": shared[:22] + H.random_tokens(89, 11, 8)}

    def run(rid, seq, portions):
        tokens, worst = requests[rid], 0.0
        want = plain_windowed_logits(w, tokens, store)
        for n in portions:
            old, new = seq.length, min(len(tokens), seq.length + n)
            if new == old:
                break
            assert cache.reserve(seq, new)
            got = runner.step([StepEntry(seq, tokens[old:new], list(range(new - old)))]).cpu().numpy()
            for boundary in range((old // 4 + 1) * 4, new + 1, 4):
                cache.publish(tokens, seq, boundary)
            for i, row in enumerate(got):
                err = np.abs(row - want[old + i]).max() / (tol * (1 + np.abs(want[old + i]).max()))
                worst = max(worst, err)
                assert err <= 1.0, f"{rid} position {old + i}: {err:.2f} of the bound"
        assert seq.length == len(tokens)
        return worst

    a = cache.create()
    worst = run("a", a, [3] * 20)                       # portions shorter than the window: every page is offered live
    b = cache.reuse_prefix(requests["b"])
    assert b.length == 24 and b.blocks[0] == a.blocks[0][:6]
    # b computes position 24 next and reads keys from 15 on: the windowed group's pages of tokens 12..23, which a wrote
    assert b.blocks[1][:3 * per] == [FREED] * (3 * per) and FREED not in b.blocks[1][3 * per:6 * per]
    assert set(b.blocks[1][3 * per:6 * per]) <= {p for e in cache._prefixes.values() for p in e.pages[1] or ()}
    worst = max(worst, run("b", b, [5, 1, 1, 9, 4]))
    a.release(); b.release()
    c = cache.reuse_prefix(requests["c"])               # only the cache holds the pages now
    assert c.length == 20 and c.blocks[1][:2 * per] == [FREED] * (2 * per) and FREED not in c.blocks[1][2 * per:5 * per]
    # the last tokens of c one by one through recorded decode steps: block tables of two groups with pages of
    # different sizes in the graph's static buffers
    from sprout_lm_amd.sampling import SamplingParams
    tokens_c, want_c = requests["c"], plain_windowed_logits(w, requests["c"], store)
    requests["c"] = tokens_c[:-4]
    worst = max(worst, run("c", c, [2, 7]))
    requests["c"] = tokens_c
    for position in range(len(tokens_c) - 4, len(tokens_c)):
        assert cache.reserve(c, position + 1)
        pending = runner.launch_decode([StepEntry(c, [tokens_c[position]], [0])], [SamplingParams()], [0])
        assert pending is not None, "the step did not run from a recorded graph"
        runner.finish_decode(pending)
        err = np.abs(pending.logits[0].cpu().numpy() - want_c[position]).max() / (tol * (1 + np.abs(want_c[position]).max()))
        worst = max(worst, err)
        assert err <= 1.0, f"c position {position} through a recorded step: {err:.2f} of the bound"
    assert c.length == len(tokens_c)
    c.release()
    cache.clear_prefixes()
    assert cache.free_pages() == [40, 40 * per]
    print(f"windowed prefix sharing {dtype}: worst {worst:.2f} of the bound")


# A third toy architecture: a layer that holds TWO mixers which both keep something (attention with pages beside a
# running mean whose state comes as two named pieces), in a block kind of its own, and a per-token array that the
# engine does not know (the token's segment), registered here and delivered to eager and recorded steps alike.

def register_dual_toy():
    from dataclasses import dataclass
    from typing import ClassVar

    import sprout_lm_amd as S
    from sprout_lm_amd import ops
    from sprout_lm_amd.cache import StateSpec
    from sprout_lm_amd.config.base import ModelConfig
    from sprout_lm_amd.engine.batch import register_step_array
    from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
    from sprout_lm_amd.parts import Block, Mixer, register_part, registered_parts
    from sprout_lm_amd.weights import TensorSpec

    if "toy_segment_mean" in registered_parts("mixer"):
        return

    register_step_array("toy_segment", "token", lambda layout: layout.positions // 7)

    @register_part("mixer", "toy_segment_mean")
    class SegmentMean(Mixer):
        """y_t = W . mean(h_0 .. h_t) + bias[segment(t) % 4].  The state is kept as two named pieces, the running
        sum and the count; the segment of every token comes from the step array registered above."""

        graph_safe = True

        def __init__(self, hidden):
            self.hidden = hidden

        def cache_spec(self):
            return {"sum": StateSpec((self.hidden,), "float32"), "count": StateSpec((1,), "float32")}

        def tensors(self):
            return {"proj.weight": TensorSpec((self.hidden, self.hidden)), "segment_bias.weight": TensorSpec((4, self.hidden))}

        def forward(self, ctx, h, residual, cache):
            total, count = cache["sum"].state, cache["count"].state
            if ctx.max_q_len == 1:
                slots = ctx.state_slots.long()
                sums = total.index_select(0, slots) + h.float()
                counts = count.index_select(0, slots) + 1
                mean = (sums / counts).to(h.dtype).contiguous()
                ops.gemm(mean, self.w["proj.weight"], residual, accumulate=True)
                total.index_copy_(0, slots, sums)
                count.index_copy_(0, slots, counts)
            else:
                for start, n, slot in zip(ctx.host["q_start"], ctx.host["q_len"], ctx.host["state_slots"]):
                    sums = torch.cumsum(h[start:start + n].float(), 0) + total[slot]
                    counts = count[slot] + torch.arange(1, n + 1, device=h.device, dtype=torch.float32)[:, None]
                    mean = (sums / counts).to(h.dtype).float()
                    residual[start:start + n] += mean @ self.w["proj.weight"].float().T
                    total[slot] = sums[-1]
                    count[slot] = counts[-1]
            segment = (ctx.extra["toy_segment"][:h.shape[0]] % 4).long()
            residual.add_(self.w["segment_bias.weight"].float().index_select(0, segment))

    @register_part("block", "toy_two_mixers")
    class TwoMixers(Block):
        """x += attention(norm(x)) + mean(norm(x)); x += feed_forward(norm(x))."""

        graph_safe = True

        def __init__(self, norm, attn, mean, ffn_norm, ffn):
            self.norm, self.attn, self.mean, self.ffn_norm, self.ffn = norm, attn, mean, ffn_norm, ffn

        def parts(self):
            return {"norm": self.norm, "attn": self.attn, "mean": self.mean, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

        def forward(self, ctx, residual, caches):
            T, Hd = residual.shape
            h = ctx.buffer("normed", (T, Hd), ctx.act_dtype)
            self.norm.forward(ctx, residual, h)
            self.attn.forward(ctx, h, residual, caches["attn"])
            self.mean.forward(ctx, h, residual, caches["mean"])
            self.ffn_norm.forward(ctx, residual, h)
            self.ffn.forward(ctx, h, residual)

    @dataclass(frozen=True)
    class DualConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyDualForCausalLM"
        model_types: ClassVar[tuple] = ("toy_dual",)
        hidden: int = 0
        inner: int = 0
        vocab: int = 0
        heads: int = 0
        kv_heads: int = 0
        layers: int = 0
        eps: float = 0.0
        theta: float = 0.0

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "layers", "eps", "theta")})

        def to_dict(self):
            return {"architectures": [self.architecture], "model_type": "toy_dual",
                    **{k: getattr(self, k) for k in ("hidden", "inner", "vocab", "heads", "kv_heads", "layers", "eps", "theta")}}

    def build(cfg):
        hd = cfg.hidden // cfg.heads
        norm = lambda prefix: PartPlan("norm", "rmsnorm", {"size": cfg.hidden, "eps": cfg.eps}, prefix)
        layers, schedule = [], []
        for i in range(cfg.layers):
            layers.append(LayerPlan("toy_two_mixers", {
                "norm": norm(f"l{i}.n1."),
                "attn": PartPlan("mixer", "attention", {
                    "hidden": cfg.hidden, "heads": cfg.heads, "kv_heads": cfg.kv_heads, "head_dim": hd,
                    "position": PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": cfg.theta})}, f"l{i}.attn."),
                "mean": PartPlan("mixer", "toy_segment_mean", {"hidden": cfg.hidden}, f"l{i}.mean."),
                "ffn_norm": norm(f"l{i}.n2."),
                "ffn": PartPlan("feed_forward", "gated_mlp", {"hidden": cfg.hidden, "inner": cfg.inner}, f"l{i}.mlp.")}))
            schedule.append(LayerCall(i, {"attn": 3 * i, "mean.sum": 3 * i + 1, "mean.count": 3 * i + 2}))
        return ModelPlan("ToyDualForCausalLM", cfg, cfg.hidden, cfg.vocab, 512, (0,),
                         PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.hidden}, "embed."),
                         layers, schedule, norm("final."),
                         PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.hidden, "tied": True}, "head."))

    S.register_architecture("ToyDualForCausalLM", DualConfig, build, model_types=("toy_dual",))


DUAL = dict(model_type="toy_dual", hidden=64, inner=112, vocab=113, heads=4, kv_heads=2, layers=2, eps=1e-5, theta=1e4)


def plain_dual_logits(w, tokens, store):
    c = DUAL
    hd = c["hidden"] // c["heads"]
    pos = np.arange(len(tokens))
    x = P.f32(w["embed.weight"][np.asarray(tokens)])
    for i in range(c["layers"]):
        n = store(P.rms_norm(x, w[f"l{i}.n1.weight"], c["eps"]))
        p = f"l{i}.attn."
        q = store(P.rope_neox(store(P.linear(n, w[p + "q_proj.weight"], w[p + "q_proj.bias"])), pos, hd, c["theta"]))
        k = store(P.rope_neox(store(P.linear(n, w[p + "k_proj.weight"], w[p + "k_proj.bias"])), pos, hd, c["theta"]))
        v = store(P.linear(n, w[p + "v_proj.weight"], w[p + "v_proj.bias"]))
        a = store(P.causal_gqa_attention(q, k, v, c["heads"], c["kv_heads"], hd))
        x = P.f32(x + P.linear(a, w[p + "o_proj.weight"]))
        mean = store(np.cumsum(n.astype(np.float64), 0) / np.arange(1, len(tokens) + 1)[:, None])
        x = P.f32(x + P.linear(mean, w[f"l{i}.mean.proj.weight"]))
        x = P.f32(x + w[f"l{i}.mean.segment_bias.weight"][(pos // 7) % 4])
        n = store(P.rms_norm(x, w[f"l{i}.n2.weight"], c["eps"]))
        gate, up = store(P.linear(n, w[f"l{i}.mlp.gate_proj.weight"])), store(P.linear(n, w[f"l{i}.mlp.up_proj.weight"]))
        x = P.f32(x + P.linear(store(P.swiglu(gate, up)), w[f"l{i}.mlp.down_proj.weight"]))
    return P.linear(store(P.rms_norm(x, w["final.weight"], c["eps"])), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_with_two_mixers_that_both_keep_something(tmp_path, dtype):
    """A block kind, a mixer and a per-token step array defined in this file: every layer holds attention (pages)
    beside a running mean (two named state tensors), so a call of the run order names three cache slots by part.
    Replayed whole, with the last tokens one by one, in portions down to two tokens and mixed with so few pages
    that they are used again, and decoded through recorded graphs: every row against the plain function."""
    register_dual_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.cache import StateSpec
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.engine.trace import TraceSession
    from sprout_lm_amd.sampling import SamplingParams
    from sprout_lm_amd.weights import write_model_folder
    from tests import traces
    folder = str(tmp_path / "dual")
    write_model_folder(folder, S.config_from_dict(DUAL), seed=29, dtype=torch.bfloat16, std=0.15)
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    tol = 3e-5 if dtype == "float32" else 4e-2
    requests = {f"r{i}": H.random_tokens(113, n, 40 + i) for i, n in enumerate([37, 9, 70, 44, 25, 61])}
    want = {k: plain_dual_logits(w, t, store) for k, t in requests.items()}
    pool = sum(sorted(-(-len(t) // 8) for t in requests.values())[-4:])        # pages of 8: the four longest fit, no more
    worst = 0.0
    for family, trace in (("whole", traces.whole(requests)), ("tail", traces.tail_decoded(requests, tail=20)),
                          ("portions", traces.portions(requests)), ("mixed", traces.mixed(requests, seed=5))):
        runner = ModelRunner.from_folder(folder, dtype, block_size=8, num_blocks=pool, max_sequences=4, prefix_caching=True)
        # three slots a layer, named by part: pages for the attention, two state tensors for the mean
        assert runner.parts.call_slots[1] == {"attn": (3, True), "mean.sum": (4, True), "mean.count": (5, True)}
        assert [g.slots for g in runner.cache.groups] == [[0, 3]]
        assert [(g.spec, g.slots) for g in runner.cache.state_groups] == [(StateSpec((64,)), [1, 4]), (StateSpec((1,)), [2, 5])]
        assert not runner.parts.prefix_sharing and not runner.cache.prefix_caching     # the plan's word, not the manager's
        session = TraceSession(runner)
        for record, rows in zip(trace.steps, trace.expected):
            logits = session.run_step(record)
            got = logits.cpu().numpy() if rows else None
            for i, (rid, pos) in enumerate(rows):
                err = np.abs(got[i] - want[rid][pos]).max() / (tol * (1 + np.abs(want[rid][pos]).max()))
                worst = max(worst, err)
                assert err <= 1.0, f"{family} {rid} position {pos}: {err:.2f} of the bound"
        assert runner.cache.free_pages() == [pool] and not session.live
    # three requests decoded through recorded graphs (a step of four rows, one of them padding)
    runner = ModelRunner.from_folder(folder, dtype, block_size=8, num_blocks=40, max_sequences=3)
    assert runner.parts.graph_safe and not runner.parts.graph_safe_portions
    names = ["r0", "r2", "r3"]
    seqs = {k: runner.cache.create() for k in names}
    fed = {"r0": 20, "r2": 31, "r3": 2}
    for k, n in fed.items():
        assert runner.cache.reserve(seqs[k], n)
        runner.step([StepEntry(seqs[k], requests[k][:n], [])])
    for _ in range(17):
        entries = []
        for k in names:
            assert runner.cache.reserve(seqs[k], fed[k] + 1)
            entries.append(StepEntry(seqs[k], [requests[k][fed[k]]], [0]))
        pending = runner.launch_decode(entries, [SamplingParams()] * 3, [0] * 3)
        assert pending is not None, "the step did not run from a recorded graph"
        runner.finish_decode(pending)
        got = pending.logits[:3].cpu().numpy()
        for row, k in zip(got, names):
            err = np.abs(row - want[k][fed[k]]).max() / (tol * (1 + np.abs(want[k][fed[k]]).max()))
            worst = max(worst, err)
            assert err <= 1.0, f"recorded decode {k} position {fed[k]}: {err:.2f} of the bound"
            fed[k] += 1
    assert runner._graphs.replays == 17
    print(f"two mixers a layer {dtype}: worst {worst:.2f} of the bound")


# A fourth toy: a mixer whose cached keys and values differ in width and are kept in float32 whatever the model
# computes in (`PagedKVSpec.value_dim`, `.dtype`).  No attention kernel of the engine takes such a cache; the toy
# gathers its pages itself.  What is shown is that the cache manager, the step's block tables and slot mapping and
# the runner serve a cache of that description without a change to the engine's files.

def register_latent_toy():
    from dataclasses import dataclass
    from typing import ClassVar

    import sprout_lm_amd as S
    from sprout_lm_amd import ops
    from sprout_lm_amd.cache import PagedKVSpec
    from sprout_lm_amd.config.base import ModelConfig
    from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
    from sprout_lm_amd.parts import Mixer, register_part, registered_parts
    from sprout_lm_amd.weights import TensorSpec

    if "toy_narrow_values" in registered_parts("mixer"):
        return

    @register_part("mixer", "toy_narrow_values")
    class NarrowValues(Mixer):
        """Causal attention of `heads` query heads over ONE cached key of width key_dim and ONE cached value of
        width value_dim per token (no position encoding): y = W_o . concat_h softmax(q_h . k / sqrt(key_dim)) . v."""

        def __init__(self, hidden, heads, key_dim, value_dim):
            self.hidden, self.heads, self.key_dim, self.value_dim = hidden, heads, key_dim, value_dim

        def cache_spec(self):
            return PagedKVSpec(1, self.key_dim, value_dim=self.value_dim, dtype="float32")

        def cache_elements_per_token(self):
            return self.key_dim + self.value_dim

        def tensors(self):
            return {"q.weight": TensorSpec((self.heads * self.key_dim, self.hidden)), "k.weight": TensorSpec((self.key_dim, self.hidden)),
                    "v.weight": TensorSpec((self.value_dim, self.hidden)), "o.weight": TensorSpec((self.hidden, self.heads * self.value_dim))}

        def forward(self, ctx, h, residual, cache):
            T = h.shape[0]
            out = {}
            for name, width in (("q", self.heads * self.key_dim), ("k", self.key_dim), ("v", self.value_dim)):
                out[name] = torch.empty(T, width, dtype=h.dtype, device=h.device)
                ops.gemm(h, self.w[f"{name}.weight"], out[name])
            pages, page = cache.k.shape[0], cache.page_size
            assert cache.k.shape == (pages, 1, page, self.key_dim) and cache.v.shape == (pages, 1, self.value_dim, page)
            assert cache.k.dtype == cache.v.dtype == torch.float32
            slots = cache.slot_mapping[:T].long()
            cache.k.view(pages * page, self.key_dim)[slots] = out["k"].float()
            cache.v[slots // page, 0, :, slots % page] = out["v"].float()
            mixed = torch.empty(T, self.heads * self.value_dim, dtype=torch.float32, device=h.device)
            for s, (start, n, length) in enumerate(zip(ctx.host["q_start"], ctx.host["q_len"], ctx.host["ctx_len"])):
                table = cache.block_tables[s, :-(-int(length) // page)].long()
                keys = cache.k[table, 0].reshape(-1, self.key_dim)[:length]
                values = cache.v[table, 0].permute(0, 2, 1).reshape(-1, self.value_dim)[:length]
                q = out["q"][start:start + n].float().view(n, self.heads, self.key_dim)
                scores = torch.einsum("nhd,kd->nhk", q, keys) / math.sqrt(self.key_dim)
                position = (length - n + torch.arange(n, device=h.device))[:, None, None]
                scores = scores.masked_fill(torch.arange(length, device=h.device)[None, None, :] > position, float("-inf"))
                mixed[start:start + n] = torch.einsum("nhk,kv->nhv", torch.softmax(scores, -1), values).reshape(n, -1)
            ops.gemm(mixed.to(h.dtype), self.w["o.weight"], residual, accumulate=True)

    @dataclass(frozen=True)
    class LatentConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyLatentForCausalLM"
        model_types: ClassVar[tuple] = ("toy_latent",)
        hidden: int = 0
        inner: int = 0
        vocab: int = 0
        heads: int = 0
        key_dim: int = 0
        value_dim: int = 0
        eps: float = 0.0

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in ("hidden", "inner", "vocab", "heads", "key_dim", "value_dim", "eps")})

        def to_dict(self):
            return {"architectures": [self.architecture], "model_type": "toy_latent",
                    **{k: getattr(self, k) for k in ("hidden", "inner", "vocab", "heads", "key_dim", "value_dim", "eps")}}

    def build(cfg):
        norm = lambda prefix: PartPlan("norm", "rmsnorm", {"size": cfg.hidden, "eps": cfg.eps}, prefix)
        mlp = lambda prefix: PartPlan("feed_forward", "gated_mlp", {"hidden": cfg.hidden, "inner": cfg.inner}, prefix)
        hd = cfg.hidden // cfg.heads
        mixers = [PartPlan("mixer", "attention", {"hidden": cfg.hidden, "heads": cfg.heads, "kv_heads": cfg.heads, "head_dim": hd,
                                                  "position": PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": 1e4})}, "l0.attn."),
                  PartPlan("mixer", "toy_narrow_values", {"hidden": cfg.hidden, "heads": cfg.heads, "key_dim": cfg.key_dim,
                                                          "value_dim": cfg.value_dim}, "l1.mix.")]
        layers = [LayerPlan("pre_norm", {"mixer_norm": norm(f"l{i}.n1."), "mixer": m, "ffn_norm": norm(f"l{i}.n2."),
                                         "ffn": mlp(f"l{i}.mlp.")}) for i, m in enumerate(mixers)]
        return ModelPlan("ToyLatentForCausalLM", cfg, cfg.hidden, cfg.vocab, 512, (0,),
                         PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.hidden}, "embed."),
                         layers, [LayerCall(0, 0), LayerCall(1, 1)], norm("final."),
                         PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.hidden, "tied": True}, "head."))

    S.register_architecture("ToyLatentForCausalLM", LatentConfig, build, model_types=("toy_latent",))


LATENT = dict(model_type="toy_latent", hidden=64, inner=96, vocab=103, heads=2, key_dim=24, value_dim=8, eps=1e-6)


def plain_latent_logits(w, tokens, store):
    c = LATENT
    hd = c["hidden"] // c["heads"]
    pos = np.arange(len(tokens))
    x = P.f32(w["embed.weight"][np.asarray(tokens)])

    def mlp(x, i):
        n = store(P.rms_norm(x, w[f"l{i}.n2.weight"], c["eps"]))
        gate, up = store(P.linear(n, w[f"l{i}.mlp.gate_proj.weight"])), store(P.linear(n, w[f"l{i}.mlp.up_proj.weight"]))
        return P.f32(x + P.linear(store(P.swiglu(gate, up)), w[f"l{i}.mlp.down_proj.weight"]))

    n = store(P.rms_norm(x, w["l0.n1.weight"], c["eps"]))
    p = "l0.attn."
    q = store(P.rope_neox(store(P.linear(n, w[p + "q_proj.weight"], w[p + "q_proj.bias"])), pos, hd, 1e4))
    k = store(P.rope_neox(store(P.linear(n, w[p + "k_proj.weight"], w[p + "k_proj.bias"])), pos, hd, 1e4))
    v = store(P.linear(n, w[p + "v_proj.weight"], w[p + "v_proj.bias"]))
    a = store(P.causal_gqa_attention(q, k, v, c["heads"], c["heads"], hd))
    x = mlp(P.f32(x + P.linear(a, w[p + "o_proj.weight"])), 0)
    n = store(P.rms_norm(x, w["l1.n1.weight"], c["eps"]))
    q = store(P.linear(n, w["l1.mix.q.weight"])).astype(np.float64).reshape(len(tokens), c["heads"], c["key_dim"])
    k = store(P.linear(n, w["l1.mix.k.weight"])).astype(np.float64)
    v = store(P.linear(n, w["l1.mix.v.weight"])).astype(np.float64)
    mixed = np.zeros((len(tokens), c["heads"] * c["value_dim"]))
    for t in range(len(tokens)):
        for h in range(c["heads"]):
            s = k[:t + 1] @ q[t, h] / math.sqrt(c["key_dim"])
            e = np.exp(s - s.max())
            mixed[t, h * c["value_dim"]:(h + 1) * c["value_dim"]] = (e / e.sum()) @ v[:t + 1]
    x = mlp(P.f32(x + P.linear(store(P.f32(mixed)), w["l1.mix.o.weight"])), 1)
    return P.linear(store(P.rms_norm(x, w["final.weight"], c["eps"])), w["embed.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_cache_whose_keys_and_values_differ_in_width(tmp_path, dtype):
    """Keys of 24 numbers, values of 8, both kept in float32 under either compute dtype, beside an ordinary
    attention layer: two cache groups, the toy's pools of the shapes and dtype it asked for; mixed replay with so
    few pages that they are used again, against the plain function."""
    register_latent_toy()
    import sprout_lm_amd as S
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.trace import TraceSession
    from sprout_lm_amd.weights import write_model_folder
    from tests import traces
    folder = str(tmp_path / "latent")
    write_model_folder(folder, S.config_from_dict(LATENT), seed=41, dtype=torch.bfloat16, std=0.15)
    from safetensors.torch import load_file
    w = {k: v.float().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    store = P.bf16_round if dtype == "bfloat16" else P.f32
    tol = 3e-5 if dtype == "float32" else 4e-2
    requests = {f"r{i}": H.random_tokens(103, n, 60 + i) for i, n in enumerate([37, 12, 58, 41, 26])}
    want = {k: plain_latent_logits(w, t, store) for k, t in requests.items()}
    pool = sum(sorted(-(-len(t) // 8) for t in requests.values())[-4:])
    runner = ModelRunner.from_folder(folder, dtype, block_size=8, num_blocks=pool, max_sequences=4)
    ordinary, narrow = runner.cache.groups
    assert narrow.k.shape == (1, pool, 1, 8, 24) and narrow.v.shape == (1, pool, 1, 8, 8) and narrow.v.dtype == torch.float32
    assert ordinary.k.dtype == (torch.float32 if dtype == "float32" else torch.bfloat16) and ordinary.k.shape[-1] == 32
    assert not runner.parts.graph_safe
    worst = 0.0
    for trace in (traces.mixed(requests, seed=9), traces.portions(requests)):
        session = TraceSession(runner)
        for record, rows in zip(trace.steps, trace.expected):
            logits = session.run_step(record)
            got = logits.cpu().numpy() if rows else None
            for i, (rid, pos) in enumerate(rows):
                err = np.abs(got[i] - want[rid][pos]).max() / (tol * (1 + np.abs(want[rid][pos]).max()))
                worst = max(worst, err)
                assert err <= 1.0, f"{rid} position {pos}: {err:.2f} of the bound"
        assert runner.cache.free_pages() == [pool, pool] and not session.live
    print(f"narrow values {dtype}: worst {worst:.2f} of the bound")
