"""Generality of the parts: a toy architecture defined here, registered, built, loaded and stepped
without a change to the framework's files.

It has a mixer with state of its own (one vector per request, kept in a state slot), a feed-forward
with routing, another position encoding, a windowed attention layer beside an all-keys one (two cache
groups), a layer that runs twice, and an execution that reads another execution's cache.  It is no
model of anyone's.  A plain whole-sequence implementation, also here, is what it is compared with.
"""
import json
import random
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_qwen3 as plain
from test_model_gpu import cut_chunks, cut_mixed, cut_tail, cut_whole, replay

pytestmark = pytest.mark.gpu

F32 = torch.float32
WINDOW = 12


# --------------------------------------------------------------------------- the toy parts
def define_toy():
    """Registers the toy parts and the toy architecture (once); returns the configuration class."""
    from vosti_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from vosti_amd.config.registry import _ARCHITECTURES
    from vosti_amd.parts import (FeedForward, Mixer, ParamSpec, PositionEncoding, StateSlotSpec, register_part)

    if "ToyHybridForCausalLM" in _ARCHITECTURES:
        return _ARCHITECTURES["ToyHybridForCausalLM"]

    @register_part("mixer", "toy_decay")
    class ToyDecay(Mixer):
        """state_t = sigmoid(a) * state_{t-1} + x_t, per request; y_t = state_t W^T."""
        replayable = False           # forward walks the step's host numbers: a recording would repeat one step's slots

        def __init__(self, kernels, hidden_size):
            super().__init__(kernels)
            self.h = hidden_size

        def params(self):
            return {"decay": ParamSpec((self.h,), init=("uniform", -1.0, 1.0)), "out_proj.weight": ParamSpec((self.h, self.h))}

        def load(self, tensors):
            self.decay, self.w = tensors["decay"], tensors["out_proj.weight"]

        def cache_spec(self):
            return StateSlotSpec((self.h,), torch.float32)

        def forward(self, x, ctx, cache):
            a = torch.sigmoid(self.decay.float())
            y = torch.empty_like(x, dtype=torch.float32)
            row = 0
            for n, start, slot in zip(ctx.host_q_lens, ctx.host_starts, ctx.host_state_slots):
                state = torch.zeros(self.h, device=x.device) if start == 0 else cache.state[slot]
                for t in range(n):
                    state = a * state + x[row + t].float()
                    y[row + t] = state
                cache.state[slot] = state
                row += n
            return self.kernels.gemm(y.to(x.dtype), self.w)

    @register_part("feed_forward", "toy_routed")
    class ToyRouted(FeedForward):
        """Top-1 of E small SwiGLU experts, weighted by the router's softmax probability."""

        def __init__(self, kernels, hidden_size, intermediate_size, num_experts):
            super().__init__(kernels)
            self.h, self.i, self.e = hidden_size, intermediate_size, num_experts

        def params(self):
            p = {"router.weight": ParamSpec((self.e, self.h), init=("normal", 0.5))}
            for e in range(self.e):
                p[f"experts.{e}.gate_up.weight"] = ParamSpec((2 * self.i, self.h))
                p[f"experts.{e}.down.weight"] = ParamSpec((self.h, self.i))
            return p

        def load(self, tensors):
            self.t = dict(tensors)

        def forward(self, x, ctx):
            k = self.kernels
            probs = torch.softmax(x.float() @ self.t["router.weight"].float().t(), dim=-1)
            choice = torch.argmax(probs, dim=-1)
            out = torch.zeros_like(x, dtype=torch.float32)
            for e in range(self.e):
                idx = torch.nonzero(choice == e).flatten()
                if idx.numel():
                    h = k.gemm(k.swiglu(k.gemm(x[idx].contiguous(), self.t[f"experts.{e}.gate_up.weight"])), self.t[f"experts.{e}.down.weight"])
                    out[idx] = h.float() * probs[idx, e:e + 1]
            return out.to(x.dtype)

    @register_part("position", "toy_additive")
    class ToyAdditive(PositionEncoding):
        """q and k get a learned vector per absolute position added."""

        def __init__(self, kernels, head_dim, max_positions):
            super().__init__(kernels)
            self.d, self.n = head_dim, max_positions

        def params(self):
            return {"table": ParamSpec((self.n, self.d), init=("normal", 0.3))}

        def load(self, tensors):
            self.table = tensors["table"]

        def apply(self, q, k, positions):
            t = self.table[positions.long()][:, None, :]
            return (q.float() + t.float()).to(q.dtype), (k.float() + t.float()).to(k.dtype)

    @register_architecture("ToyHybridForCausalLM")
    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int = 131
        hidden_size: int = 48
        heads: int = 3
        kv_heads: int = 1
        head_dim: int = 16
        inter: int = 40
        experts: int = 3
        max_positions: int = 160
        eps: float = 1e-5
        theta: float = 100.0
        architecture: str = "ToyHybridForCausalLM"

        @classmethod
        def from_dict(cls, raw):
            return cls(**{k: raw[k] for k in cls.__dataclass_fields__ if k in raw and k != "architecture"})

        def to_dict(self):
            d = asdict(self)
            d["architectures"] = [d.pop("architecture")]
            return d

        def model_spec(self):
            H, d = self.hidden_size, self.head_dim
            norm = PartSpec("rmsnorm", {"size": H, "eps": self.eps})
            hnorm = PartSpec("rmsnorm", {"size": d, "eps": self.eps})
            rope = PartSpec("rotary", {"head_dim": d, "rotary_dim": 8, "theta": self.theta, "max_positions": self.max_positions})
            add = PartSpec("toy_additive", {"head_dim": d, "max_positions": self.max_positions})

            def attn(window, position, qk_norm):
                return PartSpec("attention", {"hidden_size": H, "num_heads": self.heads, "num_kv_heads": self.kv_heads,
                                              "head_dim": d, "scale": 0.3, "window": window, "position": position,
                                              "q_norm": hnorm if qk_norm else None, "k_norm": hnorm if qk_norm else None})
            swiglu = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": self.inter})
            routed = PartSpec("toy_routed", {"hidden_size": H, "intermediate_size": 24, "num_experts": self.experts})
            mixers = [attn(0, rope, True), PartSpec("toy_decay", {"hidden_size": H}), attn(WINDOW, add, False)]
            ffns = [swiglu, routed, swiglu]
            layers = []
            for i, (m, f) in enumerate(zip(mixers, ffns)):
                probe = {"mixer": m, "feed_forward": f}
                names = {"norms.input.weight": f"l{i}.n1", "norms.post_mixer.weight": f"l{i}.n2"}
                # Tensor names: the parameter paths themselves, under the layer's prefix.
                from vosti_amd.parts import build_part
                from vosti_amd.models.decoder import walk_params
                for cat, spec in (("mixer", m), ("feed_forward", f)):
                    for path, _, _, _ in walk_params(build_part(cat, spec, None), cat + "."):
                        names[path] = f"l{i}.{path}"
                layers.append(LayerSpec("prenorm", m, f, {"input": norm, "post_mixer": norm}, names))
            return ModelSpec(
                architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=H, max_positions=self.max_positions,
                embedding=PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": H}),
                layers=tuple(layers),
                # Layer 0 runs twice (each execution has a cache of its own); the last execution of
                # layer 2 reads the keys and values that its first execution stored.
                schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0), ScheduleEntry(2, cache_from=2)),
                final_norm=norm, head=PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": H, "tied": False}),
                names={"embedding.weight": "emb", "final_norm.weight": "norm", "head.weight": "head"})

    return ToyConfig


# ------------------------------------------------------------------- the plain toy model
class PlainToy:
    def __init__(self, model_dir):
        from safetensors.torch import load_file
        self.c = json.loads((model_dir / "config.json").read_text())
        self.w = {n: t.float() for n, t in load_file(str(model_dir / "model.safetensors")).items()}

    def attention_layer(self, i, x, positions, kv=None):
        c, w = self.c, self.w
        T, nq, nkv, d = x.shape[0], c["heads"], c["kv_heads"], c["head_dim"]
        p = f"l{i}.mixer."
        q = plain.linear(x, w[p + "q_proj.weight"], F32).view(T, nq, d)
        k = plain.linear(x, w[p + "k_proj.weight"], F32).view(T, nkv, d)
        v = plain.linear(x, w[p + "v_proj.weight"], F32).view(T, nkv, d)
        if i == 0:
            q = plain.head_rms_norm(q, w[p + "q_norm.weight"], c["eps"], F32)
            k = plain.head_rms_norm(k, w[p + "k_norm.weight"], c["eps"], F32)
            cos, sin = plain.rope_tables(c["max_positions"], 8, c["theta"], F32)
            q, k = plain.apply_rope(q, cos, sin, positions, F32), plain.apply_rope(k, cos, sin, positions, F32)
            window = 0
        else:
            t = w[p + "position.table"][positions][:, None, :]
            q, k = q + t, k + t
            window = WINDOW
        if kv is not None:
            k, v = kv
        out = plain.attention(q, k, v, 0.3, F32, window=window)
        return plain.linear(out.reshape(T, nq * d), w[p + "o_proj.weight"], F32), (k, v)

    def decay_layer(self, x):
        a = torch.sigmoid(self.w["l1.mixer.decay"])
        state, ys = torch.zeros(x.shape[1]), []
        for t in range(x.shape[0]):
            state = a * state + x[t]
            ys.append(state)
        return plain.linear(torch.stack(ys), self.w["l1.mixer.out_proj.weight"], F32)

    def ffn(self, i, x):
        w = self.w
        p = f"l{i}.feed_forward."
        if i != 1:
            gu = torch.cat([plain.linear(x, w[p + "gate_proj.weight"], F32), plain.linear(x, w[p + "up_proj.weight"], F32)], 1)
            return plain.linear(plain.swiglu(gu, F32), w[p + "down_proj.weight"], F32)
        probs = torch.softmax(x @ w[p + "router.weight"].t(), dim=-1)
        out = torch.zeros_like(x)
        for t in range(x.shape[0]):
            e = int(torch.argmax(probs[t]))
            h = plain.linear(plain.swiglu(plain.linear(x[t:t + 1], w[p + f"experts.{e}.gate_up.weight"], F32), F32),
                             w[p + f"experts.{e}.down.weight"], F32)
            out[t] = h[0] * probs[t, e]
        return out

    def logits(self, ids):
        c, w = self.c, self.w
        positions = torch.arange(len(ids))
        x = w["emb"][torch.tensor(ids)]
        saved = None
        for entry, (i, reads) in enumerate([(0, False), (1, False), (2, False), (0, False), (2, True)]):
            n = plain.rms_norm(x, w[f"l{i}.n1"], c["eps"], F32)
            if i == 1:
                m = self.decay_layer(n)
            else:
                m, kv = self.attention_layer(i, n, positions, saved if reads else None)
                if entry == 2:
                    saved = kv
            x = x + m
            x = x + self.ffn(i, plain.rms_norm(x, w[f"l{i}.n2"], c["eps"], F32))
        return plain.linear(plain.rms_norm(x, w["norm"], c["eps"], F32), w["head"], F32)


@pytest.fixture(scope="module")
def toy_dir(tmp_path_factory):
    from vosti_amd.weights import write_random_model
    cfg = define_toy()()
    return write_random_model(cfg, 3, tmp_path_factory.mktemp("toy"), dtype=torch.float32)


def toy_prompts():
    rng = random.Random(2)
    return [[rng.randrange(131) for _ in range(n)] for n in (3, 29, 64, 150, 41)]


def test_toy_architecture_is_registered_built_and_stepped(toy_dir):
    from vosti_amd.cache import CachePool
    from vosti_amd.config import load_config
    from vosti_amd.engine import ModelRunner
    from vosti_amd.models import load_model
    from vosti_amd.parts import PagedKV, StateSlots

    assert type(load_config(toy_dir)).__name__ == "ToyConfig"
    model = load_model(toy_dir, "float32")
    assert not model.layers[2].mixer._fused and model.layers[0].mixer._fused
    prompts = toy_prompts()
    ref = [PlainToy(toy_dir).logits(p) for p in prompts]
    page = 8
    mixed_steps, mixed_pages = cut_mixed(prompts, page, seed=9)

    def runner(pages):
        pool = CachePool(model, page_size=page, num_pages=pages, num_slots=6)
        assert pool.group_windows == [0, WINDOW] and not pool.manager.prefix_cache
        kinds = [type(e) for e in pool.entries]
        assert kinds == [PagedKV, StateSlots, PagedKV, PagedKV, PagedKV]
        assert pool.entries[4].k is pool.entries[2].k and not pool.entries[4].writable and pool.entries[3].k is not pool.entries[0].k
        return ModelRunner(model, pool)

    whole = replay(runner(-(-150 // page)), cut_whole(prompts))
    for i, p in enumerate(prompts):
        got = torch.stack([whole[(i, j)] for j in range(len(p))])
        torch.testing.assert_close(got, ref[i], rtol=1e-4, atol=2e-5, msg=lambda m: f"request {i}: {m}")
    for label, steps, pages in (("tail", cut_tail(prompts), 19), ("chunks", cut_chunks(prompts), 19), ("mixed", mixed_steps, mixed_pages)):
        got = replay(runner(pages), steps)
        worst = max((got[k] - whole[k]).abs().max().item() for k in whole)
        # The toy parts use library routines whose summation order may depend on the batch: not bitwise, but tight.
        assert worst < 2e-5, (label, worst)


def test_window_pages_go_back_while_a_request_lives(toy_dir):
    """The windowed group needs pages for the window and the portion only, however long the request is."""
    from vosti_amd.cache import CachePool
    from vosti_amd.engine import ModelRunner, StepEntry
    from vosti_amd.models import load_model
    model = load_model(toy_dir, "float32")
    p = toy_prompts()[3]
    ref = PlainToy(toy_dir).logits(p)
    pool = CachePool(model, page_size=8, num_pages=19, num_slots=2, window_pages=4)    # 4 pages: window 12 + portion 8, page-rounded
    r = ModelRunner(model, pool)
    rows = []
    for start in range(0, len(p), 8):
        chunk = p[start:start + 8]
        rows.append(r.kernels.to_f32(r.step([StepEntry(0, chunk, list(range(len(chunk))))])).cpu())
        assert pool.manager.free_pages(1) >= 1 and pool.manager.check() == ""
    torch.testing.assert_close(torch.cat(rows), ref, rtol=1e-4, atol=2e-5)
    r.finish(0)
    assert pool.manager.free_pages(0) == 19 and pool.manager.free_pages(1) == 4


def test_toy_generation_through_the_engine(toy_dir):
    from vosti_amd.engine import Engine
    from vosti_amd.sampling import SamplingParams
    prompts = toy_prompts()[:3]
    plain_model = PlainToy(toy_dir)
    # Asked to record its decode steps, the engine does not: one of the toy's parts says that it cannot be replayed.
    engine = Engine(toy_dir, dtype="float32", num_pages=40, page_size=8, max_num_seqs=3, max_num_batched_tokens=32, graphs=True)
    outs = engine.generate(prompts, SamplingParams(max_tokens=10))
    assert engine.runner.graph_stats["captured"] == 0 and engine.runner.graph_stats["replayed"] == 0
    for p, o in zip(prompts, outs):
        ids = list(p)
        for tok in o:
            row = plain_model.logits(ids)[-1]
            assert row[tok] >= row.max() - 1e-5
            ids.append(tok)
