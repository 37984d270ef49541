"""A toy mixer with state of its own, defined here, is registered, built into a
model beside the framework's attention, loaded, and stepped, without a change to
the framework's files.  Its per-request state lives in the cache manager's state
slots; portions and single tokens must give the same result."""
from dataclasses import dataclass

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def build_toy():
    from runtime import register_part, make_part, register_architecture, StateNeed, TensorSpec
    from runtime.config import unregister_architecture
    from runtime.parts import Mixer, TokenEmbedding, LMHead, unregister_part
    from runtime.models import Model, ScheduleEntry

    class DecayMixer(Mixer):
        """s_t = decay * s_{t-1} + h_t;  out = s_t W^T, added to the residual."""

        def __init__(self, name, hidden, decay):
            self.name, self.hidden, self.decay = name, hidden, decay

        def state_need(self):
            return StateNeed((self.hidden,), "float32")

        def tensor_specs(self):
            return [TensorSpec(self.name + ".mix.weight", (self.hidden, self.hidden))]

        def bind(self, tensors, dtype):
            self.weight = tensors[self.name + ".mix.weight"].float()

        def forward(self, h, residual, ctx, site):
            state = ctx.cache.state_storage[site]
            slots = ctx.state_slots.cpu().tolist()
            row = 0
            for (request, start, count), slot in zip(ctx.segments, slots):
                s = state[slot]
                for t in range(count):          # a scan over the portion
                    s = self.decay * s + h[row + t].float()
                    residual[row + t] += s @ self.weight.T
                state[slot] = s
                row += count
            return residual

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        hidden_size: int
        decay: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["vocab_size"], raw["hidden_size"], raw["decay"], raw["max_position_embeddings"], raw["rms_norm_eps"])

    def build(c):
        emb = TokenEmbedding("embed", c.vocab_size, c.hidden_size)
        def norm(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        rope = make_part("position", "rotary", head_dim=16, theta=1e4, max_positions=c.max_position_embeddings)
        attention = make_part("mixer", "attention", name="l0.attn", hidden=c.hidden_size, heads=2, kv_heads=1, head_dim=16, position=rope)
        layers = [
            make_part("block", "prenorm", mixer_norm=norm("l0.n1"), mixer=attention, ffn_norm=norm("l0.n2"),
                      ffn=make_part("ffn", "gated_mlp", name="l0.mlp", hidden=c.hidden_size, intermediate=40)),
            make_part("block", "prenorm", mixer_norm=norm("l1.n1"), mixer=make_part("mixer", "toy-decay", name="l1", hidden=c.hidden_size, decay=c.decay),
                      ffn_norm=norm("l1.n2"), ffn=make_part("ffn", "gated_mlp", name="l1.mlp", hidden=c.hidden_size, intermediate=24)),
        ]
        # layer 1 runs twice: shared weights, a state of its own at each place in the order
        return Model(c, emb, layers, norm("final"), LMHead("head", c.vocab_size, c.hidden_size),
                     schedule=[ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1)])

    register_part("mixer", "toy-decay", DecayMixer)
    register_architecture("toy-decay-lm", ToyConfig, build)

    def cleanup():
        unregister_part("mixer", "toy-decay")
        unregister_architecture("toy-decay-lm")
    return cleanup


def plain_toy(raw, w, tokens):
    import plain_llama as P
    H, decay, eps = raw["hidden_size"], raw["decay"], raw["rms_norm_eps"]
    x = w["embed.weight"][tokens]
    T = len(tokens)

    def decay_layer(x):
        h = P.rmsnorm(x, w["l1.n1.weight"], eps)
        s, out = np.zeros(H), []
        for t in range(T):
            s = decay * s + h[t]
            out.append(s @ w["l1.mix.weight"].T)
        x = x + np.stack(out)
        h = P.rmsnorm(x, w["l1.n2.weight"], eps)
        return x + P.linear(P.swiglu(P.linear(h, w["l1.mlp.gate_proj.weight"]), P.linear(h, w["l1.mlp.up_proj.weight"])), w["l1.mlp.down_proj.weight"])

    def attention_layer(x):
        h = P.rmsnorm(x, w["l0.n1.weight"], eps)
        q = P.rope(P.linear(h, w["l0.attn.q_proj.weight"]).reshape(T, 2, 16), np.arange(T), 1e4)
        k = P.rope(P.linear(h, w["l0.attn.k_proj.weight"]).reshape(T, 1, 16), np.arange(T), 1e4)
        v = P.linear(h, w["l0.attn.v_proj.weight"]).reshape(T, 1, 16)
        x = x + P.linear(P.causal_attention(q, k, v).reshape(T, 32), w["l0.attn.o_proj.weight"])
        h = P.rmsnorm(x, w["l0.n2.weight"], eps)
        return x + P.linear(P.swiglu(P.linear(h, w["l0.mlp.gate_proj.weight"]), P.linear(h, w["l0.mlp.up_proj.weight"])), w["l0.mlp.down_proj.weight"])

    x = decay_layer(x); x = attention_layer(x); x = decay_layer(x)
    return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    import json
    import plain_llama as P
    from runtime.engine import load_model, write_random_model, ModelRunner, StepEntry
    cleanup = build_toy()
    try:
        raw = {"model_type": "toy-decay-lm", "vocab_size": 61, "hidden_size": 24, "decay": 0.7,
               "max_position_embeddings": 96, "rms_norm_eps": 1e-5}
        # the random-weights mode serves a registered architecture it has never seen
        tmp_path.mkdir(exist_ok=True)
        from runtime.engine.loading import build_from_config_dict
        from runtime.weights import write_model_folder
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=3, dtype=torch.float32)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype="float32")
        assert set(model.state_needs()) == {0, 2} and set(model.cache_needs()) == {1}
        runner = ModelRunner(model, n_pages=12, page_size=8, max_requests=3)
        tokens = {"x": np.random.default_rng(0).integers(0, 61, 30).tolist(), "y": np.random.default_rng(1).integers(0, 61, 17).tolist()}
        want = {k: plain_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got = {"x": [], "y": []}
        plan = [[("x", 9), ("y", 2)], [("x", 1), ("y", 7)], [("y", 1)], [("x", 13), ("y", 1)], [("x", 7), ("y", 6)]]
        fed = {"x": 0, "y": 0}
        for step in plan:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            np.testing.assert_allclose(np.concatenate(got[k]), want[k], rtol=2e-4, atol=2e-5)
        # a released slot is zeroed for its next owner
        runner.release("x"); runner.create("z")
        out = runner.step([StepEntry("z", tokens["y"], list(range(17)))]).cpu().numpy()
        np.testing.assert_allclose(out, want["y"], rtol=2e-4, atol=2e-5)
        runner.cache.check()
    finally:
        cleanup()
