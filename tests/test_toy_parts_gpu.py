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
SEEN = []      # (launch value a step array was filled with, the batch's own), by RowsOfSegments.fill


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
    class RowsOfSegments:
        """A step array of this file's own (the framework has no such list): for every row of the step the first row
        of its segment (-1 for a padding row), then for every row its segment (0 for a padding row).  Its launch
        value, the longest portion of the step, is recorded in SEEN with the true one."""

        def words(self, rows, segments):
            return 2 * rows

        def launch_value(self, batch):
            return max(batch.counts)

        def fill(self, out, batch, value):
            rows = len(out) // 2
            out[:rows], out[rows:] = -1, 0
            for segment, (row, count) in enumerate(zip(batch.first_row, batch.counts)):
                out[row:row + count], out[rows + row:rows + row + count] = row, segment
            SEEN.append((value, max(batch.counts)))

    class PrefixSumMixer(Mixer):
        """s_t = s_{t-1} + h_t; out = s_t W^T: DecayMixer with a decay of 1, but as launches only (no host reads, so it
        runs under graph capture too), which takes a list that no step carries by itself: RowsOfSegments."""

        def __init__(self, name, hidden, decay, declared):
            assert decay == 1.0
            self.name, self.hidden, self.declared = name, hidden, declared

        def state_need(self):
            return StateNeed((self.hidden,), "float32")

        def step_arrays(self):
            return [RowsOfSegments()] if self.declared else []     # else: asked for at the first step

        def tensor_specs(self):
            return [TensorSpec(self.name + ".mix.weight", (self.hidden, self.hidden))]

        def bind(self, tensors, dtype):
            self.weight = tensors[self.name + ".mix.weight"].float()

        def forward(self, h, residual, ctx, site):
            links, _ = ctx.step_array(RowsOfSegments())
            T = ctx.n_rows
            first, segment = links[:T], links[T:2 * T].long()
            valid = first >= 0
            r = torch.arange(T, device=h.device)
            earlier_of_the_same = (first[:, None] == first[None, :]) & (r[None, :] <= r[:, None]) & valid[None, :]
            state = ctx.cache.state_storage[site]
            slot = ctx.state_slots.long().index_select(0, segment)
            x = h.float() * valid[:, None]
            s = earlier_of_the_same.float() @ x + state.index_select(0, slot)
            residual += (s @ self.weight.T) * valid[:, None]
            state.index_add_(0, slot, x)
            return residual

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        hidden_size: int
        decay: float
        max_position_embeddings: int
        rms_norm_eps: float
        mixer: str = "toy-decay"
        declared: bool = False

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["vocab_size"], raw["hidden_size"], raw["decay"], raw["max_position_embeddings"], raw["rms_norm_eps"],
                       raw.get("mixer", "toy-decay"), raw.get("declared", False))

    def build(c):
        emb = TokenEmbedding("embed", c.vocab_size, c.hidden_size)
        def norm(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        rope = make_part("position", "rotary", head_dim=16, theta=1e4, max_positions=c.max_position_embeddings)
        attention = make_part("mixer", "attention", name="l0.attn", hidden=c.hidden_size, heads=2, kv_heads=1, head_dim=16, position=rope)
        layers = [
            make_part("block", "prenorm", mixer_norm=norm("l0.n1"), mixer=attention, ffn_norm=norm("l0.n2"),
                      ffn=make_part("ffn", "gated_mlp", name="l0.mlp", hidden=c.hidden_size, intermediate=40)),
            make_part("block", "prenorm", mixer_norm=norm("l1.n1"),
                      mixer=make_part("mixer", c.mixer, name="l1", hidden=c.hidden_size, decay=c.decay,
                                      **({"declared": c.declared} if c.mixer == "toy-prefix-sum" else {})),
                      ffn_norm=norm("l1.n2"), ffn=make_part("ffn", "gated_mlp", name="l1.mlp", hidden=c.hidden_size, intermediate=24)),
        ]
        # layer 1 runs twice: shared weights, a state of its own at each place in the order
        return Model(c, emb, layers, norm("final"), LMHead("head", c.vocab_size, c.hidden_size),
                     schedule=[ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1)])

    register_part("mixer", "toy-decay", DecayMixer)
    register_part("mixer", "toy-prefix-sum", PrefixSumMixer)
    register_architecture("toy-decay-lm", ToyConfig, build)

    def cleanup():
        unregister_part("mixer", "toy-decay")
        unregister_part("mixer", "toy-prefix-sum")
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

    import plain_llama as P
    from runtime.engine import load_model, ModelRunner, StepEntry
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


@pytest.mark.parametrize("execution, declared", [("eager", True), ("eager", False), ("graph", True), ("graph", False)])
def test_a_mixer_brings_a_step_array_of_its_own(tmp_path, execution, declared):
    """A mixer defined here needs a list per step that the step function knows nothing of.  It declares it (or asks
    for it at its first step), the step function carries it with its metadata, filled by the array's own code, and
    under captured programs its launch value is part of a program's key, rounded up."""
    import plain_llama as P
    from runtime.engine import load_model, ModelRunner, StepEntry
    cleanup = build_toy()
    try:
        raw = {"model_type": "toy-decay-lm", "vocab_size": 61, "hidden_size": 24, "decay": 1.0, "mixer": "toy-prefix-sum",
               "declared": declared, "max_position_embeddings": 96, "rms_norm_eps": 1e-5}
        from runtime.engine.loading import build_from_config_dict
        from runtime.weights import write_model_folder
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=5, dtype=torch.float32)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype="float32")
        assert any(type(a).__name__ == "RowsOfSegments" for a in model.step_arrays()) == declared
        runner = ModelRunner(model, n_pages=16, page_size=8, max_requests=3, execution=execution)
        tokens = {"x": np.random.default_rng(0).integers(0, 61, 38).tolist(), "y": np.random.default_rng(1).integers(0, 61, 25).tolist()}
        want = {k: plain_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        plan = [[("x", 9), ("y", 2)], [("x", 1), ("y", 7)], [("y", 1)], [("x", 13), ("y", 1)], [("x", 7), ("y", 6)]] + [[("x", 1), ("y", 1)]] * 8
        del SEEN[:]
        for step in plan:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            np.testing.assert_allclose(np.concatenate(got[k]), want[k], rtol=2e-4, atol=2e-5)
        told = runner.report()
        assert sum("RowsOfSegments" in a for a in told["step_arrays"]) == 1
        assert len(SEEN) == len(plan)                                       # filled once a step, whoever asked
        if execution == "eager":
            assert all(value == true for value, true in SEEN)
        else:
            assert all(true <= value < 2 * true for value, true in SEEN) and told["replays"] >= 6
        runner.cache.check()
    finally:
        cleanup()


def test_a_step_that_fails_after_a_state_was_written_cannot_be_tried_again(tmp_path):
    """The toy model updates a per-request state in its first layer; here the last layer of the order raises in the
    middle of a step.  Lengths and pages go back (the cache manager's part of the promise), but the first layer's
    state already holds the step's tokens and nothing keeps the old one: the requests of that step are refused from
    then on instead of being stepped twice over the same tokens, other requests go on, and a released and recreated
    request starts from a zeroed state and gives the right logits."""
    import plain_llama as P
    from runtime.engine import load_model, ModelRunner, StepEntry
    cleanup = build_toy()
    try:
        raw = {"model_type": "toy-decay-lm", "vocab_size": 61, "hidden_size": 24, "decay": 0.7,
               "max_position_embeddings": 96, "rms_norm_eps": 1e-5}
        from runtime.engine.loading import build_from_config_dict
        from runtime.weights import write_model_folder
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=3, dtype=torch.float32)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype="float32")
        runner = ModelRunner(model, n_pages=12, page_size=8, max_requests=3)
        tokens = np.random.default_rng(0).integers(0, 61, 20).tolist()
        want = plain_toy(raw, w, tokens)
        runner.create("x"); runner.create("bystander")
        runner.step([StepEntry("x", tokens[:6], []), StepEntry("bystander", tokens[:3], [])])
        mixer, calls = model.layers[1].mixer, []
        real = mixer.forward

        def fails_at_its_second_place(h, residual, ctx, site, **kw):
            calls.append(site)
            if len(calls) == 2:
                raise RuntimeError("injected")
            return real(h, residual, ctx, site, **kw)

        mixer.forward = fails_at_its_second_place
        free = runner.cache.free_pages()
        with pytest.raises(RuntimeError, match="injected"):
            runner.step([StepEntry("x", tokens[6:15], [8])])
        mixer.forward = real
        assert runner.length("x") == 6 and runner.cache.free_pages() == free      # lengths and pages stand where they stood
        runner.cache.check()
        with pytest.raises(RuntimeError, match="cannot be stepped again"):
            runner.step([StepEntry("x", tokens[6:15], [8])])
        with pytest.raises(ValueError, match="last step"):
            runner.pick(None, torch.zeros(1, 61, device=DEV), [(0.0, 0, 0)])        # no logits of a step that never ran
        out = runner.step([StepEntry("bystander", tokens[3:], list(range(17)))]).cpu().numpy()   # others go on
        np.testing.assert_allclose(out, want[3:], rtol=2e-4, atol=2e-5)
        runner.release("x"); runner.create("x")
        out = runner.step([StepEntry("x", tokens, list(range(20)))]).cpu().numpy()
        np.testing.assert_allclose(out, want, rtol=2e-4, atol=2e-5)
        runner.cache.check()
    finally:
        cleanup()


def build_routed_toy():
    """A feed-forward with routing (two experts, the best one scaled by its softmax weight) and a position
    encoding of its own (rotary angles that grow linearly with the pair index), both defined here."""
    from runtime import register_part, make_part, register_architecture, TensorSpec
    from runtime.config import unregister_architecture
    from runtime.parts import FeedForward, Part, TokenEmbedding, LMHead, unregister_part
    from runtime.models import Model

    class LinearRotary(Part):
        """Pair (i, i + D/2) of a head turns by pos * step * (i + 1)."""

        def __init__(self, head_dim, step, max_positions):
            self.head_dim, self.step, self.max_positions, self._tables = head_dim, step, max_positions, None

        def prepare(self, device, dtype):
            a = np.arange(self.max_positions, dtype=np.float64)[:, None] * self.step * np.arange(1, self.head_dim // 2 + 1)[None, :]
            self._tables = (torch.from_numpy(np.cos(a).astype(np.float32)).to(device), torch.from_numpy(np.sin(a).astype(np.float32)).to(device))

        def tables(self):
            return self._tables

    class RoutedMLP(FeedForward):
        """out = p_e * expert_e(h) for the expert e with the largest router logit; p = softmax of the logits (float)."""

        def __init__(self, name, hidden, intermediate, experts):
            self.name, self.hidden, self.intermediate, self.experts = name, hidden, intermediate, experts

        def tensor_specs(self):
            specs = [TensorSpec(f"{self.name}.router.weight", (self.experts, self.hidden))]
            for e in range(self.experts):
                specs += [TensorSpec(f"{self.name}.experts.{e}.gate_proj.weight", (self.intermediate, self.hidden)),
                          TensorSpec(f"{self.name}.experts.{e}.up_proj.weight", (self.intermediate, self.hidden)),
                          TensorSpec(f"{self.name}.experts.{e}.down_proj.weight", (self.hidden, self.intermediate))]
            return specs

        def bind(self, tensors, dtype):
            self.w = {k[len(self.name) + 1:]: v.float() for k, v in tensors.items() if k.startswith(self.name + ".")}

        def forward(self, h, residual, ctx, norm=None):
            x = h.float()
            p = torch.softmax(x @ self.w["router.weight"].T, dim=-1)
            best = p.argmax(-1)
            for e in range(self.experts):
                act = torch.nn.functional.silu(x @ self.w[f"experts.{e}.gate_proj.weight"].T) * (x @ self.w[f"experts.{e}.up_proj.weight"].T)
                out = (act @ self.w[f"experts.{e}.down_proj.weight"].T) * p[:, e:e + 1]
                residual += torch.where((best == e)[:, None], out, torch.zeros_like(out))
            return residual

    @dataclass(frozen=True)
    class RoutedConfig:
        vocab_size: int
        hidden_size: int
        experts: int
        angle_step: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "experts", "angle_step", "max_position_embeddings", "rms_norm_eps")))

    def build(c):
        def norm(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        turning = make_part("position", "toy-linear-rotary", head_dim=16, step=c.angle_step, max_positions=c.max_position_embeddings)
        still = make_part("position", "none", head_dim=16, max_positions=c.max_position_embeddings)
        def attention(n, position):
            return make_part("mixer", "attention", name=n, hidden=c.hidden_size, heads=3, kv_heads=1, head_dim=16, position=position)
        layers = [
            make_part("block", "prenorm", mixer_norm=norm("l0.n1"), mixer=attention("l0.attn", turning), ffn_norm=norm("l0.n2"),
                      ffn=make_part("ffn", "toy-routed", name="l0.moe", hidden=c.hidden_size, intermediate=20, experts=c.experts)),
            make_part("block", "prenorm", mixer_norm=norm("l1.n1"), mixer=attention("l1.attn", still), ffn_norm=norm("l1.n2"),
                      ffn=make_part("ffn", "gated_mlp", name="l1.mlp", hidden=c.hidden_size, intermediate=24)),
        ]
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), layers, norm("final"),
                     LMHead("head", c.vocab_size, c.hidden_size))

    register_part("position", "toy-linear-rotary", LinearRotary)
    register_part("ffn", "toy-routed", RoutedMLP)
    register_architecture("toy-routed-lm", RoutedConfig, build)

    def cleanup():
        unregister_part("position", "toy-linear-rotary")
        unregister_part("ffn", "toy-routed")
        unregister_architecture("toy-routed-lm")
    return cleanup


def plain_routed_toy(raw, w, tokens, chosen=None):
    import plain_llama as P
    eps, step, E = raw["rms_norm_eps"], raw["angle_step"], raw["experts"]
    T = len(tokens)
    x = w["embed.weight"][tokens]

    def turn(v):   # [T, heads, 16]: pair (i, i + 8) by pos * step * (i + 1)
        a = np.arange(T)[:, None, None] * step * np.arange(1, 9)[None, None, :]
        lo, hi = v[..., :8], v[..., 8:]
        return np.concatenate([lo * np.cos(a) - hi * np.sin(a), hi * np.cos(a) + lo * np.sin(a)], axis=-1)

    def attention(x, p, rotate):
        h = P.rmsnorm(x, w[p + ".n1.weight"], eps)
        q = P.linear(h, w[p + ".attn.q_proj.weight"]).reshape(T, 3, 16)
        k = P.linear(h, w[p + ".attn.k_proj.weight"]).reshape(T, 1, 16)
        v = P.linear(h, w[p + ".attn.v_proj.weight"]).reshape(T, 1, 16)
        if rotate:
            q, k = turn(q), turn(k)
        return x + P.linear(P.causal_attention(q, k, v).reshape(T, 48), w[p + ".attn.o_proj.weight"])

    x = attention(x, "l0", True)
    h = P.rmsnorm(x, w["l0.n2.weight"], eps)
    logits = P.linear(h, w["l0.moe.router.weight"])
    prob = np.exp(logits - logits.max(-1, keepdims=True)); prob /= prob.sum(-1, keepdims=True)
    best = logits.argmax(-1)
    if chosen is not None:
        chosen.extend(best.tolist())
    out = np.zeros_like(x)
    for e in range(E):
        pre = f"l0.moe.experts.{e}."
        y = P.linear(P.swiglu(P.linear(h, w[pre + "gate_proj.weight"]), P.linear(h, w[pre + "up_proj.weight"])), w[pre + "down_proj.weight"])
        out += np.where((best == e)[:, None], y * prob[:, e:e + 1], 0.0)
    x = x + out
    x = attention(x, "l1", False)
    h = P.rmsnorm(x, w["l1.n2.weight"], eps)
    x = x + P.linear(P.swiglu(P.linear(h, w["l1.mlp.gate_proj.weight"]), P.linear(h, w["l1.mlp.up_proj.weight"])), w["l1.mlp.down_proj.weight"])
    return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])


def test_toy_routed_feed_forward_and_position_encoding_are_registered_built_and_stepped(tmp_path):
    """A feed-forward with routing and a position encoding of another law, defined in this file, in one model beside the
    framework's attention, norm and dense feed-forward (one layer without any position encoding): registered,
    given random weights, loaded and stepped in portions, without a change to the framework's files."""
    import plain_llama as P
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import write_model_folder
    cleanup = build_routed_toy()
    try:
        raw = {"model_type": "toy-routed-lm", "vocab_size": 53, "hidden_size": 24, "experts": 2, "angle_step": 0.37,
               "max_position_embeddings": 64, "rms_norm_eps": 1e-5}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=5, dtype=torch.float32)
        cfg, w = P.read_folder(tmp_path)
        w["l0.moe.router.weight"] = w["l0.moe.router.weight"] * 40      # decided routing: both experts are used
        from safetensors.torch import save_file
        save_file({k: torch.from_numpy(np.asarray(v, np.float32)) for k, v in w.items()}, str(tmp_path / "model.safetensors"))
        model = load_model(tmp_path, dtype="float32")
        assert set(model.cache_needs()) == {0, 1} and not model.state_needs()
        runner = ModelRunner(model, n_pages=12, page_size=8, max_requests=2)
        tokens = {"x": np.random.default_rng(2).integers(0, 53, 29).tolist(), "y": np.random.default_rng(3).integers(0, 53, 16).tolist()}
        chosen = []
        want = {k: plain_routed_toy(raw, w, v, chosen) for k, v in tokens.items()}
        assert min(chosen.count(0), chosen.count(1)) >= 5                # both experts do work
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        for step in [[("x", 11), ("y", 2)], [("x", 1), ("y", 5)], [("x", 1), ("y", 1)], [("x", 16), ("y", 8)]]:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            np.testing.assert_allclose(np.concatenate(got[k]), want[k], rtol=3e-4, atol=3e-5)
        # the position encoding matters: the same tokens without the turn give other logits
        raw_still = dict(raw, angle_step=0.0)
        assert np.abs(plain_routed_toy(raw_still, w, tokens["x"]) - want["x"]).max() > 1e-3
        runner.cache.check()
    finally:
        cleanup()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_with_interleaved_pairs(tmp_path, dtype):
    """A position encoding, defined here, whose pairs are neighbouring coordinates (2i, 2i + 1): it states its
    pairing, the framework's attention turns queries and keys by that rule (the kernels that fuse the rotation
    into the projection know the split-half rule only and step aside), and prompts cut into portions beside
    decoded tokens match a plain implementation that multiplies complex numbers."""
    import plain_llama as P
    from conftest import assert_close
    from runtime import register_part, make_part, register_architecture
    from runtime.config import unregister_architecture
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.models import Model
    from runtime.parts import Part, TokenEmbedding, LMHead, unregister_part
    from runtime.weights import write_model_folder

    class NeighbourPairs(Part):
        pairing = "interleaved"

        def __init__(self, head_dim, theta, max_positions):
            self.head_dim, self.theta, self.max_positions, self._tables = head_dim, theta, max_positions, None

        def prepare(self, device, dtype):
            half = self.head_dim // 2
            a = np.arange(self.max_positions, dtype=np.float64)[:, None] * self.theta ** (-np.arange(half) * 2.0 / self.head_dim)[None, :]
            self._tables = (torch.from_numpy(np.cos(a).astype(np.float32)).to(device), torch.from_numpy(np.sin(a).astype(np.float32)).to(device))

        def tables(self):
            return self._tables

    @dataclass(frozen=True)
    class PairsConfig:
        vocab_size: int
        hidden_size: int
        theta: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "theta", "max_position_embeddings", "rms_norm_eps")))

    HEADS, KV, D = 4, 2, 16

    def build(c):
        def norm(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        position = make_part("position", "toy-neighbour-pairs", head_dim=D, theta=c.theta, max_positions=c.max_position_embeddings)
        layers = [make_part("block", "prenorm", mixer_norm=norm(f"l{i}.n1"),
                            mixer=make_part("mixer", "attention", name=f"l{i}.attn", hidden=c.hidden_size, heads=HEADS, kv_heads=KV,
                                            head_dim=D, position=position),
                            ffn_norm=norm(f"l{i}.n2"),
                            ffn=make_part("ffn", "gated_mlp", name=f"l{i}.mlp", hidden=c.hidden_size, intermediate=40))
                  for i in range(2)]
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), layers, norm("final"),
                     LMHead("head", c.vocab_size, c.hidden_size))

    def plain(raw, w, tokens):
        T, eps = len(tokens), raw["rms_norm_eps"]
        angle = np.arange(T)[:, None] * raw["theta"] ** (-np.arange(D // 2) * 2.0 / D)[None, :]

        def turn(v):      # [T, heads, D]: (v[2i] + j v[2i+1]) * exp(j angle_i)
            z = (v[..., 0::2] + 1j * v[..., 1::2]) * np.exp(1j * angle)[:, None, :]
            out = np.empty_like(v)
            out[..., 0::2], out[..., 1::2] = z.real, z.imag
            return out

        x = w["embed.weight"][tokens]
        for i in range(2):
            h = P.rmsnorm(x, w[f"l{i}.n1.weight"], eps)
            q = turn(P.linear(h, w[f"l{i}.attn.q_proj.weight"]).reshape(T, HEADS, D))
            k = turn(P.linear(h, w[f"l{i}.attn.k_proj.weight"]).reshape(T, KV, D))
            v = P.linear(h, w[f"l{i}.attn.v_proj.weight"]).reshape(T, KV, D)
            x = x + P.linear(P.causal_attention(q, k, v).reshape(T, HEADS * D), w[f"l{i}.attn.o_proj.weight"])
            h = P.rmsnorm(x, w[f"l{i}.n2.weight"], eps)
            x = x + P.linear(P.swiglu(P.linear(h, w[f"l{i}.mlp.gate_proj.weight"]), P.linear(h, w[f"l{i}.mlp.up_proj.weight"])),
                             w[f"l{i}.mlp.down_proj.weight"])
        return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])

    register_part("position", "toy-neighbour-pairs", NeighbourPairs)
    register_architecture("toy-pairs-lm", PairsConfig, build)
    try:
        raw = {"model_type": "toy-pairs-lm", "vocab_size": 67, "hidden_size": 48, "theta": 50.0, "max_position_embeddings": 96,
               "rms_norm_eps": 1e-5}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=8, dtype=torch.bfloat16, std=0.15)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype=dtype)
        runner = ModelRunner(model, n_pages=16, page_size=8, max_requests=2)
        tokens = {"x": np.random.default_rng(4).integers(0, 67, 40).tolist(), "y": np.random.default_rng(5).integers(0, 67, 21).tolist()}
        want = {k: plain(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        for step in [[("x", 13), ("y", 2)], [("x", 1), ("y", 9)], [("x", 1), ("y", 1)], [("x", 25), ("y", 9)]]:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            assert_close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
        # the pairing matters: the split-half rule on the same weights gives other logits
        q = np.random.default_rng(0).standard_normal((3, 1, D))
        assert np.abs(P.rope(q, [1, 2, 3], 50.0) - q).max() > 0.1
        half_turned = P.rope(q, [1, 2, 3], 50.0)
        z = (q[..., 0::2] + 1j * q[..., 1::2]) * np.exp(1j * (np.asarray([1, 2, 3])[:, None] * 50.0 ** (-np.arange(D // 2) * 2.0 / D)))[:, None, :]
        assert np.abs(half_turned[..., 0::2] - z.real).max() > 0.1
        runner.cache.check()
    finally:
        unregister_part("position", "toy-neighbour-pairs")
        unregister_architecture("toy-pairs-lm")


def build_shared_cache_toy():
    """A norm of another law (centred, with a bias: nothing the product kernels can take over) and a layer whose
    attention keeps no keys of its own and reads the cache of the layer before, both in one model beside the
    framework's norm, attention and feed-forward."""
    from runtime import register_part, make_part, register_architecture, TensorSpec
    from runtime.config import unregister_architecture
    from runtime.parts import Part, TokenEmbedding, LMHead, unregister_part
    from runtime.models import Model, ScheduleEntry

    class CentredNorm(Part):
        """y = (x - mean) / sqrt(var + eps) * weight + bias over the row, in float."""

        def __init__(self, name, dim, eps):
            self.name, self.dim, self.eps = name, dim, eps

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.dim,), init="one_plus_normal"), TensorSpec(self.name + ".bias", (self.dim,))]

        def bind(self, tensors, dtype):
            self.weight, self.bias = tensors[self.name + ".weight"].float(), tensors[self.name + ".bias"].float()

        def forward(self, x, ctx, rows=None, tag="norm"):
            if rows is not None:
                x = x[rows.long()]
            centred = x - x.mean(-1, keepdim=True)
            y = centred * torch.rsqrt(centred.square().mean(-1, keepdim=True) + self.eps) * self.weight + self.bias
            out = ctx.buffer(tag, tuple(y.shape), ctx.dtype)
            out.copy_(y)
            return out

    @dataclass(frozen=True)
    class SharedConfig:
        vocab_size: int
        hidden_size: int
        heads: int
        kv_heads: int
        head_dim: int
        intermediate_size: int
        rope_theta: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "heads", "kv_heads", "head_dim", "intermediate_size",
                                          "rope_theta", "max_position_embeddings", "rms_norm_eps")))

    def build(c):
        def rms(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        def centred(n): return make_part("norm", "toy-centred", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        position = make_part("position", "rotary", head_dim=c.head_dim, theta=c.rope_theta, max_positions=c.max_position_embeddings)
        def attention(n, own_kv):
            return make_part("mixer", "attention", name=n, hidden=c.hidden_size, heads=c.heads, kv_heads=c.kv_heads,
                             head_dim=c.head_dim, position=position, own_kv=own_kv)
        def mlp(n): return make_part("ffn", "gated_mlp", name=n, hidden=c.hidden_size, intermediate=c.intermediate_size)
        layers = [
            make_part("block", "prenorm", mixer_norm=rms("l0.n1"), mixer=attention("l0.attn", True), ffn_norm=rms("l0.n2"), ffn=mlp("l0.mlp")),
            make_part("block", "prenorm", mixer_norm=centred("l1.n1"), mixer=attention("l1.attn", False), ffn_norm=centred("l1.n2"), ffn=mlp("l1.mlp")),
            make_part("block", "prenorm", mixer_norm=rms("l2.n1"), mixer=attention("l2.attn", True), ffn_norm=centred("l2.n2"), ffn=mlp("l2.mlp")),
        ]
        # the second layer reads the keys and values that the first one wrote
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), layers, centred("final"),
                     LMHead("head", c.vocab_size, c.hidden_size),
                     schedule=[ScheduleEntry(0), ScheduleEntry(1, reads=0), ScheduleEntry(2)])

    register_part("norm", "toy-centred", CentredNorm)
    register_architecture("toy-shared-cache-lm", SharedConfig, build)

    def cleanup():
        unregister_part("norm", "toy-centred")
        unregister_architecture("toy-shared-cache-lm")
    return cleanup


def plain_shared_cache_toy(raw, w, tokens):
    import plain_llama as P
    eps, theta = raw["rms_norm_eps"], raw["rope_theta"]
    nh, nkv, D = raw["heads"], raw["kv_heads"], raw["head_dim"]
    T = len(tokens)
    pos = np.arange(T)

    def centred(x, p):
        x = np.asarray(x, np.float64)
        c = x - x.mean(-1, keepdims=True)
        return c / np.sqrt((c * c).mean(-1, keepdims=True) + eps) * w[p + ".weight"] + w[p + ".bias"]

    def mlp(h, p):
        return P.linear(P.swiglu(P.linear(h, w[p + ".gate_proj.weight"]), P.linear(h, w[p + ".up_proj.weight"])), w[p + ".down_proj.weight"])

    def keys_values(h, p):
        k = P.rope(P.linear(h, w[p + ".k_proj.weight"]).reshape(T, nkv, D), pos, theta)
        return k, P.linear(h, w[p + ".v_proj.weight"]).reshape(T, nkv, D)

    def attend(h, p, k, v):
        q = P.rope(P.linear(h, w[p + ".q_proj.weight"]).reshape(T, nh, D), pos, theta)
        return P.linear(P.causal_attention(q, k, v).reshape(T, nh * D), w[p + ".o_proj.weight"])

    x = np.asarray(w["embed.weight"], np.float64)[tokens]
    h = P.rmsnorm(x, w["l0.n1.weight"], eps)
    k0, v0 = keys_values(h, "l0.attn")
    x = x + attend(h, "l0.attn", k0, v0)
    x = x + mlp(P.rmsnorm(x, w["l0.n2.weight"], eps), "l0.mlp")
    x = x + attend(centred(x, "l1.n1"), "l1.attn", k0, v0)          # its own queries over the first layer's keys and values
    x = x + mlp(centred(x, "l1.n2"), "l1.mlp")
    h = P.rmsnorm(x, w["l2.n1.weight"], eps)
    k2, v2 = keys_values(h, "l2.attn")
    x = x + attend(h, "l2.attn", k2, v2)
    x = x + mlp(centred(x, "l2.n2"), "l2.mlp")
    return P.linear(centred(x, "final"), w["head.weight"])


@pytest.mark.parametrize("dtype, execution", [("float32", "eager"), ("bfloat16", "eager"), ("bfloat16", "graph")])
def test_toy_norm_and_a_layer_that_reads_another_layers_cache(tmp_path, dtype, execution):
    """A norm defined in this file (not one the product kernels can fuse) and an order of layers in which the second
    keeps no cache and reads the first one's: registered, given random weights, loaded and stepped in portions beside
    decoded tokens, against a plain implementation; only two of the three layers have pages."""
    import plain_llama as P
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import write_model_folder
    cleanup = build_shared_cache_toy()
    try:
        raw = {"model_type": "toy-shared-cache-lm", "vocab_size": 67, "hidden_size": 40, "heads": 4, "kv_heads": 2, "head_dim": 16,
               "intermediate_size": 56, "rope_theta": 5000.0, "max_position_embeddings": 128, "rms_norm_eps": 1e-5}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=11, dtype=torch.float32 if dtype == "float32" else torch.bfloat16, std=0.15)
        cfg, w = P.read_folder(tmp_path)
        assert "l1.attn.k_proj.weight" not in w and "l1.attn.q_proj.weight" in w and "l1.n1.bias" in w
        model = load_model(tmp_path, dtype=dtype)
        assert set(model.cache_needs()) == {0, 2} and model.site_of(1) == 0
        runner = ModelRunner(model, n_pages=14, page_size=8, max_requests=2, execution=execution)
        tokens = {"x": np.random.default_rng(4).integers(0, 67, 41).tolist(), "y": np.random.default_rng(5).integers(0, 67, 19).tolist()}
        want = {k: plain_shared_cache_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        plan = [[("x", 17), ("y", 3)], [("x", 1), ("y", 9)], [("x", 1), ("y", 1)], [("x", 1), ("y", 1)], [("x", 21), ("y", 5)]]
        for step in plan:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        from conftest import assert_close
        for k in tokens:
            assert_close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
        runner.cache.check()
    finally:
        cleanup()


def build_window_toy():
    """Layers with different needs in one model: two whose attention looks back over a window of keys (they share a
    group of pages, which are given back as the window passes them) around one that sees all keys (a group of its
    own).  Only the framework's parts, put together here."""
    from runtime import make_part, register_architecture
    from runtime.config import unregister_architecture
    from runtime.parts import TokenEmbedding, LMHead
    from runtime.models import Model

    @dataclass(frozen=True)
    class WindowConfig:
        vocab_size: int
        hidden_size: int
        heads: int
        kv_heads: int
        head_dim: int
        window: int
        intermediate_size: int
        rope_theta: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "heads", "kv_heads", "head_dim", "window", "intermediate_size",
                                          "rope_theta", "max_position_embeddings", "rms_norm_eps")))

    def build(c):
        def rms(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        position = make_part("position", "rotary", head_dim=c.head_dim, theta=c.rope_theta, max_positions=c.max_position_embeddings)
        def layer(n, window):
            return make_part("block", "prenorm", mixer_norm=rms(n + ".n1"),
                             mixer=make_part("mixer", "attention", name=n + ".attn", hidden=c.hidden_size, heads=c.heads,
                                             kv_heads=c.kv_heads, head_dim=c.head_dim, position=position, window=window),
                             ffn_norm=rms(n + ".n2"),
                             ffn=make_part("ffn", "gated_mlp", name=n + ".mlp", hidden=c.hidden_size, intermediate=c.intermediate_size))
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), [layer("l0", c.window), layer("l1", None), layer("l2", c.window)],
                     rms("final"), LMHead("head", c.vocab_size, c.hidden_size))

    register_architecture("toy-window-lm", WindowConfig, build)
    return lambda: unregister_architecture("toy-window-lm")


def plain_window_toy(raw, w, tokens):
    import plain_llama as P
    eps, theta, nh, nkv, D = raw["rms_norm_eps"], raw["rope_theta"], raw["heads"], raw["kv_heads"], raw["head_dim"]
    T = len(tokens)
    pos = np.arange(T)
    x = np.asarray(w["embed.weight"], np.float64)[tokens]
    for name, window in (("l0", raw["window"]), ("l1", None), ("l2", raw["window"])):
        h = P.rmsnorm(x, w[name + ".n1.weight"], eps)
        q = P.rope(P.linear(h, w[name + ".attn.q_proj.weight"]).reshape(T, nh, D), pos, theta)
        k = P.rope(P.linear(h, w[name + ".attn.k_proj.weight"]).reshape(T, nkv, D), pos, theta)
        v = P.linear(h, w[name + ".attn.v_proj.weight"]).reshape(T, nkv, D)
        x = x + P.linear(P.causal_attention(q, k, v, window=window).reshape(T, nh * D), w[name + ".attn.o_proj.weight"])
        h = P.rmsnorm(x, w[name + ".n2.weight"], eps)
        x = x + P.linear(P.swiglu(P.linear(h, w[name + ".mlp.gate_proj.weight"]), P.linear(h, w[name + ".mlp.up_proj.weight"])),
                         w[name + ".mlp.down_proj.weight"])
    return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])


@pytest.mark.parametrize("dtype, execution", [("float32", "eager"), ("bfloat16", "eager"), ("bfloat16", "graph"), ("float32", "graph")])
def test_layers_with_a_window_beside_layers_without_share_no_pages_and_give_theirs_back(tmp_path, dtype, execution):
    """Two groups of pages in one model (a window of 20 keys; all keys).  Requests run in portions longer and
    shorter than the window beside decoded tokens; the window group has far fewer pages than a request has keys,
    so the pages that the window has passed are taken again, by the same request and by the other."""
    import plain_llama as P
    from conftest import assert_close
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import write_model_folder
    cleanup = build_window_toy()
    try:
        raw = {"model_type": "toy-window-lm", "vocab_size": 71, "hidden_size": 40, "heads": 6, "kv_heads": 2, "head_dim": 16,
               "window": 20, "intermediate_size": 48, "rope_theta": 3000.0, "max_position_embeddings": 256, "rms_norm_eps": 1e-5}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=13, dtype=torch.float32 if dtype == "float32" else torch.bfloat16, std=0.15)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype=dtype)
        needs = model.cache_needs()
        assert needs[0] == needs[2] and needs[0].window == 20 and needs[1].window is None
        # 8 keys a page; the requests hold 150 + 61 keys: 27 pages where all keys stay
        runner = ModelRunner(model, n_pages=28, page_size=8, max_requests=2, execution=execution)
        groups = {g.need.window: g for g in runner.cache.groups}
        assert set(groups) == {20, None} and len(groups[20].sites) == 2 and len(groups[None].sites) == 1
        tokens = {"x": np.random.default_rng(6).integers(0, 71, 150).tolist(), "y": np.random.default_rng(7).integers(0, 71, 61).tolist()}
        want = {k: plain_window_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        plan = [[("x", 45), ("y", 2)], [("x", 1), ("y", 7)], [("x", 1), ("y", 1)], [("x", 33), ("y", 1)], [("x", 2), ("y", 30)],
                [("x", 1), ("y", 1)], [("x", 50), ("y", 1)], [("x", 1), ("y", 17)], [("x", 16), ("y", 1)]]
        most_window_pages = 0
        for step in plan:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
            runner.cache.check()
            most_window_pages = max(most_window_pages, groups[20].pool.used)
        assert fed == {k: len(v) for k, v in tokens.items()}
        for k in tokens:
            assert_close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
        # the window group never held more than a window and a portion a request (here: 20 + 50 and 20 + 30 keys, 8 a page)
        assert most_window_pages <= 9 + 7 + 2, most_window_pages
        assert groups[None].pool.used == 19 + 8
        runner.release("x"); runner.release("y")
        runner.cache.check()
        assert all(g.pool.used == 0 for g in runner.cache.groups)
    finally:
        cleanup()


def build_partial_rotary_toy():
    """The framework's attention with other constants than the architecture's: a rotary embedding that turns only the
    first 8 of a head's 24 coordinates, and a score scale that is not 1/sqrt(head size); the second layer is plain."""
    from runtime import make_part, register_architecture
    from runtime.config import unregister_architecture
    from runtime.parts import TokenEmbedding, LMHead
    from runtime.models import Model

    @dataclass(frozen=True)
    class PartialConfig:
        vocab_size: int
        hidden_size: int
        rotary_dim: int
        score_scale: float
        rope_theta: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "rotary_dim", "score_scale", "rope_theta",
                                          "max_position_embeddings", "rms_norm_eps")))

    def build(c):
        def rms(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        partial = make_part("position", "rotary", head_dim=24, theta=c.rope_theta, max_positions=c.max_position_embeddings, rotary_dim=c.rotary_dim)
        whole = make_part("position", "rotary", head_dim=24, theta=c.rope_theta, max_positions=c.max_position_embeddings)
        def layer(n, position, scale):
            return make_part("block", "prenorm", mixer_norm=rms(n + ".n1"),
                             mixer=make_part("mixer", "attention", name=n + ".attn", hidden=c.hidden_size, heads=3, kv_heads=3,
                                             head_dim=24, position=position, scale=scale),
                             ffn_norm=rms(n + ".n2"),
                             ffn=make_part("ffn", "gated_mlp", name=n + ".mlp", hidden=c.hidden_size, intermediate=40))
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), [layer("l0", partial, c.score_scale), layer("l1", whole, None)],
                     rms("final"), LMHead("head", c.vocab_size, c.hidden_size))

    register_architecture("toy-partial-rotary-lm", PartialConfig, build)
    return lambda: unregister_architecture("toy-partial-rotary-lm")


def plain_partial_rotary_toy(raw, w, tokens):
    import plain_llama as P
    eps, theta, rot, scale = raw["rms_norm_eps"], raw["rope_theta"], raw["rotary_dim"], raw["score_scale"]
    T, nh, D = len(tokens), 3, 24
    pos = np.arange(T)
    x = np.asarray(w["embed.weight"], np.float64)[tokens]
    for name, turned, s in (("l0", rot, scale), ("l1", D, 1 / np.sqrt(D))):
        h = P.rmsnorm(x, w[name + ".n1.weight"], eps)
        q = P.linear(h, w[name + ".attn.q_proj.weight"]).reshape(T, nh, D)
        k = P.linear(h, w[name + ".attn.k_proj.weight"]).reshape(T, nh, D)
        v = P.linear(h, w[name + ".attn.v_proj.weight"]).reshape(T, nh, D)
        # the first `turned` coordinates turn (pairs (i, i + turned/2) by pos * theta^(-2i/turned)), the rest pass
        q = np.concatenate([P.rope(q[..., :turned], pos, theta), q[..., turned:]], axis=-1)
        k = np.concatenate([P.rope(k[..., :turned], pos, theta), k[..., turned:]], axis=-1)
        q = q * (s * np.sqrt(D))                                   # the plain attention divides by sqrt(D)
        x = x + P.linear(P.causal_attention(q, k, v).reshape(T, nh * D), w[name + ".attn.o_proj.weight"])
        h = P.rmsnorm(x, w[name + ".n2.weight"], eps)
        x = x + P.linear(P.swiglu(P.linear(h, w[name + ".mlp.gate_proj.weight"]), P.linear(h, w[name + ".mlp.up_proj.weight"])),
                         w[name + ".mlp.down_proj.weight"])
    return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])


@pytest.mark.parametrize("dtype, execution", [("float32", "eager"), ("bfloat16", "eager"), ("bfloat16", "graph")])
def test_attention_with_a_partial_rotary_embedding_and_a_scale_of_its_own(tmp_path, dtype, execution):
    """The constants of a part are its parameters: a head of 24 coordinates (not a power of two) of which 8 turn, and
    scores scaled by 0.31, through the framework's attention in portions beside decoded tokens."""
    import plain_llama as P
    from conftest import assert_close
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import write_model_folder
    cleanup = build_partial_rotary_toy()
    try:
        raw = {"model_type": "toy-partial-rotary-lm", "vocab_size": 59, "hidden_size": 48, "rotary_dim": 8, "score_scale": 0.31,
               "rope_theta": 700.0, "max_position_embeddings": 96, "rms_norm_eps": 1e-6}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=17, dtype=torch.float32 if dtype == "float32" else torch.bfloat16, std=0.15)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype=dtype)
        runner = ModelRunner(model, n_pages=16, page_size=8, max_requests=2, execution=execution)
        tokens = {"x": np.random.default_rng(8).integers(0, 59, 44).tolist(), "y": np.random.default_rng(9).integers(0, 59, 23).tolist()}
        want = {k: plain_partial_rotary_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        for step in [[("x", 19), ("y", 2)], [("x", 1), ("y", 11)], [("x", 1), ("y", 1)], [("x", 23), ("y", 9)]]:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            assert_close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
        # both constants matter: with all 24 coordinates turned, or with the usual scale, the logits are others
        assert np.abs(plain_partial_rotary_toy(dict(raw, rotary_dim=24), w, tokens["x"]) - want["x"]).max() > 1e-3
        assert np.abs(plain_partial_rotary_toy(dict(raw, score_scale=1 / np.sqrt(24)), w, tokens["x"]) - want["x"]).max() > 1e-3
        runner.cache.check()
    finally:
        cleanup()


def build_biased_toy():
    """The framework's attention and feed-forward with biases on their projections (no architecture of the family has
    them): the first layer on all seven projections, the second on q/k/v only."""
    from runtime import make_part, register_architecture
    from runtime.config import unregister_architecture
    from runtime.parts import TokenEmbedding, LMHead
    from runtime.models import Model

    @dataclass(frozen=True)
    class BiasedConfig:
        vocab_size: int
        hidden_size: int
        rope_theta: float
        max_position_embeddings: int
        rms_norm_eps: float

        @classmethod
        def from_dict(cls, raw):
            return cls(*(raw[k] for k in ("vocab_size", "hidden_size", "rope_theta", "max_position_embeddings", "rms_norm_eps")))

    def build(c):
        def rms(n): return make_part("norm", "rmsnorm", name=n, dim=c.hidden_size, eps=c.rms_norm_eps)
        position = make_part("position", "rotary", head_dim=16, theta=c.rope_theta, max_positions=c.max_position_embeddings)
        def layer(n, out_bias, mlp_bias):
            return make_part("block", "prenorm", mixer_norm=rms(n + ".n1"),
                             mixer=make_part("mixer", "attention", name=n + ".attn", hidden=c.hidden_size, heads=4, kv_heads=2,
                                             head_dim=16, position=position, bias=True, out_bias=out_bias),
                             ffn_norm=rms(n + ".n2"),
                             ffn=make_part("ffn", "gated_mlp", name=n + ".mlp", hidden=c.hidden_size, intermediate=56, bias=mlp_bias))
        return Model(c, TokenEmbedding("embed", c.vocab_size, c.hidden_size), [layer("l0", True, True), layer("l1", False, False)],
                     rms("final"), LMHead("head", c.vocab_size, c.hidden_size))

    register_architecture("toy-biased-lm", BiasedConfig, build)
    return lambda: unregister_architecture("toy-biased-lm")


def plain_biased_toy(raw, w, tokens, without=()):
    """`without`: names of biases taken as zero."""
    import plain_llama as P
    eps, theta = raw["rms_norm_eps"], raw["rope_theta"]
    T, nh, nkv, D = len(tokens), 4, 2, 16
    pos = np.arange(T)

    def lin(x, name):
        y = P.linear(x, w[name + ".weight"])
        if name + ".bias" in w and name + ".bias" not in without:
            y = y + np.asarray(w[name + ".bias"], np.float64)
        return y

    x = np.asarray(w["embed.weight"], np.float64)[tokens]
    for name in ("l0", "l1"):
        h = P.rmsnorm(x, w[name + ".n1.weight"], eps)
        q = P.rope(lin(h, name + ".attn.q_proj").reshape(T, nh, D), pos, theta)
        k = P.rope(lin(h, name + ".attn.k_proj").reshape(T, nkv, D), pos, theta)
        v = lin(h, name + ".attn.v_proj").reshape(T, nkv, D)
        k, v = np.repeat(k, nh // nkv, axis=1), np.repeat(v, nh // nkv, axis=1)
        x = x + lin(P.causal_attention(q, k, v).reshape(T, nh * D), name + ".attn.o_proj")
        h = P.rmsnorm(x, w[name + ".n2.weight"], eps)
        x = x + lin(P.swiglu(lin(h, name + ".mlp.gate_proj"), lin(h, name + ".mlp.up_proj")), name + ".mlp.down_proj")
    return P.linear(P.rmsnorm(x, w["final.weight"], eps), w["head.weight"])


@pytest.mark.parametrize("dtype, execution", [("float32", "eager"), ("bfloat16", "eager"), ("bfloat16", "graph")])
def test_projections_with_biases(tmp_path, dtype, execution):
    """A bias is a parameter of the framework's own attention and feed-forward: the products run as they are, a small
    kernel adds the bias before the rotary embedding, the activation or the residual sum; portions beside decoded tokens."""
    import plain_llama as P
    from conftest import assert_close
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import write_model_folder
    cleanup = build_biased_toy()
    try:
        raw = {"model_type": "toy-biased-lm", "vocab_size": 67, "hidden_size": 40, "rope_theta": 900.0,
               "max_position_embeddings": 96, "rms_norm_eps": 1e-6}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        names = [spec.name for spec in blueprint.tensor_specs()]
        assert sum(n.endswith(".bias") for n in names) == 7 + 3
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=23, dtype=torch.float32 if dtype == "float32" else torch.bfloat16, std=0.15)
        cfg, w = P.read_folder(tmp_path)
        model = load_model(tmp_path, dtype=dtype)
        runner = ModelRunner(model, n_pages=16, page_size=8, max_requests=2, execution=execution)
        tokens = {"x": np.random.default_rng(18).integers(0, 67, 41).tolist(), "y": np.random.default_rng(19).integers(0, 67, 25).tolist()}
        want = {k: plain_biased_toy(raw, w, v) for k, v in tokens.items()}
        runner.create("x"); runner.create("y")
        got, fed = {"x": [], "y": []}, {"x": 0, "y": 0}
        for step in [[("x", 17), ("y", 2)], [("x", 1), ("y", 12)], [("x", 1), ("y", 1)], [("x", 22), ("y", 10)]]:
            entries = [StepEntry(k, tokens[k][fed[k]:fed[k] + n], list(range(n))) for k, n in step]
            out = runner.step(entries).float().cpu().numpy()
            row = 0
            for k, n in step:
                got[k].append(out[row:row + n]); row += n; fed[k] += n
        for k in tokens:
            assert_close(np.concatenate(got[k]), want[k], dtype, f"request {k}")
        # every kind of bias matters: with one of them taken as zero the logits are others
        for name in ("l0.attn.q_proj.bias", "l0.attn.k_proj.bias", "l1.attn.v_proj.bias", "l0.attn.o_proj.bias",
                     "l0.mlp.gate_proj.bias", "l0.mlp.up_proj.bias", "l0.mlp.down_proj.bias"):
            assert np.abs(plain_biased_toy(raw, w, tokens["x"], without=(name,)) - want["x"]).max() > 1e-3, name
        runner.cache.check()
    finally:
        cleanup()


@pytest.mark.parametrize("execution, overlap", [("eager", False), ("graph", True)])
def test_scheduler_generates_with_a_model_of_two_page_groups(tmp_path, execution, overlap):
    """The entry point over the model with windowed and full layers: requests admitted by what each group of pages
    can promise, prompts cut into portions, greedy tokens equal to the plain implementation's, every page given back."""
    import plain_llama as P
    from runtime.engine.loading import build_from_config_dict
    from runtime.engine.scheduler import Engine
    from runtime.weights import write_model_folder
    cleanup = build_window_toy()
    try:
        raw = {"model_type": "toy-window-lm", "vocab_size": 71, "hidden_size": 40, "heads": 6, "kv_heads": 2, "head_dim": 16,
               "window": 20, "intermediate_size": 48, "rope_theta": 3000.0, "max_position_embeddings": 256, "rms_norm_eps": 1e-5}
        tmp_path.mkdir(exist_ok=True)
        _, _, blueprint = build_from_config_dict(raw)
        write_model_folder(tmp_path, raw, blueprint.tensor_specs(), seed=13, dtype=torch.float32, std=0.3)
        cfg, w = P.read_folder(tmp_path)
        prompts = [np.random.default_rng(20 + i).integers(0, 71, n).tolist() for i, n in enumerate((37, 5, 52, 18))]

        def plain_greedy(prompt, steps):
            tokens, new = list(prompt), []
            for _ in range(steps):
                row = plain_window_toy(raw, w, tokens)[-1]
                top = np.sort(row)[-2:]
                assert top[1] - top[0] > 1e-3, "a near-tie in the plain logits: choose other weights"
                new.append(int(row.argmax())); tokens.append(new[-1])
            return new

        want = [plain_greedy(p, 9) for p in prompts]
        engine = Engine.from_folder(tmp_path, dtype="float32", pages=12, page_size=8, execution=execution, max_active=3,
                                    token_budget=24, prefill_chunk=16, policy="decode_first", overlap=overlap)
        got = engine.generate(prompts, max_new_tokens=9)
        assert got == want
        cache = engine.runner.cache
        cache.check()
        assert all(g.pool.used == 0 for g in cache.groups) and len(cache.groups) == 2
        # 12 pages of 8 keys a group: the longest request (52 + 8 keys) takes 8 of the group that keeps all keys, so
        # the four requests cannot all have been live at once
        assert max(step["active"] for step in engine.trace) <= 3
    finally:
        cleanup()


PLUGIN = '''"""An architecture of a module of its own: the framework's parts under other config.json keys."""
from dataclasses import dataclass

from runtime import make_part, register_architecture
from runtime.models import Model
from runtime.parts import LMHead, TokenEmbedding


@dataclass(frozen=True)
class KeysConfig:
    width: int
    depth: int
    n_heads: int
    n_kv: int
    head: int
    ffn: int
    vocab: int
    theta: float
    eps: float
    max_len: int

    @classmethod
    def from_dict(cls, raw):
        return cls(*(raw[k] for k in ("width", "depth", "n_heads", "n_kv", "head", "ffn", "vocab", "theta", "eps", "max_len")))


def build(c):
    def norm(name):
        return make_part("norm", "rmsnorm", name=name, dim=c.width, eps=c.eps)
    position = make_part("position", "rotary", head_dim=c.head, theta=c.theta, max_positions=c.max_len)
    layers = []
    for i in range(c.depth):
        p = f"model.layers.{i}"
        layers.append(make_part(
            "block", "prenorm", mixer_norm=norm(p + ".input_layernorm"),
            mixer=make_part("mixer", "attention", name=p + ".self_attn", hidden=c.width, heads=c.n_heads, kv_heads=c.n_kv,
                            head_dim=c.head, position=position),
            ffn_norm=norm(p + ".post_attention_layernorm"),
            ffn=make_part("ffn", "gated_mlp", name=p + ".mlp", hidden=c.width, intermediate=c.ffn)))
    return Model(c, TokenEmbedding("model.embed_tokens", c.vocab, c.width), layers, norm("model.norm"),
                 LMHead("lm_head", c.vocab, c.width), max_positions=c.max_len, vocab_size=c.vocab)


register_architecture(["other-keys-lm"], KeysConfig, build)
'''


def test_an_architecture_of_a_module_of_its_own_runs_through_both_programs(tmp_path):
    """A module outside the package registers an architecture at import; `--plugin` names it to the command line and to
    the replay program, which then choose it by config.json as they choose the framework's own.  Without the option the
    registry's error names the architecture it does not know."""
    import json, os, subprocess, sys
    from pathlib import Path
    import plain_llama as P
    from runtime.config import unregister_architecture
    from runtime.engine.loading import build_from_config_dict, import_plugins
    from runtime.weights import write_model_folder
    root = Path(__file__).resolve().parent.parent
    (tmp_path / "other_keys_plugin.py").write_text(PLUGIN)
    raw = {"model_type": "other-keys-lm", "width": 72, "depth": 2, "n_heads": 6, "n_kv": 2, "head": 16, "ffn": 120, "vocab": 211,
           "theta": 5e4, "eps": 1e-6, "max_len": 128}
    sys.path.insert(0, str(tmp_path))
    try:
        import_plugins(["other_keys_plugin"])
        _, _, blueprint = build_from_config_dict(raw)
        folder = tmp_path / "model"
        write_model_folder(folder, raw, blueprint.tensor_specs(), seed=9, dtype=torch.float32)
    finally:
        sys.path.remove(str(tmp_path))
        sys.modules.pop("other_keys_plugin", None)
        unregister_architecture("other-keys-lm")
    _, w = P.read_folder(folder)
    cfg = dict(num_hidden_layers=2, hidden_size=72, num_attention_heads=6, num_key_value_heads=2, head_dim=16, rope_theta=5e4,
               rms_norm_eps=1e-6, tie_word_embeddings=False)
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([str(root), str(tmp_path)]))
    base = [sys.executable, "-m", "runtime", "--checkpoint", str(folder), "--dtype", "float32", "--tokens", "5,6,7", "--max-new-tokens", "4",
            "--execution", "eager"]
    proc = subprocess.run(base + ["--plugin", "other_keys_plugin"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert json.loads(proc.stdout)["requests"][0]["generated"] == P.greedy(cfg, w, [5, 6, 7], 4)
    proc = subprocess.run(base, capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode != 0 and "other-keys-lm" in proc.stderr
    tokens = np.random.default_rng(3).integers(0, 211, 40).tolist()
    trace = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:33], "want": [32]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[33:], "want": list(range(7))}], "end": ["a"]}]
    proc = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(tmp_path / "out"),
                           "--max-tokens", "64", "--plugin", "other_keys_plugin"], input="".join(json.dumps(t) + "\n" for t in trace),
                          capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0 and proc.stdout.split() == ["done", "0", "done", "1"], proc.stderr[-2000:]
    want = P.forward(cfg, w, tokens)
    got = np.concatenate([np.fromfile(tmp_path / "out" / f"{i}.f32", dtype="<f4").reshape(-1, 211) for i in (0, 1)])
    np.testing.assert_allclose(got, want[32:], rtol=2e-4, atol=2e-5)
