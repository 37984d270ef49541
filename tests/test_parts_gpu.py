"""Each part of a layer alone against the plain implementation, driven through
the step context of a real runner (so the cache and metadata are the engine's)."""
import numpy as np
import pytest
import torch

import plain_llama as P


pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def f64(t):
    return t.detach().double().cpu().numpy()


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def setup(request, folders):
    from runtime.engine import load_model, ModelRunner, StepEntry
    name = "c"
    model = load_model(folders[name], dtype=request.param)
    runner = ModelRunner(model, n_pages=16, page_size=8)
    cfg, w = P.read_folder(folders[name])
    return model, runner, cfg, w, request.param, StepEntry


def close(got, want, dtype):
    """float32: largest difference over largest magnitude; bfloat16: relative rmse."""
    if dtype == "float32":
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err < 2e-5, err
    else:
        err = np.linalg.norm(got - want) / (np.linalg.norm(want) + 1e-30)
        assert err < 0.02, err


def test_norm_part(setup):
    model, runner, cfg, w, dtype, StepEntry = setup
    runner.create("n")
    ctx = runner._context([StepEntry("n", [1, 2, 3], [])], runner.cache.append_many([("n", 3)]))
    x = torch.randn(3, cfg["hidden_size"], device=DEV) * 2
    norm = model.layers[1].ffn_norm
    got = norm.forward(x, ctx)
    close(f64(got), P.rmsnorm(f64(x), w["model.layers.1.post_attention_layernorm.weight"], cfg["rms_norm_eps"]), dtype)
    runner.release("n")


def test_position_part_tables(setup):
    model, *_ , cfg, w, dtype, _ = setup
    rope = model.layers[0].mixer.position
    cos, sin = rope.tables()
    d = cfg["head_dim"]
    ang = np.arange(cfg["max_position_embeddings"])[:, None] * cfg["rope_theta"] ** (-np.arange(d // 2) * 2.0 / d)
    assert cos.dtype == torch.float32 and tuple(cos.shape) == (cfg["max_position_embeddings"], d // 2)
    np.testing.assert_allclose(f64(cos), np.cos(ang), atol=1e-7)
    np.testing.assert_allclose(f64(sin), np.sin(ang), atol=1e-7)


def test_ffn_part(setup):
    model, runner, cfg, w, dtype, StepEntry = setup
    runner.create("f")
    ctx = runner._context([StepEntry("f", [1] * 5, [])], runner.cache.append_many([("f", 5)]))
    h32 = torch.randn(5, cfg["hidden_size"], device=DEV)
    h = h32.to(model.dtype)
    res = torch.randn(5, cfg["hidden_size"], device=DEV)
    want = f64(res) + P.linear(P.swiglu(P.linear(f64(h), w["model.layers.0.mlp.gate_proj.weight"]),
                                        P.linear(f64(h), w["model.layers.0.mlp.up_proj.weight"])),
                               w["model.layers.0.mlp.down_proj.weight"])
    got = model.layers[0].ffn.forward(h, res.clone(), ctx)
    assert got.dtype == torch.float32   # the residual stream stays float
    close(f64(got), want, dtype)
    runner.release("f")


def test_attention_part_in_two_portions(setup):
    model, runner, cfg, w, dtype, StepEntry = setup
    nh, nkv, D, H = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"], cfg["hidden_size"]
    mixer = model.layers[1].mixer
    T = 21
    h_all = (torch.randn(T, H, device=DEV)).to(model.dtype)
    res_all = torch.randn(T, H, device=DEV)
    p = "model.layers.1.self_attn."
    pos = np.arange(T)
    q = P.rope(P.linear(f64(h_all), w[p + "q_proj.weight"]).reshape(T, nh, D), pos, cfg["rope_theta"])
    k = P.rope(P.linear(f64(h_all), w[p + "k_proj.weight"]).reshape(T, nkv, D), pos, cfg["rope_theta"])
    v = P.linear(f64(h_all), w[p + "v_proj.weight"]).reshape(T, nkv, D)
    want = f64(res_all) + P.linear(P.causal_attention(q, k, v).reshape(T, nh * D), w[p + "o_proj.weight"])
    runner.create("m")
    outs = []
    for lo, hi in ((0, 13), (13, 21)):   # the second portion attends to the first through the cache
        ctx = runner._context([StepEntry("m", [0] * (hi - lo), [])], runner.cache.append_many([("m", hi - lo)]))
        outs.append(mixer.forward(h_all[lo:hi].contiguous(), res_all[lo:hi].clone(), ctx, site=1).clone())
    close(f64(torch.cat(outs)), want, dtype)
    runner.release("m")


def test_block_part(setup):
    model, runner, cfg, w, dtype, StepEntry = setup
    tokens = [7, 100, 3, 999, 50, 2, 2, 640]
    want = P.forward(cfg, w, tokens, upto_layer=1)
    runner.create("b")
    ctx = runner._context([StepEntry("b", tokens, [])], runner.cache.append_many([("b", len(tokens))]))
    x = model.embedding.forward(ctx)
    np.testing.assert_array_equal(f64(x), w["model.embed_tokens.weight"][tokens])
    got = model.layers[0].forward(x, ctx, 0)
    close(f64(got), want, dtype)
    runner.release("b")
    runner.cache.check()


def test_product_left_to_the_next_norm_only_if_that_norm_adds_it(folders, monkeypatch, no_gemv):
    """ctx.add_product leaves a product that the wide kernel cuts into slices to the norm named in ctx.next_norm, if
    that norm says it adds partial sums; RMSNorm.forward then gives the norm of the finished rows and finishes them;
    any other reader (no norm named, a norm of another kind, ctx.settle) gets finished rows."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.kernels import ops
    from runtime.parts import RMSNorm
    for limit in ("WIDE_MIN_BYTES", "WIDE_MIN_BYTES_FEW_ROWS", "WIDE_MIN_BYTES_MANY_ROWS"):
        monkeypatch.setattr(ops, limit, 0)
    model = load_model(folders["a"], dtype="bfloat16")
    runner = ModelRunner(model, n_pages=16, page_size=8)
    runner.create("u")
    ctx = runner._context([StepEntry("u", [1] * 6, [])], runner.cache.append_many([("u", 6)]))
    torch.manual_seed(0)
    M, N, K = 6, 64, 8192
    a = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(N, K, device=DEV) * 0.02).bfloat16()
    r = torch.randn(M, N, device=DEV)
    assert ops._wide_plan(M, N, K, False) > 0, "this shape was meant to be cut into slices"
    want = ops.gemm(a, w, r.clone(), residual=None) + r

    class OtherNorm:                  # knows nothing of partial sums
        def forward(self, x, ctx):
            return x * 2

    norm = RMSNorm("n", N, 1e-5)
    norm.weight = 1 + 0.1 * torch.randn(N, device=DEV)
    for reader in (None, OtherNorm()):
        ctx.next_norm = reader
        x = ctx.add_product(a, w, r.clone())
        assert ctx.unfinished is None
        torch.testing.assert_close(x, want, rtol=1e-5, atol=1e-5)
    ctx.next_norm = norm
    x = ctx.add_product(a, w, r.clone())
    assert ctx.unfinished is not None and torch.equal(x, r)
    y = norm.forward(x, ctx)
    assert ctx.unfinished is None
    torch.testing.assert_close(x, want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(y.float(), ops.rmsnorm(want, norm.weight, torch.empty(M, N, device=DEV), 1e-5), rtol=2e-2, atol=2e-2)
    x = ctx.add_product(a, w, r.clone())
    with pytest.raises(RuntimeError):
        ctx.add_product(a, w, r.clone())          # a second one before the first was added
    with pytest.raises(RuntimeError):
        ctx.settle(torch.zeros(M, N, device=DEV))  # other rows
    ctx.settle(x)
    torch.testing.assert_close(x, want, rtol=1e-5, atol=1e-5)
    ctx.settle(x)                                  # nothing left: no change
    torch.testing.assert_close(x, want, rtol=1e-5, atol=1e-5)
    runner.release("u")


def test_head_part_tied_and_untied(folders):
    from runtime.engine import load_model
    tied = load_model(folders["a"], dtype="bfloat16")
    untied = load_model(folders["b"], dtype="bfloat16")
    assert tied.head.weight.data_ptr() == tied.embedding.weight.data_ptr()      # one buffer when tied
    assert untied.head.weight.data_ptr() != untied.embedding.weight.data_ptr()
    assert tied.head.tensor_specs() == [] and len(untied.head.tensor_specs()) == 1


def test_stored_32bit_matrix_runs_in_bf16_by_rounding(tmp_path, folders):
    """A folder stored in float32: the float32 run uses the values as they are,
    the bfloat16 run rounds matrices to nearest even and keeps norm weights float."""
    import json
    from safetensors.torch import load_file, save_file
    from runtime.engine import load_model
    src = folders["a"]
    tensors = {k: (v.float() + 1e-3) for k, v in load_file(str(src / "model.safetensors")).items()}
    (tmp_path / "config.json").write_text((src / "config.json").read_text())
    save_file(tensors, str(tmp_path / "model.safetensors"))
    m32 = load_model(tmp_path, dtype="float32")
    m16 = load_model(tmp_path, dtype="bfloat16")
    name = "model.layers.0.mlp.down_proj.weight"
    assert torch.equal(m32.layers[0].ffn.w_down.cpu(), tensors[name])
    assert torch.equal(m16.layers[0].ffn.w_down.cpu(), tensors[name].to(torch.bfloat16))
    assert m16.layers[0].ffn_norm.weight.dtype == torch.float32
    assert torch.equal(m16.layers[0].ffn_norm.weight.cpu(), tensors["model.layers.0.post_attention_layernorm.weight"])
