"""Host-side pieces of the Ratilorn worker (no GPU): the configuration reader, the registry, the block and slot layout, and the
plain implementation's own mechanisms against closed forms and against themselves (whole against token by token)."""
import json
import math

import pytest
import torch

import ratilorn_oracle as O
from swiftllm_amd import registry
from swiftllm_amd.model_config import RatilornModelConfig


def test_config_reads_every_layer():
    layers = [O.parallel_layer(heads=6, kv_heads=3, dim=16, vdim=24, s_heads=4, s_vdim=6, state=10, groups=2, conv=3,
                               norm_groups=3, mlp=O.moe_mlp(ff=12, experts=6, top=2, groups=(3, 2), shared=20)),
              O.attention_layer(heads=4, kv_heads=2, dim=8, vdim=12, v_mix=False, mlp=None),
              O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=24, v_mix=True, mlp=O.dense_mlp(36)),
              O.attention_layer(heads=2, kv_heads=2, dim=32, vdim=12, v_mix=True,
                                mlp=O.moe_mlp(ff=16, experts=5, top=1, groups=None, shared=0))]
    cfg = RatilornModelConfig(O.make_config(layers=layers, width=44, vocab=37, max_positions=96, logit_scale=1.7))
    assert (cfg.hidden_size, cfg.vocab_size, cfg.max_position_embeddings, cfg.norm_eps, cfg.logit_scale) == (44, 37, 96, 1e-5, 1.7)
    par = cfg.layers[0].mixer
    assert (par.left.q_size, par.left.k_size, par.left.v_size, par.left.o_size, par.left.sigmoid) == (96, 48, 72, 144, False)
    assert (par.right.inner, par.right.conv_channels, par.right.proj_size, par.right.state_elems) == (24, 64, 92, 240)
    assert (par.right.groups, par.right.conv_taps, par.right.norm_groups) == (2, 3, 3)
    m = cfg.layers[0].mlp
    assert (m.kind, m.ffn_inter_dim, m.num_experts, m.top_k, m.group_count, m.group_keep, m.shared_ffn_inter_dim) == \
        ("moe", 12, 6, 2, 3, 2, 20)
    assert cfg.layers[1].mlp is None and not cfg.layers[1].mixer.v_mix and cfg.layers[1].mixer.sigmoid
    assert cfg.layers[2].mlp.kind == "dense" and cfg.layers[2].mlp.ffn_inter_dim == 36
    last = cfg.layers[3].mlp
    assert (last.group_count, last.group_keep, last.shared_ffn_inter_dim) == (1, 1, 0)       # no groups: every expert eligible
    assert cfg.v_mix_layers == [2, 3] and cfg.has_state
    assert cfg.kv_elems_per_token() == (48 + 72) + (16 + 24) + (24 + 24) + (64 + 24)
    assert not RatilornModelConfig(O.make_config(layers=[O.attention_layer()])).has_state


def test_config_refuses_what_cannot_run():
    with pytest.raises(ValueError):     # blended values of different sizes
        RatilornModelConfig(O.make_config(layers=[O.attention_layer(kv_heads=2, vdim=16), O.attention_layer(kv_heads=2, vdim=8)]))
    RatilornModelConfig(O.make_config(layers=[O.attention_layer(kv_heads=2, vdim=16),
                                              O.attention_layer(kv_heads=2, vdim=8, v_mix=False)]))
    with pytest.raises(ValueError):
        RatilornModelConfig(O.make_config(layers=[O.attention_layer(heads=3, kv_heads=2)]))
    with pytest.raises(ValueError):
        RatilornModelConfig(O.make_config(layers=[O.parallel_layer(s_heads=3, groups=2)]))
    with pytest.raises(ValueError):
        RatilornModelConfig(O.make_config(layers=[O.parallel_layer(s_heads=3, s_vdim=8, norm_groups=5)]))
    with pytest.raises(ValueError):     # the kept groups hold fewer experts than are to be chosen
        RatilornModelConfig(O.make_config(layers=[O.attention_layer(mlp=O.moe_mlp(experts=8, top=3, groups=(4, 1)))]))
    with pytest.raises(ValueError):
        RatilornModelConfig(O.make_config(layers=[O.attention_layer(mlp=O.moe_mlp(experts=9, top=2, groups=(4, 2)))]))
    bad = O.make_config()
    bad["layers"][0]["type"] = "delta"
    with pytest.raises(ValueError):
        RatilornModelConfig(bad)


def test_registry_knows_the_design(tmp_path):
    cfg = O.make_config()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert registry.architecture_of(cfg) == "Ratilorn"
    assert isinstance(registry.load_model_config(str(tmp_path)), RatilornModelConfig)
    assert registry.MODELS["Ratilorn"][1].endswith(":RatilornModel")
    from swiftllm_amd.csrc import build
    assert {"sigmoid_attn.hip", "ssd.hip", "moe.hip", "rms_stream.hip", "qknorm_kv.hip"} <= set(build.MODEL_SOURCES["Ratilorn"])
    assert set(build.MODEL_SOURCES["Ratilorn"]) <= set(build.SOURCES)


def test_checkpoint_names_and_shapes_round_trip(tmp_path):
    """What the test writer writes is what the framework's reader finds: every tensor the loader asks for, with its shape."""
    from swiftllm_amd.worker.kekapel_weight import _checkpoint_getter
    cfg = O.make_config()
    W = O.random_weights(cfg, 0)
    O.write_checkpoint(str(tmp_path), cfg, W)
    get = _checkpoint_getter(str(tmp_path))
    for name, shape in O.tensor_shapes(cfg).items():
        assert torch.equal(get(name, shape).float(), W[name])
    with pytest.raises(ValueError):
        get("embed", (cfg["vocab"] + 1, cfg["width"]))


# ---- the plain implementation against closed forms -----------------------------------------------------------------------------
def test_router_choice_by_hand():
    # 8 experts in 4 groups of 2, keep 2, top 3. Choice scores c = sigmoid(z) + correction.
    s = torch.tensor([[0.9, 0.1, 0.5, 0.5, 0.2, 0.95, 0.6, 0.3]], dtype=torch.float64)
    z = torch.log(s / (1 - s))
    corr = torch.tensor([0.0, 0.0, 0.3, 0.3, 0.0, -0.9, 0.0, 0.0], dtype=torch.float64)
    # c = [.9 .1 | .8 .8 | .2 .05 | .6 .3]; group scores 1.0, 1.6, 0.25, 0.9 -> groups 1 and 0 are kept
    idx, w = O.route(z, corr, 3, {"count": 4, "keep": 2})
    assert sorted(idx[0].tolist()) == [0, 2, 3]
    chosen = s[0, idx[0]]
    assert torch.allclose(w[0], chosen / chosen.sum())          # the weights use s WITHOUT the correction
    # without groups the best three by c are 0, 2, 3 as well; with keep = 1 only group 1 is left and top must fit it
    assert sorted(O.route(z, corr, 2, {"count": 4, "keep": 1})[0][0].tolist()) == [2, 3]
    # negative choice scores: masking an excluded expert with a zero would let it win
    neg = torch.full((1, 8), -2.0, dtype=torch.float64)
    idx, _ = O.route(z, neg, 2, {"count": 4, "keep": 1})
    g = (torch.sigmoid(z) + neg).view(4, 2).sum(-1)         # all choice scores are negative here: a zero would win
    assert int(g.argmax()) == idx[0, 0] // 2 == idx[0, 1] // 2 == 2


def test_group_of_one_expert_scores_by_that_expert():
    z = torch.tensor([[0.1, 2.0, -1.0, 0.5]], dtype=torch.float64)
    idx, w = O.route(z, torch.zeros(4, dtype=torch.float64), 2, {"count": 4, "keep": 2})
    assert sorted(idx[0].tolist()) == [1, 3]
    assert abs(float(w.sum()) - 1) < 1e-12


def test_sigmoid_attention_of_one_key_by_hand():
    cfg = O.make_config(layers=[O.attention_layer(heads=2, kv_heads=1, dim=4, vdim=3, mlp=None)], width=8)
    W = {k: v.double() for k, v in O.random_weights(cfg, 1).items()}
    mx, p, eps = cfg["layers"][0]["mixer"], "l0.mix.", 1e-5
    W[p + "o"] = torch.eye(6, dtype=torch.float64)
    h = torch.randn(2, 8, dtype=torch.float64)
    out, v = O.sigmoid_attention(h, W, p, mx, eps)
    q = O.unit_rms((h @ W[p + "q"].T + W[p + "q.b"]).view(2, 2, 4), eps)
    k = O.unit_rms((h @ W[p + "k"].T + W[p + "k.b"]).view(2, 1, 4), eps)
    # the first token sees itself only, at distance 0: no distance term
    a0 = torch.sigmoid(torch.stack([(q[0, hh] * k[0, 0]).sum() * mx["scale"] + W[p + "pb"][hh] for hh in range(2)]))
    mixed = W[p + "talk"] @ a0
    assert torch.allclose(out[0].view(2, 3), mixed.view(2, 1) * v[0].view(1, 3))
    # the second token's weight on the first key carries r1 ln(1 + r2)
    s = (q[1, 1] * k[0, 0]).sum() * mx["scale"] - W[p + "r1"][1] * math.log(1 + float(W[p + "r2"][1])) + W[p + "pb"][1]
    a10 = torch.sigmoid(s)
    a11 = torch.sigmoid((q[1, 1] * k[1, 0]).sum() * mx["scale"] + W[p + "pb"][1])
    # with an identity mixing matrix head 1 would give a10 v_0 + a11 v_1
    W[p + "talk"] = torch.eye(2, dtype=torch.float64)
    out2, _ = O.sigmoid_attention(h, W, p, mx, eps)
    assert torch.allclose(out2[1].view(2, 3)[1], a10 * v[0] + a11 * v[1])


def test_recurrence_whole_equals_token_by_token_with_carried_state():
    """The plain recurrence run whole against a second plain form that carries the state and the convolution's last inputs
    from token to token: what the framework's slots have to hold."""
    rt = {"heads": 2, "vdim": 3, "state": 5, "groups": 2, "conv": 3, "norm_groups": 2}
    cfg = O.make_config(layers=[{"type": "parallel", "mlp": None, "mixer": {
        "left": {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 0.5}, "right": rt}}], width=8)
    W = {k: v.double() for k, v in O.random_weights(cfg, 2).items()}
    p, eps = "l0.mix.right.", 1e-5
    h = torch.randn(9, 8, dtype=torch.float64)
    whole = O.state_space_mixer(h, W, p, rt, eps)
    inner, gn = 6, 10
    S = torch.zeros(2, 5, 3, dtype=torch.float64)
    tail = torch.zeros(2, inner + 2 * gn, dtype=torch.float64)        # the last taps - 1 inputs of the convolution
    for t in range(9):
        proj = W[p + "in"] @ h[t]
        z, xbc, dt = proj[:inner], proj[inner:2 * inner + 2 * gn], proj[2 * inner + 2 * gn:]
        window = torch.cat((tail, xbc.view(1, -1)))
        tail = window[1:]
        conv = (window * W[p + "conv"].T).sum(0) + W[p + "conv.b"]
        act = O.silu(conv)
        x, B, C = act[:inner].view(2, 3), act[inner:inner + gn].view(2, 5), act[inner + gn:].view(2, 5)
        dts = torch.log1p(torch.exp(dt + W[p + "dt_bias"]))
        y = torch.zeros(2, 3, dtype=torch.float64)
        for hh in range(2):
            S[hh] = torch.exp(-torch.exp(W[p + "A_log"][hh]) * dts[hh]) * S[hh] + dts[hh] * torch.outer(B[hh], x[hh])
            y[hh] = S[hh].T @ C[hh] + W[p + "D"][hh] * x[hh]
        gated = y.reshape(-1) * O.silu(z)
        normed = O.unit_rms(gated.view(2, 3), eps).reshape(-1) * W[p + "norm"]
        assert torch.allclose(W[p + "o"] @ normed, whole[t], atol=1e-10)


def test_layer_norms_the_result_not_the_input():
    cfg = O.make_config(layers=[O.attention_layer(mlp=O.dense_mlp(16))], width=16)
    W = {k: v.double() for k, v in O.random_weights(cfg, 3).items()}
    toks = [3, 1, 4, 1, 5]
    logits, streams = O.forward(W, cfg, toks)
    x = O.embed_tokens(W, toks)
    m, _ = O.sigmoid_attention(x, W, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    x = x + O.unit_rms(m, 1e-5) * (1 + W["l0.norm1"])
    x = x + O.unit_rms(O.gated_unit(x, W, "l0.mlp."), 1e-5) * (1 + W["l0.norm2"])
    assert torch.allclose(streams[0], x)
    assert torch.allclose(logits, (O.unit_rms(x, 1e-5) * (1 + W["final.norm"])) @ W["embed"].T * cfg["logit_scale"])


def test_block_and_slot_layout():
    from swiftllm_amd.worker.ratilorn_model import RatilornModel
    cfg = O.make_config()
    mcfg = RatilornModelConfig(cfg)

    class Probe(RatilornModel):       # (layout only: no device, no weights)
        def __init__(self):
            self.model_config = mcfg
            self.engine_config = type("E", (), {"block_size": 16})()
            self._layout_pool()

    probe = Probe()
    at = 0
    for layer, sl in zip(mcfg.layers, probe.pool_slices):
        mx = layer.attention
        assert sl.k_offset == at and sl.v_offset == at + mx.k_size * 16 and sl.k_offset % 8 == 0
        at = sl.v_offset + mx.v_size * 16
        at += -at % 8
    assert probe.block_elems == at
