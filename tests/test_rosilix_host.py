"""Host-side pieces of the Rosilix worker (no GPU): the configuration reader, the registry, the block layout, and the plain
implementation's own mechanisms against closed forms."""
import json
import math

import pytest
import torch

import rosilix_oracle as O
from swiftllm_amd import registry
from swiftllm_amd.model_config import RosilixModelConfig, RotaryConfig


def test_config_reads_every_layer():
    layers = [O.latent_mixer(heads=5, dim=24, rot_dim=8, vdim=40, kv_rank=48, base=5000.0),
              O.diff_mixer(heads=6, kv_heads=2, dim=16, vdim=24, chunk=20, rot_dims=12, diff=0.4),
              O.latent_mixer(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=48, base=5000.0, kv_from=0),
              O.diff_mixer(heads=3, kv_heads=3, dim=8, vdim=8, chunk=None, rot_dims=8)]
    cfg = RosilixModelConfig(O.make_config(layers, width=48, vocab=70, ff=56, embed_scale=3.0, no_mlp=(2,)))
    assert (cfg.hidden_size, cfg.vocab_size, cfg.embedding_scale, cfg.norm_eps) == (48, 70, 3.0, 1e-5)
    a, b, c, d = (l.mixer for l in cfg.layers)
    assert (a.q_size, a.dkv_size, a.k_size, a.v_size, a.o_size, a.kv_from) == (160, 56, 56, 48, 200, -1)
    assert (b.q_size, b.k_size, b.v_size, b.o_size, b.chunk, b.rot.dims, b.diff) == (192, 64, 48, 144, 20, 12, 0.4)
    assert (c.kv_from, c.q_size) == (0, 32) and d.chunk == 0 and d.num_kv_heads == 3
    assert cfg.layers[2].mlp is None and cfg.layers[0].mlp.ffn_inter_dim == 56
    # the borrowing layer caches nothing: two latent rows (key + transposed value copy) and the two differential layers
    assert cfg.kv_elems_per_token() == (56 + 48) + (64 + 48) + (48 + 24)
    assert cfg.max_position_embeddings == RosilixModelConfig.DEFAULT_MAX_POSITIONS
    raw = O.make_config(layers)
    raw["max_positions"] = 300
    assert RosilixModelConfig(raw).max_position_embeddings == 300


def test_config_refuses_bad_borrowing_and_rotations():
    with pytest.raises(ValueError):
        RosilixModelConfig(O.make_config([O.latent_mixer(kv_from=1), O.latent_mixer()]))
    with pytest.raises(ValueError):
        RosilixModelConfig(O.make_config([O.diff_mixer(), O.latent_mixer(kv_from=0)]))
    with pytest.raises(ValueError):
        RosilixModelConfig(O.make_config([O.latent_mixer(), O.latent_mixer(kv_from=0), O.latent_mixer(kv_from=1)]))
    with pytest.raises(ValueError):
        RosilixModelConfig(O.make_config([O.latent_mixer(kv_rank=32), O.latent_mixer(kv_rank=16, kv_from=0)]))
    with pytest.raises(ValueError):
        RosilixModelConfig(O.make_config([O.diff_mixer(dim=16, rot_dims=18)]))
    bad = O.make_config([O.diff_mixer()])
    bad["layers"][0]["mlp"] = {"kind": "moe", "ff": 8}
    with pytest.raises(ValueError):
        RosilixModelConfig(bad)


def test_registry_knows_the_design(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(O.make_config([O.diff_mixer()])))
    assert type(registry.load_model_config(str(tmp_path))).__name__ == "RosilixModelConfig"
    assert registry.model_class(str(tmp_path)).__name__ == "RosilixModel"


def test_rotary_frequencies():
    rot = RotaryConfig({"dims": 8, "base": 100.0}, 16)
    assert rot.frequencies() == pytest.approx([1.0, 100 ** -0.25, 0.1, 100 ** -0.75])
    assert RotaryConfig(None, 16).dims == 0


def test_rotation_keeps_lengths_and_relative_angles():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(9, 3, 12, generator=g, dtype=torch.float64)
    pos = torch.arange(9)
    y = O.rotate_pairs(x, pos, 8, 50.0)
    assert torch.allclose(y[..., 8:], x[..., 8:]) and torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    assert torch.allclose(y[0], x[0])                                   # position 0 turns nothing
    # a dot product of two rotated vectors depends on the distance only
    q, k = x[0, 0].expand(9, 12).unsqueeze(1), x[0, 1].expand(9, 12).unsqueeze(1)
    qr, kr = O.rotate_pairs(q, pos, 8, 50.0), O.rotate_pairs(k, pos, 8, 50.0)
    assert math.isclose(float(qr[5, 0] @ kr[2, 0]), float(qr[8, 0] @ kr[5, 0]), rel_tol=1e-9)


def test_masks_and_sink():
    m = O.chunk_mask(10, 4)
    assert m[5].tolist() == [False] * 4 + [True, True] + [False] * 4 and m[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert m[3].tolist() == [True] * 4 + [False] * 6
    s = torch.zeros(1, 3, dtype=torch.float64)
    p = O.softmax_rows(s, torch.ones(1, 3, dtype=torch.bool), sink=0.0)
    assert torch.allclose(p, torch.full((1, 3), 0.25, dtype=torch.float64))      # the sink counts once and has no value
    p = O.softmax_rows(s, torch.ones(1, 3, dtype=torch.bool), sink=500.0)        # a huge sink does not overflow
    assert float(p.sum()) < 1e-200 or float(p.sum()) == 0.0


def test_block_layout_of_the_worker():
    """Slices of a block: every caching layer's keys then values, 16-byte aligned; a borrowing layer shares the lender's."""
    from swiftllm_amd.engine_config import EngineConfig
    from swiftllm_amd.worker.rosilix_model import RosilixModel
    layers = [O.latent_mixer(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=13), O.diff_mixer(heads=2, kv_heads=1, dim=6, vdim=10, rot_dims=4),
              O.latent_mixer(heads=3, dim=4, rot_dim=4, vdim=8, kv_rank=13, kv_from=0)]
    cfg = RosilixModelConfig(O.make_config(layers))
    model = RosilixModel.__new__(RosilixModel)
    model.model_config = cfg
    model.engine_config = EngineConfig(model_path="", use_dummy=True, block_size=16, gpu_mem_utilization=0.9,
                                       num_cpu_blocks=0, max_seqs_in_block_table=2, max_blocks_per_seq=4, max_batch_size=2,
                                       max_tokens_in_batch=64)
    model._layout_pool()
    s0, s1, s2 = (model.pool_slices[i] for i in range(3))
    assert (s0.k_offset, s0.v_offset) == (0, 17 * 16) and s2 is s0
    assert s1.k_offset == (17 + 13) * 16 and s1.v_offset == s1.k_offset + 12 * 16
    assert model.block_elems == s1.v_offset + 10 * 16 and model.block_elems % 8 == 0
