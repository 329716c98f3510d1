"""RosilixModel — the data-plane worker for the Rosilix design.

The worker protocol, the token-level `step`, the block pool, the block managers, hipGraph replay of decode steps and
swapping are SteppedModel's (stepped_model.py); this file adds what is Rosilix's:

  * the layout of a block: for every differential attention layer the keys of both score maps and the shared values; for
    every latent attention layer with a compression of its own ONE row per token — the normed latent and the rotated shared
    key part as the key, the latent again (transposed) as the value. A layer that borrows reads the lender's slice;
  * the stack: scaled embedding, then per sublayer
        m = sublayer(h);  x += norm_post(m);  h = norm_pre_of_the_next(x)       one fused launch (kernels/rms_stream.py)
    with the stream x in fp32 and projections in the compute dtype (bfloat16 / float16, or true float32).
The design keeps no per-sequence state besides the cache.
"""
from typing import List

import torch

from swiftllm_amd.engine_config import EngineConfig
from swiftllm_amd.model_config import RosilixModelConfig

from .kernels.layernorm import embed_positions
from .kernels.linear import pack_weight, packable
from .kernels.rms_stream import gated_add_rmsnorm
from .kernels.window_attn import PoolSlice
from .layers.kekapel_layer import _project
from .layers.lorulix_layer import StepContext
from .layers.rosilix_layer import RosilixDiffAttention, RosilixFeedForward, RosilixLatentAttention
from .rosilix_weight import load_rosilix_weights
from .stepped_model import SteppedModel


class _Sublayer:
    """One residual update of the stack: x += norm_post(f(h)), h = norm_pre(x)."""
    __slots__ = ("op", "pre", "post", "ends_layer")


class RosilixModel(SteppedModel):
    CONFIG_CLASS = RosilixModelConfig

    @torch.inference_mode()
    def __init__(self, engine_config: EngineConfig):
        self.sublayers: List[_Sublayer] = []
        self.pool_slices = {}
        super().__init__(engine_config)
        # the design has no position table: a sequence is bounded by what its block-table row can map
        self.max_seq_len = min(self.model_config.max_position_embeddings,
                               engine_config.max_blocks_per_seq * engine_config.block_size)

    def _layout_pool(self):
        """Offsets (in elements) of every caching layer's keys and values inside a block."""
        cfg, bs = self.model_config, self.engine_config.block_size
        off = 0
        self.pool_slices = {}
        for i, layer in enumerate(cfg.layers):
            if layer.mixer.kv_from < 0:
                k_off = off
                off += layer.mixer.k_size * bs
                self.pool_slices[i] = PoolSlice(k_off, off)
                off += layer.mixer.v_size * bs
                off += -off % 8         # every slice starts on a 16-byte boundary
        for i, layer in enumerate(cfg.layers):
            if layer.mixer.kv_from >= 0:
                self.pool_slices[i] = self.pool_slices[layer.mixer.kv_from]
        self.block_elems = max(off, 8)

    def _build(self):
        cfg, ecfg = self.model_config, self.engine_config
        self.weight = load_rosilix_weights(cfg, self.dtype, ecfg.model_path, ecfg.use_dummy, self.device)
        skinny = bool(getattr(ecfg, "use_skinny_gemm", False)) and self.dtype != torch.float32
        if skinny and getattr(ecfg, "pack_decode_weights", False):
            for t in self.weight.projection_tensors():
                if packable(t):
                    pack_weight(t)
        self._skinny = skinny
        eps = cfg.norm_eps
        self.sublayers = []
        for i, (lcfg, lw) in enumerate(zip(cfg.layers, self.weight.layers)):
            s = _Sublayer()
            kind = RosilixDiffAttention if lcfg.type == "attention" else RosilixLatentAttention
            s.op = kind(lcfg, lw, eps, skinny, self.pool_slices[i], self.max_seq_len)
            s.pre, s.post, s.ends_layer = lw.norm1, lw.norm1b, lcfg.mlp is None
            self.sublayers.append(s)
            if lcfg.mlp is not None:
                f = _Sublayer()
                f.op = RosilixFeedForward(lcfg, lw, skinny)
                f.pre, f.post, f.ends_layer = lw.norm2, lw.norm2b, True
                self.sublayers.append(f)

    @torch.inference_mode()
    def _run_stack(self, dev: dict, use_pool: bool) -> torch.Tensor:
        """Embedding -> every sublayer -> the fp32 stream [T, width]."""
        cfg, w = self.model_config, self.weight
        eps = cfg.norm_eps
        ctx = StepContext(self.kv_pool if use_pool else None, self.gpu_block_manager.block_table if use_pool else None,
                          dev["tok_seq"], dev["tok_pos"], (dev["tile_row0"], dev["tile_cnt"]), None)
        x, _ = embed_positions(dev["input_ids"], dev["tok_pos"], w.embed, None, cfg.embedding_scale, keep_copy=False)
        tap = self.layer_tap
        subs = self.sublayers
        h = gated_add_rmsnorm(x, pre=subs[0].pre, eps=eps, out_dtype=self.dtype)
        for i, s in enumerate(subs):
            m = s.op.forward(h, ctx)
            nxt = subs[i + 1].pre if i + 1 < len(subs) else None
            h = gated_add_rmsnorm(x, m, s.post, pre=nxt, eps=eps)
            if tap is not None and s.ends_layer:
                tap.append(x.clone())
        return x

    @torch.inference_mode()
    def _logits(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """The model's norm of the asked-for rows and the vocabulary projection -> [rows, vocab] in the compute dtype."""
        h = gated_add_rmsnorm(x, pre=self.weight.final_norm, eps=self.model_config.norm_eps, out_dtype=self.dtype,
                              row_idx=rows)
        return _project(h, self.weight.head, self._skinny)
