"""RatilornModel — the data-plane worker for the Ratilorn design.

The worker protocol, the token-level `step`, the block pool, the block managers, hipGraph replay of decode steps and
swapping are SteppedModel's (stepped_model.py); this file adds what is Ratilorn's:

  * the layout of a block: the keys and values of every layer's attention (a sigmoid attention layer's own, a parallel
    layer's left mixer's);
  * the layout of a state slot (StateSlotManager): per parallel layer the carried inputs of its recurrence's convolution and
    the fp32 state [heads, state, vdim];
  * the stack: embedding with learned positions, then per sublayer
        a (, b) = sublayer(h)             h is the stream itself in the compute dtype: no norm in front of a sublayer
        x += norm(c (a' + b'));  h = x    one fused launch between two sublayers (kernels/rms_stream.py: post_norm_add)
    where a parallel layer's two results are normed separately and averaged, a mixture's routed and shared results are
    summed as they are. The stream x is fp32, projections run in the compute dtype (bfloat16 / float16, or true float32).
The values of the first value-blending attention layer of a step stay alive until the last such layer has read them.
"""
from typing import List

import torch

from swiftllm_amd.engine_config import EngineConfig
from swiftllm_amd.model_config import RatilornModelConfig

from .kernels.layernorm import embed_positions
from .kernels.linear import pack_weight, packable
from .kernels.rms_stream import StateRef, gated_add_rmsnorm, post_norm_add
from .kernels.window_attn import PoolSlice
from .layers.kekapel_layer import _project
from .layers.lorulix_layer import StepContext
from .layers.ratilorn_layer import RatilornFeedForward, RatilornParallel, RatilornSigmoidAttention, ValueShare
from .ratilorn_weight import load_ratilorn_weights
from .state_slots import StateSlotManager
from .stepped_model import SteppedModel


class _Sublayer:
    """One residual update of the stack: x += norm_post(coef * (a' + b')) with (a, b) = op(x)."""
    __slots__ = ("op", "post", "a_norm", "b_norm", "coef", "ends_layer")


class RatilornModel(SteppedModel):
    CONFIG_CLASS = RatilornModelConfig

    @torch.inference_mode()
    def __init__(self, engine_config: EngineConfig):
        self.sublayers: List[_Sublayer] = []
        self.pool_slices: List[PoolSlice] = []
        super().__init__(engine_config)

    def _layout_pool(self):
        """Offsets (in elements) of every layer's keys and values inside a block."""
        cfg, bs = self.model_config, self.engine_config.block_size
        off = 0
        self.pool_slices = []
        for layer in cfg.layers:
            mx = layer.attention
            k_off = off
            off += mx.k_size * bs
            self.pool_slices.append(PoolSlice(k_off, off))
            off += mx.v_size * bs
            off += -off % 8         # every slice starts on a 16-byte boundary
        self.block_elems = max(off, 8)

    def _build(self):
        cfg, ecfg = self.model_config, self.engine_config
        self.weight = load_ratilorn_weights(cfg, self.dtype, ecfg.model_path, ecfg.use_dummy, self.device)
        skinny = bool(getattr(ecfg, "use_skinny_gemm", False)) and self.dtype != torch.float32
        if skinny and getattr(ecfg, "pack_decode_weights", False):
            for t in self.weight.projection_tensors():
                if packable(t):
                    pack_weight(t)
        self._skinny = skinny
        eps = cfg.norm_eps
        # one slot per sequence that runs: as many as a batch holds
        self.state = StateSlotManager(ecfg.max_batch_size, self.device) if cfg.has_state else None
        self.sublayers = []
        for i, (lcfg, lw) in enumerate(zip(cfg.layers, self.weight.layers)):
            s = _Sublayer()
            if lcfg.type == "attention":
                s.op = RatilornSigmoidAttention(lcfg, lw, eps, skinny, self.pool_slices[i], cfg.max_position_embeddings)
                s.a_norm = s.b_norm = None
                s.coef = 1.0
            else:
                rt = lcfg.mixer.right
                tail_off = self.state.add_region(2 * (rt.conv_taps - 1) * rt.conv_channels)
                state_off = self.state.add_region(rt.state_elems)
                s.op = RatilornParallel(lcfg, lw, eps, skinny, self.pool_slices[i], cfg.max_position_embeddings, tail_off,
                                        state_off)
                s.a_norm, s.b_norm, s.coef = lw.left_out, lw.right_out, 0.5
            s.post, s.ends_layer = lw.norm1, lcfg.mlp is None
            self.sublayers.append(s)
            if lcfg.mlp is not None:
                f = _Sublayer()
                f.op = RatilornFeedForward(lcfg, lw, skinny)
                f.post, f.a_norm, f.b_norm, f.coef, f.ends_layer = lw.norm2, None, None, 1.0, True
                self.sublayers.append(f)
        if self.state is not None:
            self.state.allocate()

    @torch.inference_mode()
    def _run_stack(self, dev: dict, use_pool: bool) -> torch.Tensor:
        """Embedding -> every sublayer -> the fp32 stream [T, width]."""
        cfg, w = self.model_config, self.weight
        eps = cfg.norm_eps
        st = None
        if self.state is not None:
            st = StateRef(self.state.pool, dev["tok_pos"], dev["tok_start"], dev["tok_state"], dev["tok_seq"],
                          dev["seq_row0"], dev["seq_cnt"])
        ctx = StepContext(self.kv_pool if use_pool else None, self.gpu_block_manager.block_table if use_pool else None,
                          dev["tok_seq"], dev["tok_pos"], (dev["tile_row0"], dev["tile_cnt"]), st)
        x, _ = embed_positions(dev["input_ids"], dev["tok_pos"], w.embed, w.pos, 1.0, keep_copy=False)
        h = x if self.dtype == torch.float32 else x.to(self.dtype)
        share = ValueShare()
        tap = self.layer_tap
        subs = self.sublayers
        for i, s in enumerate(subs):
            a, b = s.op.forward(h, ctx, share)
            h = post_norm_add(x, a, s.post, b, s.a_norm, s.b_norm if b is not None else None, s.coef, eps=eps,
                              want_out=i + 1 < len(subs))
            if tap is not None and s.ends_layer:
                tap.append(x.clone())
        return x

    @torch.inference_mode()
    def _logits(self, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        """The model's norm (with the output scale on its weight) of the asked-for rows and the product with the embedding
        table -> [rows, vocab] in the compute dtype."""
        h = gated_add_rmsnorm(x, pre=self.weight.final_norm, eps=self.model_config.norm_eps, out_dtype=self.dtype,
                              row_idx=rows)
        return _project(h, self.weight.head, self._skinny)
