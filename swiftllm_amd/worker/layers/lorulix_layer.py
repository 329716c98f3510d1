"""The sublayers of a Lorulix layer, each a function from its (normed, convolved) input to its raw result; the bookkeeping
around them (result gate, post-norm into the fp32 stream, the next input norm and convolution) is the model's fused step."""
import torch

from ..kernels.delta_rule import delta_rule_mixer
from ..kernels.moe import moe_experts_relu2, moe_route_scores, relu_squared
from ..kernels.window_attn import qknorm_full_and_store_kv, window_attention
from .kekapel_layer import _project
from swiftllm_amd import _hip


class StepContext:
    """What the sublayers of one step share: the block pool and table, the per-token plan arrays, the state slots."""
    __slots__ = ("pool", "block_table", "tok_seq", "tok_pos", "tiles", "state")

    def __init__(self, pool, block_table, tok_seq, tok_pos, tiles, state):
        self.pool, self.block_table, self.tok_seq, self.tok_pos, self.tiles, self.state = \
            pool, block_table, tok_seq, tok_pos, tiles, state


class LorulixAttention:
    """(q | k | v) projection -> whole-projection q/k norm + query temperature + KV store -> softmax attention over every
    earlier key with the learned distance bias -> output projection. A layer that borrows another layer's keys and values
    projects queries only and reads that layer's slice of the pool."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, pool_slice, max_positions: int):
        self.mixer, self.w, self.eps, self.skinny = layer_config.mixer, weight, eps, skinny
        self.pool_slice, self.max_positions = pool_slice, max_positions
        self.own_kv = self.mixer.kv_from < 0

    def forward(self, h: torch.Tensor, ctx: StepContext):
        mx = self.mixer
        qkv = _project(h, self.w.qkv, self.skinny)
        qknorm_full_and_store_kv(qkv, self.w.q_norm, self.w.k_norm, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq,
                                 ctx.tok_pos, mx, self.eps, self.own_kv)
        if ctx.pool is None:    # memory profiling: the attention's output buffer without its reads
            attn = torch.zeros((h.shape[0], mx.num_q_heads * mx.value_dim), dtype=h.dtype, device=h.device)
        else:
            attn = window_attention(qkv, None, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos, mx,
                                    ctx.tiles, self.max_positions, rel=self.w.rel)
        return _project(attn, self.w.o, self.skinny), None, None


class LorulixDelta:
    """One fused projection -> convolutions, unit norms, the recurrence on the sequence's state, gated output norm ->
    output projection."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, tail_off: int, state_off: int):
        self.mixer, self.w, self.eps, self.skinny = layer_config.mixer, weight, eps, skinny
        self.tail_off, self.state_off = tail_off, state_off

    def forward(self, h: torch.Tensor, ctx: StepContext):
        proj = _project(h, self.w.proj, self.skinny)
        y = delta_rule_mixer(proj, self.w.conv, self.w.a_log, self.w.dt_bias, self.w.out_norm, ctx.state, self.tail_off,
                             self.state_off, self.mixer, self.eps)
        return _project(y, self.w.o, self.skinny), None, None


class LorulixFeedForward:
    """dense: clamped gated unit. moe: router -> squared-ReLU experts (+ the shared expert and its per-token gate, which
    the stream step adds in)."""

    def __init__(self, layer_config, weight, skinny: bool):
        self.mlp, self.w, self.skinny = layer_config.mlp, weight, skinny

    def forward(self, h: torch.Tensor, ctx: StepContext):
        mlp, w = self.mlp, self.w
        if mlp.kind == "dense":
            gu = _project(h, w.gate_up, self.skinny)
            y = torch.empty((h.shape[0], mlp.ffn_inter_dim), dtype=h.dtype, device=h.device)
            _hip.call("swl_glu_clamp", _hip.ptr(y), _hip.ptr(gu), h.shape[0], mlp.ffn_inter_dim, float(mlp.limit), 0,
                      _hip.dtype_code3(h.dtype), _hip.stream())
            return _project(y, w.down, self.skinny), None, None
        idx, wts = moe_route_scores(h, w.router, mlp.top_k, mlp.router_scale)
        out = moe_experts_relu2(h, idx, wts, w.up, w.down)
        if w.shared_up is None:
            return out, None, None
        fs = mlp.shared_ffn_inter_dim
        z = _project(h, w.shared_up, self.skinny)           # [T, fs + 1]: the shared expert's up rows, then its gate logit
        shared = _project(relu_squared(z, fs), w.shared_down, self.skinny)
        return out, shared, z[:, fs:fs + 1]
