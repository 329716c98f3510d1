"""The sublayers of a Ratilorn layer, each a function from the stream (in the compute dtype) to its raw result; the norm of
the result and its addition to the fp32 stream are the model's fused step (kernels/rms_stream.py: post_norm_add)."""
import torch

from ..kernels.moe import ACT_SILU, gated_unit, moe_experts, moe_route_grouped
from ..kernels.sigmoid_attn import sigmoid_attention
from ..kernels.ssd import state_space_mixer
from ..kernels.window_attn import MASK_WINDOW, AttentionSpec, masked_attention, qkv_bias_norm_store
from .kekapel_layer import _project
from .lorulix_layer import StepContext


class ValueShare:
    """The values of the first value-blending layer of a step ([T, kv_heads * vdim], a view into that layer's projection
    rows), which the later ones blend into their own."""
    __slots__ = ("first",)

    def __init__(self):
        self.first = None


class RatilornSigmoidAttention:
    """(q | k | v) projection -> biases, unit q/k per head, value blend, KV store -> sigmoid attention over every earlier key
    with the logarithmic distance penalty and post-sigmoid head mixing -> output projection."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, pool_slice, max_positions: int):
        self.mixer, self.w, self.eps, self.skinny, self.pool_slice = layer_config.mixer, weight, eps, skinny, pool_slice
        self.max_positions = max_positions

    def forward(self, h: torch.Tensor, ctx: StepContext, share: ValueShare):
        mx, w = self.mixer, self.w
        qkv = _project(h, w.qkv, self.skinny)
        other = share.first if mx.v_mix else None
        qkv_bias_norm_store(qkv, w.q_b, w.k_b, w.v_b, None, None, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq,
                            ctx.tok_pos, mx, self.eps, other, w.v_mix)
        if mx.v_mix and share.first is None:
            share.first = qkv[:, mx.q_size + mx.k_size:mx.q_size + mx.k_size + mx.v_size]
        if ctx.pool is None:    # memory profiling: the attention's output buffer without its reads
            attn = torch.zeros((h.shape[0], mx.o_size), dtype=h.dtype, device=h.device)
        else:
            attn = sigmoid_attention(qkv, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos, mx, w.talk,
                                     w.r1, w.r2, w.pb, ctx.tiles, self.max_positions)
        return _project(attn, w.o, self.skinny), None


class RatilornParallel:
    """ONE projection for both mixers (left q | k | v, then the recurrence's z | x | B | C | dt). Left: biases, weighted q/k
    norm, KV store, softmax attention over every earlier key, output projection. Right: convolution, the recurrence on the
    sequence's state, gated grouped norm, output projection. The two results leave separately: the stream step norms each
    and takes half their sum."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, pool_slice, max_positions: int, tail_off: int,
                 state_off: int):
        self.left, self.right = layer_config.mixer.left, layer_config.mixer.right
        self.w, self.eps, self.skinny, self.pool_slice, self.max_positions = weight, eps, skinny, pool_slice, max_positions
        self.tail_off, self.state_off = tail_off, state_off
        lf = self.left
        self.spec = AttentionSpec(lf.num_q_heads, lf.num_kv_heads, lf.head_dim, lf.value_dim, lf.scale, window=0,
                                  mask_kind=MASK_WINDOW)

    def forward(self, h: torch.Tensor, ctx: StepContext, share: ValueShare):
        lf, rt, w = self.left, self.right, self.w
        proj = _project(h, w.proj, self.skinny)
        qkv_bias_norm_store(proj, w.q_b, w.k_b, w.v_b, w.q_norm, w.k_norm, ctx.pool, self.pool_slice, ctx.block_table,
                            ctx.tok_seq, ctx.tok_pos, lf, self.eps)
        if ctx.pool is None:
            attn = torch.zeros((h.shape[0], lf.o_size), dtype=h.dtype, device=h.device)
        else:
            attn = masked_attention(proj, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos, self.spec,
                                    ctx.tiles, self.max_positions)
        left = _project(attn, w.left_o, self.skinny)
        y = state_space_mixer(proj[:, w.right_col:], w.conv, w.conv_b, w.a_log, w.dt_bias, w.d_skip, w.right_norm, ctx.state,
                              self.tail_off, self.state_off, rt, self.eps)
        return left, _project(y, w.right_o, self.skinny)


class RatilornFeedForward:
    """dense: down(silu(gate h) * up h). moe: sigmoid router with group-limited choice -> the same unit per chosen expert,
    weighted; the shared expert's result leaves separately (the stream step adds the two)."""

    def __init__(self, layer_config, weight, skinny: bool):
        self.mlp, self.w, self.skinny = layer_config.mlp, weight, skinny

    def _unit(self, h, gate_up, down, ff):
        return _project(gated_unit(_project(h, gate_up, self.skinny), ff, ACT_SILU), down, self.skinny)

    def forward(self, h: torch.Tensor, ctx: StepContext, share: ValueShare):
        mlp, w = self.mlp, self.w
        if mlp.kind == "dense":
            return self._unit(h, w.gate_up, w.down, mlp.ffn_inter_dim), None
        idx, wts = moe_route_grouped(h, w.router, w.correction, mlp.top_k, mlp.group_count, mlp.group_keep)
        out = moe_experts(h, idx, wts, w.gate_up, w.down, 0.0, ACT_SILU)
        if w.shared_gate_up is None:
            return out, None
        return out, self._unit(h, w.shared_gate_up, w.shared_down, mlp.shared_ffn_inter_dim)
