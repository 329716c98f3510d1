"""The sublayers of a Rosilix layer, each a function from its normed input to its raw result; the post-norm into the fp32
stream and the next input norm are the model's fused step (kernels/rms_stream.py)."""
import torch

from ..kernels.moe import relu_squared
from ..kernels.rope_kv import diff_head_combine, head_gate_, latent_rope_and_store_kv, rope_and_store_kv
from ..kernels.window_attn import MASK_CHUNK, MASK_WINDOW, AttentionSpec, masked_attention
from .kekapel_layer import _project
from .lorulix_layer import StepContext


class RosilixDiffAttention:
    """(q | k | v | gate) projection -> rotary + KV store -> chunked attention of both score maps over the shared values
    (fp32 results) -> a1 - lambda a2, unit RMS per head, (1 - diff), head gate -> output projection."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, pool_slice, max_positions: int):
        mx = self.mixer = layer_config.mixer
        self.w, self.eps, self.skinny, self.pool_slice, self.max_positions = weight, eps, skinny, pool_slice, max_positions
        # the two maps as attention heads: map-major queries and keys, key head g over value head g mod G
        self.spec = AttentionSpec(2 * mx.num_q_heads, 2 * mx.num_kv_heads, mx.head_dim, mx.value_dim, mx.scale,
                                  window=mx.chunk, mask_kind=MASK_CHUNK, num_v_heads=mx.num_kv_heads, out_f32=True)

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        mx, w = self.mixer, self.w
        proj = _project(h, w.proj, self.skinny)
        rope_and_store_kv(proj, w.freq, mx.rot.dims, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos,
                          2 * mx.num_q_heads, 2 * mx.num_kv_heads, mx.num_kv_heads, mx.head_dim, mx.value_dim)
        if ctx.pool is None:    # memory profiling: the attention's output buffer without its reads
            maps = torch.zeros((h.shape[0], 2 * mx.o_size), dtype=torch.float32, device=h.device)
        else:
            maps = masked_attention(proj, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos, self.spec,
                                    ctx.tiles, self.max_positions)
        gate = proj[:, w.gate_col:w.gate_col + mx.num_q_heads]
        y = diff_head_combine(maps, gate, w.lam, 1.0 - mx.diff, self.eps, mx.num_q_heads, mx.value_dim, h.dtype)
        return _project(y, w.o, self.skinny)


class RosilixLatentAttention:
    """(q | compressed kv | gate) projection -> rotary, latent norm and cache store -> queries folded through the key
    up-projection -> attention of all heads over the one cached row per token (key: latent | rotated part, value: latent)
    with the heads' sinks -> value up-projection per head -> head gate -> output projection. A layer that reads another
    layer's cache projects queries and gates only."""

    def __init__(self, layer_config, weight, eps: float, skinny: bool, pool_slice, max_positions: int):
        mx = self.mixer = layer_config.mixer
        self.w, self.eps, self.skinny, self.pool_slice, self.max_positions = weight, eps, skinny, pool_slice, max_positions
        self.spec = AttentionSpec(mx.num_q_heads, 1, mx.kv_rank + mx.rot_dim, mx.kv_rank, mx.scale, window=0,
                                  mask_kind=MASK_WINDOW, sink=weight.sink)

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        mx, w = self.mixer, self.w
        n, H, d, dr, r, e = h.shape[0], mx.num_q_heads, mx.head_dim, mx.rot_dim, mx.kv_rank, mx.value_dim
        proj = _project(h, w.proj, self.skinny)
        qa = torch.empty((n, H * (r + dr)), dtype=h.dtype, device=h.device)
        latent_rope_and_store_kv(proj, qa, w.freq, w.c_norm, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq,
                                 ctx.tok_pos, mx, w.dkv_col, self.eps)
        # q_abs[t, h, :] = W_uk,h^T q_unrotated[t, h, :]  -> the first kv_rank columns of every head of qa
        qn = proj[:, :H * (d + dr)].view(n, H, d + dr)[:, :, :d].transpose(0, 1)        # [H, T, d]
        torch.bmm(qn, w.uk, out=qa.view(n, H, r + dr)[:, :, :r].transpose(0, 1))      # (a strided batched product: no copy)
        if ctx.pool is None:
            att = torch.zeros((n, H * r), dtype=h.dtype, device=h.device)
        else:
            att = masked_attention(qa, ctx.pool, self.pool_slice, ctx.block_table, ctx.tok_seq, ctx.tok_pos, self.spec,
                                   ctx.tiles, self.max_positions)
        y = torch.empty((n, H * e), dtype=h.dtype, device=h.device)
        torch.bmm(att.view(n, H, r).transpose(0, 1), w.uv_t, out=y.view(n, H, e).transpose(0, 1))
        head_gate_(y, proj[:, w.gate_col:w.gate_col + H], H, e)
        return _project(y, w.o, self.skinny)


class RosilixFeedForward:
    """down(relu(up h)^2)."""

    def __init__(self, layer_config, weight, skinny: bool):
        self.mlp, self.w, self.skinny = layer_config.mlp, weight, skinny

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        z = _project(h, self.w.up, self.skinny)
        return _project(relu_squared(z, self.mlp.ffn_inter_dim), self.w.down, self.skinny)
