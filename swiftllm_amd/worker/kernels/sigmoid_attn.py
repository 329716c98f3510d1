"""Attention over the paged pool with sigmoid weights, a logarithmic distance penalty and post-sigmoid head mixing.
csrc/sigmoid_attn.hip."""
import torch

from swiftllm_amd import _hip

from .window_attn import PoolSlice


def sigmoid_attention(q: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice, block_table: torch.Tensor,
                      tok_seq: torch.Tensor, tok_pos: torch.Tensor, mixer, talk: torch.Tensor = None, r1: torch.Tensor = None,
                      r2: torch.Tensor = None, pb: torch.Tensor = None, tiles=None) -> torch.Tensor:
    """-> [T, heads * vdim] in q's dtype. q: rows whose first heads * dim columns are the (already normed) queries; keys and
    values come from the pool, which already holds this step's tokens. Per visible key j <= i:
        a[g] = sigmoid(scale q_g . k - r1[g] ln(1 + r2[g] (i - j)) + pb[g]),   a'[h] = sum_g talk[h][g] a[g]
    and out[h] = sum_j a'[h] v_j (nothing is normalised over the keys). talk [H, H], r1 / r2 / pb [H]: fp32, optional.
    `tiles` = (tile_row0, tile_cnt): given, and the shape served, the matrix-core kernel runs."""
    _hip.require_gpu_tensor(q, "q")
    H = mixer.num_q_heads
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= H * mixer.head_dim
    assert pool.is_contiguous() and pool.dtype == q.dtype and tok_pos.dtype == torch.int32 and tok_seq.dtype == torch.int32
    for t, shape in ((talk, (H, H)), (r1, (H,)), (r2, (H,)), (pb, (H,))):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == shape)
    n = q.shape[0]
    out = torch.empty((n, H * mixer.value_dim), dtype=q.dtype, device=q.device)
    esize = pool.element_size()
    kp = pool.data_ptr() + pool_slice.k_offset * esize
    vp = pool.data_ptr() + pool_slice.v_offset * esize
    _hip.call("swl_sigmoid_attn", _hip.ptr(out), _hip.ptr(q), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
              _hip.ptr(tok_pos), _hip.ptr(talk), _hip.ptr(r1), _hip.ptr(r2), _hip.ptr(pb), n, H, mixer.num_kv_heads,
              mixer.head_dim, mixer.value_dim, q.stride(0), mixer.window, float(mixer.scale), block_table.shape[1],
              pool.shape[1], _hip.dtype_code3(q.dtype), _hip.stream())
    return out
