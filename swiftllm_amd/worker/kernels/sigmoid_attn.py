"""Attention over the paged pool with sigmoid weights, a logarithmic distance penalty and post-sigmoid head mixing.
csrc/sigmoid_attn.hip."""
import torch

from swiftllm_amd import _hip

from .window_attn import PoolSlice, _split_scratch, choose_key_splits


def tiles_supported(mixer, dtype: torch.dtype) -> bool:
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    return bool(_hip.load().swl_sigmoid_attn_tiles_supported(mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
                                                             mixer.value_dim, _hip.dtype_code(dtype)))


def sigmoid_attention(q: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice, block_table: torch.Tensor,
                      tok_seq: torch.Tensor, tok_pos: torch.Tensor, mixer, talk: torch.Tensor = None, r1: torch.Tensor = None,
                      r2: torch.Tensor = None, pb: torch.Tensor = None, tiles=None, max_positions: int = 1 << 20) -> torch.Tensor:
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
    wide_ok = q.stride(0) % 4 == 0 and q.data_ptr() % 8 == 0 and kp % 8 == 0 and vp % 8 == 0 and pool.shape[1] % 4 == 0
    if tiles is not None and wide_ok and tiles_supported(mixer, q.dtype):
        row0, cnt = tiles
        splits = choose_key_splits(row0.shape[0], mixer, max_positions)
        scratch = _split_scratch(q.device, splits * n * H * mixer.value_dim) if splits > 1 else None
        _hip.call("swl_sigmoid_attn_tiles", _hip.ptr(out), _hip.ptr(q), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
                  _hip.ptr(tok_pos), _hip.ptr(row0), _hip.ptr(cnt), _hip.ptr(talk), _hip.ptr(r1), _hip.ptr(r2), _hip.ptr(pb),
                  row0.shape[0], H, mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, q.stride(0), mixer.window,
                  float(mixer.scale), block_table.shape[1], pool.shape[1], splits, _hip.ptr(scratch), n,
                  _hip.dtype_code(q.dtype), _hip.stream())
        return out
    _hip.call("swl_sigmoid_attn", _hip.ptr(out), _hip.ptr(q), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
              _hip.ptr(tok_pos), _hip.ptr(talk), _hip.ptr(r1), _hip.ptr(r2), _hip.ptr(pb), n, H, mixer.num_kv_heads,
              mixer.head_dim, mixer.value_dim, q.stride(0), mixer.window, float(mixer.scale), block_table.shape[1],
              pool.shape[1], _hip.dtype_code3(q.dtype), _hip.stream())
    return out
