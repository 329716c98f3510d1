"""Rotary positions on interleaved pairs fused with the paged KV store (plain heads, and the compressed rows of latent
attention), and the per-head steps after the softmax: the combination of two score maps, the head gate. csrc/rope_kv.hip."""
import torch

from swiftllm_amd import _hip

from .window_attn import PoolSlice


def rotary_frequencies(rot, device) -> torch.Tensor:
    """The float64 frequency table of a RotaryConfig on the device (None without rotation)."""
    if rot.dims == 0:
        return None
    return torch.tensor(rot.frequencies(), dtype=torch.float64, device=device)


def _pool_ptrs(pool, pool_slice: PoolSlice):
    if pool is None:
        return 0, 0, 0
    assert pool.is_contiguous()
    esize = pool.element_size()
    return pool.data_ptr() + pool_slice.k_offset * esize, pool.data_ptr() + pool_slice.v_offset * esize, pool.shape[1]


def rope_and_store_kv(qkv: torch.Tensor, freq: torch.Tensor, rot_dims: int, pool: torch.Tensor, pool_slice: PoolSlice,
                      block_table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, num_q_heads: int,
                      num_k_heads: int, num_v_heads: int, dim: int, vdim: int):
    """Rows [q | k | v (| anything)] of one fused projection: the query heads rotated in place, the key heads rotated into
    the pool, the value heads copied into the pool. pool None (memory profiling): queries only."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert qkv.dim() == 2 and qkv.stride(1) == 1
    assert qkv.shape[1] >= (num_q_heads + num_k_heads) * dim + num_v_heads * vdim
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == qkv.shape[0]
    assert freq is None or (freq.dtype == torch.float64 and freq.numel() == rot_dims // 2)
    kp, vp, stride = _pool_ptrs(pool, pool_slice)
    if pool is not None:
        assert pool.dtype == qkv.dtype and block_table.is_contiguous() and tok_seq.dtype == torch.int32
    _hip.call("swl_rope_store_kv", _hip.ptr(qkv), _hip.ptr(freq), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
              _hip.ptr(tok_pos), qkv.shape[0], num_q_heads, num_k_heads, num_v_heads, dim, vdim,
              rot_dims if freq is not None else 0, qkv.stride(0), block_table.shape[1] if block_table is not None else 0,
              stride, _hip.dtype_code3(qkv.dtype), _hip.stream())


def latent_rope_and_store_kv(proj: torch.Tensor, qa: torch.Tensor, freq: torch.Tensor, c_norm: torch.Tensor,
                             pool: torch.Tensor, pool_slice: PoolSlice, block_table: torch.Tensor, tok_seq: torch.Tensor,
                             tok_pos: torch.Tensor, mixer, dkv_col: int, eps: float):
    """proj rows: the query heads [dim | rot_dim] and, at column dkv_col (< 0: the layer reads another layer's cache), the
    compressed row [kv_rank | rot_dim]. Writes the rotated query parts into qa [T, heads, kv_rank + rot_dim] (columns from
    kv_rank on) and the normed latent + rotated shared key part into the pool."""
    _hip.require_gpu_tensor(proj, "proj")
    n = proj.shape[0]
    assert proj.dim() == 2 and proj.stride(1) == 1 and qa.is_contiguous() and qa.dtype == proj.dtype
    assert qa.shape == (n, mixer.num_q_heads * (mixer.kv_rank + mixer.rot_dim))
    assert freq.dtype == torch.float64 and freq.numel() == mixer.rot_dim // 2
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == n
    kp, vp, stride = _pool_ptrs(pool if dkv_col >= 0 else None, pool_slice)
    if kp:
        assert pool.dtype == proj.dtype and c_norm.dtype == torch.float32 and c_norm.numel() == mixer.kv_rank
    _hip.call("swl_latent_rope_store_kv", _hip.ptr(proj), _hip.ptr(qa), _hip.ptr(freq), _hip.ptr(c_norm), kp, vp,
              _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos), n, mixer.num_q_heads, mixer.head_dim,
              mixer.rot_dim, mixer.kv_rank, proj.stride(0), dkv_col if kp else -1, qa.stride(0),
              block_table.shape[1] if block_table is not None else 0, stride, float(eps), _hip.dtype_code3(proj.dtype),
              _hip.stream())


def diff_head_combine(maps: torch.Tensor, gate: torch.Tensor, lam: float, mult: float, eps: float, num_heads: int,
                      vdim: int, out_dtype: torch.dtype) -> torch.Tensor:
    """maps fp32 [T, 2 * heads * vdim] (map-major) -> [T, heads * vdim]: unit_rms(a1 - lam * a2) * mult * sigmoid(gate[t, h]).
    gate: [T, heads] logits, possibly a column slice of a wider matrix."""
    _hip.require_gpu_tensor(maps, "maps")
    n = maps.shape[0]
    assert maps.dtype == torch.float32 and maps.is_contiguous() and maps.shape[1] == 2 * num_heads * vdim
    assert gate is None or (gate.shape == (n, num_heads) and gate.stride(1) == 1 and gate.dtype == out_dtype)
    out = torch.empty((n, num_heads * vdim), dtype=out_dtype, device=maps.device)
    _hip.call("swl_diff_head_combine", _hip.ptr(out), _hip.ptr(maps), _hip.ptr(gate), gate.stride(0) if gate is not None else 0,
              float(lam), float(mult), float(eps), n, num_heads, vdim, _hip.dtype_code3(out_dtype), _hip.stream())
    return out


def head_gate_(y: torch.Tensor, gate: torch.Tensor, num_heads: int, vdim: int) -> torch.Tensor:
    """In place: y[t, h, :] *= sigmoid(gate[t, h])."""
    _hip.require_gpu_tensor(y, "y")
    n = y.shape[0]
    assert y.is_contiguous() and y.shape[1] == num_heads * vdim
    assert gate.shape == (n, num_heads) and gate.stride(1) == 1 and gate.dtype == y.dtype
    _hip.call("swl_head_gate", _hip.ptr(y), _hip.ptr(gate), gate.stride(0), n, num_heads, vdim, _hip.dtype_code3(y.dtype),
              _hip.stream())
    return y
