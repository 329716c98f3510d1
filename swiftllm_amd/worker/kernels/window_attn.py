"""Attention over the paged pool for models whose heads are coupled before the softmax: per-head q/k RMS norm fused with
the KV store, then sliding-window attention with tanh soft-capping and an [H, H] head-mixing matrix. Prompt portions (with
or without a cached prefix) and decoded tokens go through the same two launches: every token carries its block-table row
and its position. csrc/qknorm_kv.hip, csrc/window_attn.hip."""
import torch

from swiftllm_amd import _hip


class PoolSlice:
    """Where one layer run keeps its keys and values inside the shared block pool: element offsets inside a block."""
    __slots__ = ("k_offset", "v_offset")

    def __init__(self, k_offset: int, v_offset: int):
        self.k_offset, self.v_offset = k_offset, v_offset


def qknorm_and_store_kv(qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: torch.Tensor, pool: torch.Tensor,
                        pool_slice: PoolSlice, block_table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor,
                        mixer, eps: float):
    """qkv [T, q | k | v] of one fused projection: q heads normalised in place, k heads normalised into the pool, v heads
    copied into the pool. pool None (memory profiling): only the query norm."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == mixer.q_size + mixer.k_size + mixer.v_size
    assert q_norm.dtype == k_norm.dtype == torch.float32 and q_norm.numel() == k_norm.numel() == mixer.head_dim
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == qkv.shape[0]
    kp = vp = 0
    stride = 0
    if pool is not None:
        assert pool.is_contiguous() and pool.dtype == qkv.dtype and block_table.is_contiguous()
        assert tok_seq.dtype == torch.int32 and tok_seq.shape[0] == qkv.shape[0]
        esize = pool.element_size()
        kp = pool.data_ptr() + pool_slice.k_offset * esize
        vp = pool.data_ptr() + pool_slice.v_offset * esize
        stride = pool.shape[1]
    _hip.call("swl_qknorm_store_kv", _hip.ptr(qkv), _hip.ptr(q_norm), _hip.ptr(k_norm), kp, vp, _hip.ptr(block_table),
              _hip.ptr(tok_seq), _hip.ptr(tok_pos), qkv.shape[0], mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
              mixer.value_dim, qkv.stride(0), block_table.shape[1] if block_table is not None else 0, stride, float(eps),
              _hip.dtype_code3(qkv.dtype), _hip.stream())


def qknorm_full_and_store_kv(q_or_qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: torch.Tensor, pool: torch.Tensor,
                             pool_slice: PoolSlice, block_table: torch.Tensor, tok_seq: torch.Tensor,
                             tok_pos: torch.Tensor, mixer, eps: float, store: bool):
    """Whole-projection RMS norms (a weight per element) with the position-dependent query multiplier of `mixer`
    (q_temp_coef, q_temp_every). store: the rows are [q | k | v] and k, v go to the pool; else the rows are queries only."""
    _hip.require_gpu_tensor(q_or_qkv, "qkv")
    width = mixer.q_size + ((mixer.k_size + mixer.v_size) if store else 0)
    assert q_or_qkv.dim() == 2 and q_or_qkv.stride(1) == 1 and q_or_qkv.shape[1] == width
    assert q_norm.dtype == torch.float32 and q_norm.numel() == mixer.q_size
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == q_or_qkv.shape[0]
    kp = vp = stride = 0
    if store and pool is not None:
        assert k_norm.dtype == torch.float32 and k_norm.numel() == mixer.k_size
        assert pool.is_contiguous() and pool.dtype == q_or_qkv.dtype and block_table.is_contiguous()
        esize = pool.element_size()
        kp = pool.data_ptr() + pool_slice.k_offset * esize
        vp = pool.data_ptr() + pool_slice.v_offset * esize
        stride = pool.shape[1]
    _hip.call("swl_qknorm_full_store_kv", _hip.ptr(q_or_qkv), _hip.ptr(q_norm), _hip.ptr(k_norm), kp, vp,
              _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos), q_or_qkv.shape[0], mixer.num_q_heads,
              mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, q_or_qkv.stride(0),
              block_table.shape[1] if block_table is not None else 0, stride, float(eps), float(mixer.q_temp_coef),
              int(mixer.q_temp_every), _hip.dtype_code3(q_or_qkv.dtype), _hip.stream())


def qkv_bias_norm_store(qkv: torch.Tensor, q_b: torch.Tensor, k_b: torch.Tensor, v_b: torch.Tensor, q_norm: torch.Tensor,
                        k_norm: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice, block_table: torch.Tensor,
                        tok_seq: torch.Tensor, tok_pos: torch.Tensor, mixer, eps: float, v_other: torch.Tensor = None,
                        mix: float = 0.0):
    """qkv [T, q | k | v] of one fused projection whose biases (fp32, optional) are still to be added: q heads biased and
    normed in place (q_norm / k_norm [dim] fp32 weights shared by the heads, None: unit RMS without a weight), k heads biased
    and normed into the pool, v biased, blended as (1 - mix) v + mix v_other[t] when v_other [T, kv_heads * vdim] (a column
    slice is fine) is given, and written both back into its columns and into the pool. pool None: no store."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= mixer.q_size + mixer.k_size + mixer.v_size
    for t, size in ((q_b, mixer.q_size), (k_b, mixer.k_size), (v_b, mixer.v_size), (q_norm, mixer.head_dim),
                    (k_norm, mixer.head_dim)):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == size)
    assert tok_pos.dtype == torch.int32 and tok_pos.shape[0] == qkv.shape[0]
    assert v_other is None or (v_other.dtype == qkv.dtype and v_other.stride(1) == 1 and v_other.shape[0] == qkv.shape[0]
                               and v_other.shape[1] == mixer.v_size)
    kp = vp = stride = 0
    if pool is not None:
        assert pool.is_contiguous() and pool.dtype == qkv.dtype and block_table.is_contiguous()
        assert tok_seq.dtype == torch.int32 and tok_seq.shape[0] == qkv.shape[0]
        esize = pool.element_size()
        kp = pool.data_ptr() + pool_slice.k_offset * esize
        vp = pool.data_ptr() + pool_slice.v_offset * esize
        stride = pool.shape[1]
    _hip.call("swl_qkv_bias_norm_store", _hip.ptr(qkv), _hip.ptr(q_b), _hip.ptr(k_b), _hip.ptr(v_b), _hip.ptr(q_norm),
              _hip.ptr(k_norm), _hip.ptr(v_other), v_other.stride(0) if v_other is not None else 0, float(mix), kp, vp,
              _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos), qkv.shape[0], mixer.num_q_heads,
              mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, qkv.stride(0),
              block_table.shape[1] if block_table is not None else 0, stride, float(eps), _hip.dtype_code3(qkv.dtype),
              _hip.stream())


# Steps with at least this many tokens go to the matrix-core kernel (tiles of up to 16 queries; a decoded token is a tile of
# one: the matrix core is mostly padding there, but the kernel reads every page once with wide loads and shares a tile's pages
# out over several workgroups when there are few tiles).
TILES_MIN_TOKENS = 1
_NUM_CUS = 256
_scratch = {}       # device -> persistent fp32 scratch of the key-split partials (fixed address: hipGraph replays use it)
_retired = []


def _split_scratch(device, floats: int) -> torch.Tensor:
    buf = _scratch.get(device)
    if buf is None or buf.numel() < floats:
        if buf is not None:
            _retired.append(buf)        # a captured graph may still replay against it
        buf = torch.empty(max(floats, 1 << 20), dtype=torch.float32, device=device)
        _scratch[device] = buf
    return buf


def choose_key_splits(num_tiles: int, mixer, max_positions: int, slots: int = _NUM_CUS) -> int:
    """Workgroups per tile: enough to occupy the chip (`slots` workgroups) when a step has few tiles, never more than the
    pages a tile can see. A function of the tile count and the model only (not of positions), so a captured decode graph
    stays valid."""
    span = mixer.window if mixer.window > 0 else max_positions
    pages = span // 16 + 2
    return max(1, min(slots // max(num_tiles, 1), pages // 4, 16))


def tiles_supported(mixer, dtype: torch.dtype) -> bool:
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    return bool(_hip.load().swl_window_attn_tiles_supported(mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
                                                            mixer.value_dim, _hip.dtype_code(dtype)))


def window_attention(qkv: torch.Tensor, talk: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice,
                     block_table: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, mixer,
                     tiles=None, max_positions: int = 1 << 20, rel: torch.Tensor = None) -> torch.Tensor:
    """-> [T, heads * vdim]. The queries are the (already normalised) first columns of qkv; keys and values come from the
    pool, which already holds this step's tokens. `tiles` = (tile_row0, tile_cnt) device arrays: the step cut into runs of
    up to 16 consecutive tokens of one sequence — given, and the shape served, the matrix-core kernel runs. `talk` None: the
    heads are not mixed. `rel` (fp32 [heads, distances]): a bias added to head h's score at distance query - key."""
    _hip.require_gpu_tensor(qkv, "qkv")
    assert talk is None or (talk.dtype == torch.float32 and talk.is_contiguous()
                            and talk.shape == (mixer.num_q_heads, mixer.num_q_heads))
    assert rel is None or (rel.dtype == torch.float32 and rel.is_contiguous() and rel.shape[0] == mixer.num_q_heads)
    rel_len = rel.shape[1] if rel is not None else 0
    assert pool.is_contiguous() and pool.dtype == qkv.dtype
    n = qkv.shape[0]
    out = torch.empty((n, mixer.num_q_heads * mixer.value_dim), dtype=qkv.dtype, device=qkv.device)
    esize = pool.element_size()
    if tiles is not None and n >= TILES_MIN_TOKENS and tiles_supported(mixer, qkv.dtype):
        row0, cnt = tiles
        splits = choose_key_splits(row0.shape[0], mixer, max_positions)
        scratch = None
        if splits > 1:
            scratch = _split_scratch(qkv.device, splits * n * mixer.num_q_heads * (mixer.value_dim + 2))
        _hip.call("swl_window_attn_tiles", _hip.ptr(out), _hip.ptr(qkv), pool.data_ptr() + pool_slice.k_offset * esize,
                  pool.data_ptr() + pool_slice.v_offset * esize, _hip.ptr(block_table), _hip.ptr(tok_seq),
                  _hip.ptr(tok_pos), _hip.ptr(row0), _hip.ptr(cnt), _hip.ptr(talk), _hip.ptr(rel), rel_len, row0.shape[0],
                  mixer.num_q_heads,
                  mixer.num_kv_heads, mixer.head_dim, mixer.value_dim, qkv.stride(0), mixer.window, float(mixer.scale),
                  float(mixer.softcap), block_table.shape[1], pool.shape[1], splits, _hip.ptr(scratch), n,
                  _hip.dtype_code(qkv.dtype), _hip.stream())
        return out
    _hip.call("swl_window_attn", _hip.ptr(out), _hip.ptr(qkv), pool.data_ptr() + pool_slice.k_offset * esize,
              pool.data_ptr() + pool_slice.v_offset * esize, _hip.ptr(block_table), _hip.ptr(tok_seq), _hip.ptr(tok_pos),
              _hip.ptr(talk), _hip.ptr(rel), rel_len, n, mixer.num_q_heads, mixer.num_kv_heads, mixer.head_dim,
              mixer.value_dim, qkv.stride(0),
              mixer.window, float(mixer.scale), float(mixer.softcap), block_table.shape[1], pool.shape[1],
              _hip.dtype_code3(qkv.dtype), _hip.stream())
    return out


# ---- the same loops with other masks and denominators -----------------------------------------------------------------------
MASK_WINDOW = 0     # keys [p - window + 1, p]
MASK_CHUNK = 1      # keys [floor(p / window) * window, p]


class AttentionSpec:
    """Shape and constants of one attention over the pool, as the kernels see it (which need not be how the design counts
    its heads: two score maps over shared values are 2 H query heads, 2 G key heads and G value heads).
    num_v_heads: value heads in a page; key head g reads value head g % num_v_heads. window: sliding window or chunk size
    (mask_kind), 0 for every earlier key. sink: fp32 [num_q_heads] logits that join the denominators, or None."""
    __slots__ = ("num_q_heads", "num_kv_heads", "num_v_heads", "head_dim", "value_dim", "window", "mask_kind", "scale",
                 "softcap", "sink", "out_f32")

    def __init__(self, num_q_heads, num_kv_heads, head_dim, value_dim, scale, window=0, mask_kind=MASK_WINDOW,
                 num_v_heads=None, softcap=0.0, sink=None, out_f32=False):
        self.num_q_heads, self.num_kv_heads, self.head_dim, self.value_dim = num_q_heads, num_kv_heads, head_dim, value_dim
        self.num_v_heads = num_kv_heads if num_v_heads is None else num_v_heads
        self.window, self.mask_kind, self.scale, self.softcap, self.sink, self.out_f32 = \
            window, mask_kind, scale, softcap, sink, out_f32


def masked_tiles_supported(spec: AttentionSpec, dtype: torch.dtype) -> bool:
    if dtype not in (torch.float16, torch.bfloat16):
        return False
    return bool(_hip.load().swl_masked_attn_tiles_supported(spec.num_q_heads, spec.num_kv_heads, spec.num_v_heads,
                                                            spec.head_dim, spec.value_dim, _hip.dtype_code(dtype)))


# From this many heads over one shared key head on, a step of single tokens runs with the heads on the matrix-core tile's rows
HEAD_ROWS_MIN_HEADS = 2


def choose_heads_per_group(spec: AttentionSpec) -> int:
    """Heads of one workgroup of the matrix-core kernel (four waves): as many per wave as keep a wave's query, key and value
    fragments and accumulators in registers, so that many or wide heads are shared out over several workgroups."""
    per_wave = max(1, 512 // (spec.head_dim + spec.value_dim))
    per_wave = 4 if per_wave >= 4 else 2 if per_wave >= 2 else 1
    return min(spec.num_q_heads, 4 * per_wave)


def masked_attention(q: torch.Tensor, pool: torch.Tensor, pool_slice: PoolSlice, block_table: torch.Tensor,
                     tok_seq: torch.Tensor, tok_pos: torch.Tensor, spec: AttentionSpec, tiles=None,
                     max_positions: int = 1 << 20) -> torch.Tensor:
    """-> [T, num_q_heads * value_dim] (fp32 when spec.out_f32, else q's dtype). q: rows whose first num_q_heads * head_dim
    columns are the queries (a column slice of a wider matrix is fine); keys and values come from the pool, which already
    holds this step's tokens."""
    _hip.require_gpu_tensor(q, "q")
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= spec.num_q_heads * spec.head_dim
    assert pool.is_contiguous() and pool.dtype == q.dtype and tok_pos.dtype == torch.int32 and tok_seq.dtype == torch.int32
    sink = spec.sink
    assert sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == spec.num_q_heads)
    n = q.shape[0]
    out = torch.empty((n, spec.num_q_heads * spec.value_dim), dtype=torch.float32 if spec.out_f32 else q.dtype,
                      device=q.device)
    esize = pool.element_size()
    kp = pool.data_ptr() + pool_slice.k_offset * esize
    vp = pool.data_ptr() + pool_slice.v_offset * esize
    wide_ok = q.stride(0) % 4 == 0 and q.data_ptr() % 8 == 0 and kp % 8 == 0 and vp % 8 == 0 and pool.shape[1] % 4 == 0
    if tiles is not None and wide_ok and masked_tiles_supported(spec, q.dtype):
        row0, cnt = tiles
        if spec.num_kv_heads == 1 and row0.shape[0] == n and spec.num_q_heads >= HEAD_ROWS_MIN_HEADS:
            # every tile is one token (a decode step) and all heads read one key head: the tile's rows are the heads
            hpg, groups = -1, -(-spec.num_q_heads // 16)
            splits = choose_key_splits(row0.shape[0] * groups, spec, max_positions, slots=4 * _NUM_CUS)   # (one-wave workgroups)
        else:
            hpg = choose_heads_per_group(spec)
            groups = -(-spec.num_q_heads // hpg)
            splits = choose_key_splits(row0.shape[0] * groups, spec, max_positions)
        scratch = None
        if splits > 1:
            scratch = _split_scratch(q.device, splits * n * spec.num_q_heads * (spec.value_dim + 2))
        _hip.call("swl_masked_attn_tiles", _hip.ptr(out), _hip.ptr(q), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
                  _hip.ptr(tok_pos), _hip.ptr(row0), _hip.ptr(cnt), 0, 0, 0, row0.shape[0], spec.num_q_heads,
                  spec.num_kv_heads, spec.head_dim, spec.value_dim, q.stride(0), spec.window, float(spec.scale),
                  float(spec.softcap), block_table.shape[1], pool.shape[1], splits, _hip.ptr(scratch), n, spec.mask_kind,
                  _hip.ptr(sink), spec.num_v_heads, 1 if spec.out_f32 else 0, hpg, _hip.dtype_code(q.dtype), _hip.stream())
        return out
    _hip.call("swl_masked_attn", _hip.ptr(out), _hip.ptr(q), kp, vp, _hip.ptr(block_table), _hip.ptr(tok_seq),
              _hip.ptr(tok_pos), 0, 0, 0, n, spec.num_q_heads, spec.num_kv_heads, spec.head_dim, spec.value_dim, q.stride(0),
              spec.window, float(spec.scale), float(spec.softcap), block_table.shape[1], pool.shape[1], spec.mask_kind,
              _hip.ptr(sink), spec.num_v_heads, 1 if spec.out_f32 else 0, _hip.dtype_code3(q.dtype), _hip.stream())
    return out
