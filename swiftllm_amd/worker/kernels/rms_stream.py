"""fp32 residual stream with RMS norms, gated sublayer results and causal input convolutions with carried state.
csrc/rms_stream.hip."""
import torch

from swiftllm_amd import _hip


def gated_add_rmsnorm(x: torch.Tensor, m: torch.Tensor = None, post: torch.Tensor = None, gate: torch.Tensor = None,
                      gate_bias: torch.Tensor = None, m2: torch.Tensor = None, m2_gate: torch.Tensor = None,
                      pre: torch.Tensor = None, eps: float = 1e-6, out_dtype: torch.dtype = None,
                      row_idx: torch.Tensor = None):
    """In place on the fp32 stream x [T, width]:
        y = m (+ sigmoid(m2_gate[t]) * m2);  y *= sigmoid(gate + gate_bias);  x += y / rms(y) * post
    and returns x / rms(x) * pre in out_dtype when `pre` is given (of rows row_idx only, when given; then m must be None).
    `gate` and `m2_gate` may be column slices of wider matrices (row stride taken from the tensor)."""
    _hip.require_gpu_tensor(x, "x")
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    dtype = m.dtype if m is not None else out_dtype
    if m is not None:
        assert m.shape == x.shape and m.is_contiguous() and post is not None and post.dtype == torch.float32
        assert gate is None or (gate.shape == x.shape and gate.stride(1) == 1 and gate.dtype == dtype
                                and gate_bias.dtype == torch.float32 and gate_bias.numel() == width)
        assert m2 is None or (m2.shape == x.shape and m2.is_contiguous() and m2.dtype == dtype
                              and m2_gate.shape[0] == n and m2_gate.dtype == dtype)
    rows = n if row_idx is None else row_idx.shape[0]
    out = torch.empty((rows, width), dtype=dtype, device=x.device) if pre is not None else None
    if m is None and pre is None:
        return None
    _hip.call("swl_gated_add_rmsnorm", _hip.ptr(x), _hip.ptr(m), _hip.ptr(m2), _hip.ptr(m2_gate),
              m2_gate.stride(0) if m2_gate is not None else 0, _hip.ptr(gate), gate.stride(0) if gate is not None else 0,
              _hip.ptr(gate_bias), _hip.ptr(post), _hip.ptr(out), _hip.ptr(pre), _hip.ptr(row_idx), float(eps), rows, width,
              _hip.dtype_code3(dtype), _hip.stream())
    return out


def post_norm_add(x: torch.Tensor, a: torch.Tensor, post: torch.Tensor, b: torch.Tensor = None, a_norm: torch.Tensor = None,
                  b_norm: torch.Tensor = None, coef: float = 1.0, pre: torch.Tensor = None, eps: float = 1e-6,
                  want_out: bool = True):
    """In place on the fp32 stream x [T, width], for models whose sublayers read the stream itself:
        y = coef * (a' + b');  x += y / rms(y) * post
    with a' = a / rms(a) * a_norm when a_norm is given (else a), b' likewise (b optional). Returns the next sublayer's input
    in a's dtype: x itself, or x / rms(x) * pre when `pre` is given (None when not wanted)."""
    _hip.require_gpu_tensor(x, "x")
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and a.shape == x.shape and a.is_contiguous()
    assert b is None or (b.shape == x.shape and b.is_contiguous() and b.dtype == a.dtype)
    for w in (post, a_norm, b_norm, pre):
        assert w is None or (w.dtype == torch.float32 and w.is_contiguous() and w.numel() == width)
    out = torch.empty((n, width), dtype=a.dtype, device=x.device) if want_out else None
    _hip.call("swl_post_norm_add", _hip.ptr(x), _hip.ptr(a), _hip.ptr(a_norm), _hip.ptr(b), _hip.ptr(b_norm), float(coef),
              _hip.ptr(post), _hip.ptr(out), _hip.ptr(pre) if want_out else 0, float(eps), n, width,
              _hip.dtype_code3(a.dtype), _hip.stream())
    return out


class StateRef:
    """Where a step's kernels find per-sequence state: the slot pool, and the plan's per-token arrays."""
    __slots__ = ("pool", "tok_pos", "tok_start", "tok_state", "tok_seq", "seq_row0", "seq_cnt")

    def __init__(self, pool, tok_pos, tok_start, tok_state, tok_seq, seq_row0, seq_cnt):
        self.pool, self.tok_pos, self.tok_start, self.tok_state = pool, tok_pos, tok_start, tok_state
        self.tok_seq, self.seq_row0, self.seq_cnt = tok_seq, seq_row0, seq_cnt


def causal_conv_state(h: torch.Tensor, w: torch.Tensor, st: StateRef, tail_off: int, add_input: bool) -> torch.Tensor:
    """(h +) causal convolution of h over time per channel; w fp32, tap-major [taps, channels] (the last row multiplies the
    current token); the last taps - 1 inputs of every sequence are carried at `tail_off` inside its state slot."""
    _hip.require_gpu_tensor(h, "h")
    n, c = h.shape
    assert h.stride(1) == 1 and w.dtype == torch.float32 and w.is_contiguous() and w.shape[1] == c
    out = torch.empty((n, c), dtype=h.dtype, device=h.device)
    _hip.call("swl_causal_conv_state", _hip.ptr(out), out.stride(0), _hip.ptr(h), h.stride(0), _hip.ptr(w),
              _hip.ptr(st.pool), st.pool.stride(0), int(tail_off), _hip.ptr(st.tok_pos), _hip.ptr(st.tok_start),
              _hip.ptr(st.tok_state), _hip.ptr(st.tok_seq), n, c, w.shape[0], 1 if add_input else 0,
              _hip.dtype_code3(h.dtype), _hip.stream())
    return out
