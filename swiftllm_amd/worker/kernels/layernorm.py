"""LayerNorm over an fp32 residual stream, the embedding with learned positions, and the fused step of sandwich-norm
models (normalised sublayer output into the residual, pass-start additions, next input norm). csrc/layernorm.hip."""
import torch

from swiftllm_amd import _hip


def embed_positions(tokens: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, pos: torch.Tensor, scale: float,
                    keep_copy: bool):
    """-> (x fp32 [T, width], copy of it or None): x[t] = embed[tokens[t]] * scale + pos[positions[t]] (pos None: a model
    without learned positions)."""
    _hip.require_gpu_tensor(embed, "embed")
    n, width = tokens.shape[0], embed.shape[1]
    assert embed.is_contiguous() and tokens.dtype == torch.int32
    if pos is not None:
        assert pos.is_contiguous() and pos.shape[1] == width and embed.dtype == pos.dtype
        assert positions.dtype == torch.int32 and positions.shape[0] == n
    x = torch.empty((n, width), dtype=torch.float32, device=embed.device)
    x0 = torch.empty_like(x) if keep_copy else None
    _hip.call("swl_embed_pos", _hip.ptr(x), _hip.ptr(x0), _hip.ptr(embed), _hip.ptr(pos), _hip.ptr(tokens),
              _hip.ptr(positions), float(scale), n, width, _hip.dtype_code3(embed.dtype), _hip.stream())
    return x, x0


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out_dtype: torch.dtype,
              row_idx: torch.Tensor = None) -> torch.Tensor:
    """LayerNorm of the rows of fp32 x (of rows row_idx, when given) -> [rows, width] in out_dtype."""
    _hip.require_gpu_tensor(x, "x")
    assert x.dtype == torch.float32 and x.is_contiguous() and w.dtype == b.dtype == torch.float32
    rows = x.shape[0] if row_idx is None else row_idx.shape[0]
    out = torch.empty((rows, x.shape[1]), dtype=out_dtype, device=x.device)
    _hip.call("swl_layernorm", _hip.ptr(out), _hip.ptr(x), _hip.ptr(row_idx), _hip.ptr(w), _hip.ptr(b), float(eps), rows,
              x.shape[1], _hip.dtype_code3(out_dtype), _hip.stream())
    return out


def add_layernorm(x: torch.Tensor, y: torch.Tensor = None, mult: float = 1.0, post=None, x0: torch.Tensor = None,
                  step: torch.Tensor = None, pre=None, eps: float = 1e-6, out_dtype: torch.dtype = None):
    """In place on the fp32 stream x: x += mult * LN(y; post) (if y) + x0 (if given) + step (a [width] vector, if given);
    returns LN(x; pre) in out_dtype when `pre` = (weight, bias) is given, else None."""
    _hip.require_gpu_tensor(x, "x")
    n, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    assert y is None or (y.shape == x.shape and y.is_contiguous() and post is not None)
    assert x0 is None or (x0.shape == x.shape and x0.dtype == torch.float32 and x0.is_contiguous())
    assert step is None or (step.numel() == width and step.dtype == torch.float32 and step.is_contiguous())
    dtype = y.dtype if y is not None else out_dtype
    out = torch.empty((n, width), dtype=dtype, device=x.device) if pre is not None else None
    if y is None and x0 is None and step is None and pre is None:
        return None
    w1, b1 = post if y is not None else (None, None)
    w2, b2 = pre if pre is not None else (None, None)
    _hip.call("swl_add_layernorm", _hip.ptr(x), _hip.ptr(y), float(mult), _hip.ptr(w1), _hip.ptr(b1), _hip.ptr(x0),
              _hip.ptr(step), _hip.ptr(out), _hip.ptr(w2), _hip.ptr(b2), float(eps), n, width, _hip.dtype_code3(dtype),
              _hip.stream())
    return out
