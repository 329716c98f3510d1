"""Mixture-of-experts feed-forward: fp32 router + top-k + softmax over the chosen logits, clamped gated experts, weighted
combination. csrc/moe.hip."""
import torch

from swiftllm_amd import _hip


def moe_route(h: torch.Tensor, router: torch.Tensor, bias: torch.Tensor, top_k: int):
    """-> (expert ids int32 [T, top_k], weights fp32 [T, top_k])."""
    _hip.require_gpu_tensor(h, "h")
    n, width = h.shape
    experts = router.shape[0]
    assert h.is_contiguous() and router.dtype == bias.dtype == torch.float32 and router.is_contiguous()
    assert router.shape[1] == width and bias.numel() == experts
    idx = torch.empty((n, top_k), dtype=torch.int32, device=h.device)
    wts = torch.empty((n, top_k), dtype=torch.float32, device=h.device)
    _hip.call("swl_moe_route", _hip.ptr(idx), _hip.ptr(wts), _hip.ptr(h), _hip.ptr(router), _hip.ptr(bias), n, width,
              experts, top_k, _hip.dtype_code3(h.dtype), _hip.stream())
    return idx, wts


def moe_route_scores(h: torch.Tensor, router: torch.Tensor, top_k: int, scale: float):
    """-> (expert ids int32 [T, top_k], weights fp32 [T, top_k]): the top_k experts by fp32 logit; weights = scale * softmax
    over ALL experts at the chosen ones (not renormalised)."""
    _hip.require_gpu_tensor(h, "h")
    n, width = h.shape
    experts = router.shape[0]
    assert h.is_contiguous() and router.dtype == torch.float32 and router.is_contiguous() and router.shape[1] == width
    idx = torch.empty((n, top_k), dtype=torch.int32, device=h.device)
    wts = torch.empty((n, top_k), dtype=torch.float32, device=h.device)
    _hip.call("swl_moe_route_scores", _hip.ptr(idx), _hip.ptr(wts), _hip.ptr(h), _hip.ptr(router), 0, n, width, experts,
              top_k, float(scale), _hip.dtype_code3(h.dtype), _hip.stream())
    return idx, wts


def relu_squared(z: torch.Tensor, ff: int) -> torch.Tensor:
    """relu(z[:, :ff])^2 -> [rows, ff] (z may have more columns)."""
    assert z.dim() == 2 and z.stride(1) == 1 and z.shape[1] >= ff
    y = torch.empty((z.shape[0], ff), dtype=z.dtype, device=z.device)
    _hip.call("swl_relu_sq", _hip.ptr(y), _hip.ptr(z), z.shape[0], ff, z.stride(0), _hip.dtype_code3(z.dtype), _hip.stream())
    return y


def moe_experts_relu2(h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, up: torch.Tensor,
                      down: torch.Tensor) -> torch.Tensor:
    """-> [T, width]: sum_j wts[t, j] * down[e_j] relu(up[e_j] h[t])^2 for experts without a gate. up [experts, ff, width],
    down [experts, width, ff]. Large steps: assignments sorted by expert, a library product per expert; decode-sized 16-bit
    steps: the expert-stationary matrix-core kernel; otherwise the per-assignment kernels."""
    n, width = h.shape
    experts, ff, _ = up.shape
    top_k = idx.shape[1]
    assert up.is_contiguous() and down.is_contiguous() and down.shape == (experts, width, ff)
    assert up.dtype == down.dtype == h.dtype and idx.dtype == torch.int32 and wts.dtype == torch.float32
    code, stream = _hip.dtype_code3(h.dtype), _hip.stream()
    out = torch.empty((n, width), dtype=h.dtype, device=h.device)
    if n * top_k >= GROUPED_MIN_ROWS_PER_EXPERT * experts and not torch.cuda.is_current_stream_capturing():
        flat = idx.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        counts = torch.bincount(flat, minlength=experts).tolist()
        where = torch.empty_like(order)
        where[order] = torch.arange(order.numel(), device=order.device)
        xs = h.index_select(0, order // top_k)
        z = torch.empty((n * top_k, ff), dtype=h.dtype, device=h.device)
        off = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(xs[off:off + c], up[e].t(), out=z[off:off + c])
                off += c
        y = relu_squared(z, ff)
        rows = torch.empty((n * top_k, width), dtype=h.dtype, device=h.device)
        off = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(y[off:off + c], down[e].t(), out=rows[off:off + c])
                off += c
        _hip.call("swl_moe_combine", _hip.ptr(out), _hip.ptr(rows), _hip.ptr(where), _hip.ptr(wts), n, width, top_k, code,
                  stream)
        return out
    y = torch.empty((n * top_k, ff), dtype=h.dtype, device=h.device)
    if h.dtype != torch.float32 and _hip.load().swl_moe_expert_stationary_supported(n, width, ff, top_k, code):
        _hip.call("swl_moe_expert_stationary", _hip.ptr(y), _hip.ptr(h), _hip.ptr(up), _hip.ptr(idx), n, experts, width, ff,
                  top_k, 2, 0.0, code, stream)
        rows = torch.empty((n * top_k, width), dtype=h.dtype, device=h.device)
        _hip.call("swl_moe_expert_stationary", _hip.ptr(rows), _hip.ptr(y), _hip.ptr(down), _hip.ptr(idx), n, experts,
                  width, ff, top_k, 0, 0.0, code, stream)
        _hip.call("swl_moe_combine", _hip.ptr(out), _hip.ptr(rows), _hip.ptr(_identity(n * top_k, h.device)),
                  _hip.ptr(wts), n, width, top_k, code, stream)
        return out
    _hip.call("swl_moe_up_relu2", _hip.ptr(y), _hip.ptr(h), _hip.ptr(up), _hip.ptr(idx), n, width, ff, top_k, code, stream)
    _hip.call("swl_moe_down_combine", _hip.ptr(out), _hip.ptr(y), _hip.ptr(down), _hip.ptr(idx), _hip.ptr(wts), n, width,
              ff, top_k, code, stream)
    return out


# From this many assignments per expert on (on average), a step's expert products are library GEMMs over the assignments
# sorted by expert; below, every assignment streams its expert's rows (decode batches: capturable, no host read-back).
GROUPED_MIN_ROWS_PER_EXPERT = 16


_identities = {}


def _identity(n: int, device) -> torch.Tensor:
    """arange(n) int64 on the device, kept (a captured graph reads it at a fixed address)."""
    t = _identities.get(device)
    if t is None or t.numel() < n:
        t = torch.arange(max(n, 2048), dtype=torch.int64, device=device)
        _identities[device] = t
    return t


ACT_CLAMPED = 0     # min(g, limit) * sigmoid(1.702 g) * (clamp(u, +-limit) + 1)
ACT_SILU = 1        # silu(g) * u


def gated_unit(gu: torch.Tensor, ff: int, act: int = ACT_SILU, limit: float = 0.0) -> torch.Tensor:
    """[rows, gate | up] (products of a fused gate/up projection) -> [rows, ff] through the gated unit `act`."""
    assert gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] == 2 * ff
    y = torch.empty((gu.shape[0], ff), dtype=gu.dtype, device=gu.device)
    _hip.call("swl_glu_clamp", _hip.ptr(y), _hip.ptr(gu), gu.shape[0], ff, float(limit), int(act),
              _hip.dtype_code3(gu.dtype), _hip.stream())
    return y


def moe_route_grouped(h: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, top_k: int, group_count: int = 1,
                      group_keep: int = 1):
    """-> (expert ids int32 [T, top_k], weights fp32 [T, top_k]). Scores s = sigmoid(router h) in fp32; the experts are chosen
    by s + correction among the experts of the group_keep best of group_count equal groups (a group's score: its two largest
    choice scores added); weights = s of the chosen experts over their sum."""
    _hip.require_gpu_tensor(h, "h")
    n, width = h.shape
    experts = router.shape[0]
    assert h.is_contiguous() and router.dtype == torch.float32 and router.is_contiguous() and router.shape[1] == width
    assert correction is None or (correction.dtype == torch.float32 and correction.numel() == experts)
    idx = torch.empty((n, top_k), dtype=torch.int32, device=h.device)
    wts = torch.empty((n, top_k), dtype=torch.float32, device=h.device)
    _hip.call("swl_moe_route_grouped", _hip.ptr(idx), _hip.ptr(wts), _hip.ptr(h), _hip.ptr(router), _hip.ptr(correction), n,
              width, experts, top_k, int(group_count), int(group_keep), _hip.dtype_code3(h.dtype), _hip.stream())
    return idx, wts


def moe_experts_grouped(h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor,
                        limit: float, act: int = ACT_CLAMPED) -> torch.Tensor:
    """The same function as moe_experts for steps with many tokens: assignments sorted by expert (stable), one [rows, width]
    x [width, 2 ff] and one [rows, ff] x [ff, width] library product per expert that received tokens, the activation and
    the weighted combination as kernels. Reads the per-expert counts back to the host (one sync per call)."""
    n, width = h.shape
    experts, two_ff, _ = gate_up.shape
    ff, top_k = two_ff // 2, idx.shape[1]
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)                # sorted position -> assignment (token * top + j)
    counts = torch.bincount(flat, minlength=experts).tolist()
    where = torch.empty_like(order)
    where[order] = torch.arange(order.numel(), device=order.device)     # assignment -> sorted position
    xs = h.index_select(0, order // top_k)
    code, stream = _hip.dtype_code3(h.dtype), _hip.stream()
    gu = torch.empty((n * top_k, two_ff), dtype=h.dtype, device=h.device)
    off = 0
    for e, c in enumerate(counts):
        if c:
            torch.mm(xs[off:off + c], gate_up[e].t(), out=gu[off:off + c])
            off += c
    y = torch.empty((n * top_k, ff), dtype=h.dtype, device=h.device)
    _hip.call("swl_glu_clamp", _hip.ptr(y), _hip.ptr(gu), n * top_k, ff, float(limit), int(act), code, stream)
    rows = torch.empty((n * top_k, width), dtype=h.dtype, device=h.device)
    off = 0
    for e, c in enumerate(counts):
        if c:
            torch.mm(y[off:off + c], down[e].t(), out=rows[off:off + c])
            off += c
    out = torch.empty((n, width), dtype=h.dtype, device=h.device)
    _hip.call("swl_moe_combine", _hip.ptr(out), _hip.ptr(rows), _hip.ptr(where), _hip.ptr(wts), n, width, top_k, code,
              stream)
    return out


def moe_experts(h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor,
                limit: float, act: int = ACT_CLAMPED) -> torch.Tensor:
    """-> [T, width]: sum_j wts[t, j] * expert idx[t, j] applied to h[t]. gate_up [experts, 2 ff, width], down
    [experts, width, ff]. act: the experts' gated unit (ACT_CLAMPED with `limit`, or ACT_SILU)."""
    n, width = h.shape
    experts, two_ff, _ = gate_up.shape
    ff, top_k = two_ff // 2, idx.shape[1]
    assert gate_up.is_contiguous() and down.is_contiguous() and down.shape == (experts, width, ff)
    assert gate_up.dtype == down.dtype == h.dtype and idx.dtype == torch.int32 and wts.dtype == torch.float32
    if n * top_k >= GROUPED_MIN_ROWS_PER_EXPERT * experts and not torch.cuda.is_current_stream_capturing():
        return moe_experts_grouped(h, idx, wts, gate_up, down, limit, act)
    code, stream = _hip.dtype_code3(h.dtype), _hip.stream()
    if h.dtype != torch.float32 and _hip.load().swl_moe_expert_stationary_supported(n, width, ff, top_k, code):
        # decode-sized 16-bit step: every expert's weights are read once, whatever the number of tokens that chose it
        y = torch.empty((n * top_k, ff), dtype=h.dtype, device=h.device)
        _hip.call("swl_moe_expert_stationary", _hip.ptr(y), _hip.ptr(h), _hip.ptr(gate_up), _hip.ptr(idx), n, experts,
                  width, ff, top_k, 3 if act == ACT_SILU else 1, float(limit), code, stream)
        rows = torch.empty((n * top_k, width), dtype=h.dtype, device=h.device)
        _hip.call("swl_moe_expert_stationary", _hip.ptr(rows), _hip.ptr(y), _hip.ptr(down), _hip.ptr(idx), n, experts,
                  width, ff, top_k, 0, float(limit), code, stream)
        out = torch.empty((n, width), dtype=h.dtype, device=h.device)
        _hip.call("swl_moe_combine", _hip.ptr(out), _hip.ptr(rows), _hip.ptr(_identity(n * top_k, h.device)),
                  _hip.ptr(wts), n, width, top_k, code, stream)
        return out
    y = torch.empty((n * top_k, ff), dtype=h.dtype, device=h.device)
    _hip.call("swl_moe_gate_up", _hip.ptr(y), _hip.ptr(h), _hip.ptr(gate_up), _hip.ptr(idx), n, width, ff, top_k,
              float(limit), int(act), code, stream)
    out = torch.empty((n, width), dtype=h.dtype, device=h.device)
    _hip.call("swl_moe_down_combine", _hip.ptr(out), _hip.ptr(y), _hip.ptr(down), _hip.ptr(idx), _hip.ptr(wts), n, width,
              ff, top_k, code, stream)
    return out
