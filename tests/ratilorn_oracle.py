"""A plain, slow evaluation of the Ratilorn design: one function per mechanism, straight from the equations, on ONE sequence
given whole, in the dtype of the weights handed in (float32 or float64; nothing is rounded to 16 bits). It shares no code with
swiftllm_amd: the tests compare the framework's kernels, cache and state handling with it.

Notation: h [T, width] is a sublayer's input, W["name"] a checkpoint tensor, positions i (query) and j (key) count from 0.

    layer:      x <- x + N1(mixer(x)),  x <- x + N2(ff(x)),   N(y) = y / sqrt(mean(y^2) + eps) * (1 + w)
    attention:  q, k unit RMS per head; a[h, i, j] = sigmoid(scale q_i.k_j - r1_h ln(1 + r2_h (i - j)) + pb_h) for j <= i;
                a'[h] = sum_g talk[h, g] a[g];  out_i[h] = sum_j a'[h, i, j] v_j[kv(h)];  values of later v_mix layers are
                (1 - lam) v + lam v_first
    parallel:   0.5 (unit_rms(left) * w_left + unit_rms(right) * w_right); left = softmax attention with weighted q/k norm,
                right = the state-space recurrence S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x with a causal convolution
                in front and a gated grouped RMS norm behind
    ff:         down(silu(gate h) * up h), dense or as experts chosen by a sigmoid router with group-limited top-k
"""
import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def embed_tokens(W: dict, tokens, start: int = 0) -> torch.Tensor:
    ids = torch.as_tensor(tokens, dtype=torch.long)
    return W["embed"][ids] + W["pos"][start:start + ids.numel()]


def sigmoid_attention(h, W, p, mx, eps, v_first=None):
    """-> (mixer output [T, width], the values it attends over [T, G * vdim])."""
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = h @ W[p + "v"].T + W[p + "v.b"]
    if v_first is not None:
        lam = W[p + "vmix"]
        v = (1 - lam) * v + lam * v_first
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    rep = H // G
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    dist = (i - j).clamp(min=0).to(h.dtype)
    visible = j <= i
    a = torch.zeros(H, T, T, dtype=h.dtype)
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh // rep].T) * mx["scale"]
        s = s - W[p + "r1"][hh] * torch.log(1 + W[p + "r2"][hh] * dist)
        a[hh] = torch.where(visible, torch.sigmoid(s + W[p + "pb"][hh]), torch.zeros_like(s))
    a = torch.einsum("hg,gij->hij", W[p + "talk"], a)
    vh = v.view(T, G, dv)
    out = torch.stack([a[hh] @ vh[:, hh // rep] for hh in range(H)], dim=1).reshape(T, H * dv)
    return out @ W[p + "o"].T, v


def softmax_attention(h, W, p, mx, eps):
    T = h.shape[0]
    H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q = unit_rms(q, eps) * W[p + "q.norm"]
    k = unit_rms(k, eps) * W[p + "k.norm"]
    rep = H // G
    visible = torch.arange(T).view(1, T) <= torch.arange(T).view(T, 1)
    outs = []
    for hh in range(H):
        s = (q[:, hh] @ k[:, hh // rep].T) * mx["scale"]
        s = s.masked_fill(~visible, float("-inf"))
        outs.append(torch.softmax(s, dim=-1) @ v[:, hh // rep])
    return torch.stack(outs, dim=1).reshape(T, H * dv) @ W[p + "o"].T


def causal_conv(u, w, b):
    """u [T, C], w [C, taps] (last column multiplies the current token), zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    padded = torch.cat((torch.zeros(taps - 1, C, dtype=u.dtype), u), dim=0)
    out = b.expand(T, C).clone()
    for t in range(taps):
        out = out + padded[t:t + T] * w[:, t]
    return out


def state_space_mixer(h, W, p, mx, eps):
    T = h.shape[0]
    Hs, P, N, Gs = mx["heads"], mx["vdim"], mx["state"], mx["groups"]
    inner = Hs * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * Gs * N], proj[:, 2 * inner + 2 * Gs * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, Hs, P)
    B = xbc[:, inner:inner + Gs * N].view(T, Gs, N)
    C = xbc[:, inner + Gs * N:].view(T, Gs, N)
    dt = torch.nn.functional.softplus(dt + W[p + "dt_bias"], beta=1.0, threshold=1e9)
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * dt)          # [T, Hs]
    per = Hs // Gs
    S = torch.zeros(Hs, N, P, dtype=h.dtype)
    y = torch.zeros(T, Hs, P, dtype=h.dtype)
    for t in range(T):
        for hh in range(Hs):
            g = hh // per
            S[hh] = decay[t, hh] * S[hh] + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S[hh].T @ C[t, g] + W[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    parts = mx["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def parallel_mixer(h, W, p, mx, eps):
    left = softmax_attention(h, W, p + "left.", mx["left"], eps)
    right = state_space_mixer(h, W, p + "right.", mx["right"], eps)
    return 0.5 * (unit_rms(left, eps) * W[p + "left.out"] + unit_rms(right, eps) * W[p + "right.out"])


def gated_unit(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z, correction, top, groups=None):
    """z [T, E] router logits -> (chosen experts [T, top], their weights [T, top])."""
    s = torch.sigmoid(z)
    c = s + correction
    T, E = z.shape
    if groups:
        count, keep = groups["count"], groups["keep"]
        per = E // count
        grouped = c.view(T, count, per)
        gscore = grouped.topk(min(2, per), dim=-1).values.sum(dim=-1)
        kept = gscore.topk(keep, dim=-1).indices
        mask = torch.zeros(T, count, dtype=torch.bool)
        mask.scatter_(1, kept, True)
        c = torch.where(mask.view(T, count, 1).expand(T, count, per).reshape(T, E), c, torch.full_like(c, float("-inf")))
    idx = c.topk(top, dim=-1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, mlp):
    r = mlp["router"]
    idx, w = route(h @ W[p + "router"].T, W[p + "correction"], r["top"], r.get("groups"))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] = out[t] + we * gated_unit(h[t:t + 1], W, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_unit(h, W, p + "shared.")
    return out


def forward(W: dict, config: dict, tokens, start: int = 0):
    """-> (logits [T, vocab], [the stream after every layer])."""
    eps = config["norm"]["eps"]
    x = embed_tokens(W, tokens, start)
    v_first = None
    taps = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        if layer["type"] == "attention":
            mx = layer["mixer"]
            m, v = sigmoid_attention(x, W, p + "mix.", mx, eps, v_first if mx.get("v_mix") else None)
            if mx.get("v_mix") and v_first is None:
                v_first = v
        elif layer["type"] == "parallel":
            m = parallel_mixer(x, W, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + unit_rms(m, eps) * (1 + W[p + "norm1"])
        mlp = layer.get("mlp")
        if mlp:
            f = gated_unit(x, W, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(x, W, p + "mlp.", mlp)
            x = x + unit_rms(f, eps) * (1 + W[p + "norm2"])
        taps.append(x.clone())
    hn = unit_rms(x, eps) * (1 + W["final.norm"])
    return (hn @ W["embed"].T) * config["logit_scale"], taps


# ---- random models for the tests -----------------------------------------------------------------------------------------
def tensor_shapes(config: dict) -> dict:
    """name -> shape of every tensor a checkpoint of `config` holds."""
    w = config["width"]
    out = {"embed": (config["vocab"], w), "pos": (config["max_positions"], w), "final.norm": (w,)}

    def attention(p, mx, plain):
        H, G, d, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        out.update({p + "q": (H * d, w), p + "q.b": (H * d,), p + "k": (G * d, w), p + "k.b": (G * d,),
                    p + "v": (G * dv, w), p + "v.b": (G * dv,), p + "o": (w, H * dv)})
        if plain:
            out.update({p + "q.norm": (d,), p + "k.norm": (d,)})
        else:
            out.update({p + "vmix": (), p + "r1": (H,), p + "r2": (H,), p + "talk": (H, H), p + "pb": (H,)})

    def unit(p, ff):
        out.update({p + "gate": (ff, w), p + "up": (ff, w), p + "down": (w, ff)})

    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = (w,)
        if layer["type"] == "attention":
            attention(p + "mix.", layer["mixer"], False)
        else:
            attention(p + "mix.left.", layer["mixer"]["left"], True)
            r = layer["mixer"]["right"]
            inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
            q = p + "mix.right."
            out.update({q + "in": (2 * inner + 2 * gn + r["heads"], w), q + "conv": (inner + 2 * gn, r["conv"]),
                        q + "conv.b": (inner + 2 * gn,), q + "dt_bias": (r["heads"],), q + "A_log": (r["heads"],),
                        q + "D": (r["heads"],), q + "norm": (inner,), q + "o": (w, inner),
                        p + "mix.left.out": (w,), p + "mix.right.out": (w,)})
        mlp = layer.get("mlp")
        if not mlp:
            continue
        out[p + "norm2"] = (w,)
        if mlp["kind"] == "dense":
            unit(p + "mlp.", mlp["ff"])
        else:
            E = mlp["router"]["experts"]
            for e in range(E):
                unit(f"{p}mlp.e{e}.", mlp["expert"]["ff"])
            out.update({p + "mlp.router": (E, w), p + "mlp.correction": (E,)})
            if mlp.get("shared"):
                unit(p + "mlp.shared.", mlp["shared"]["ff"])
    return out


def random_weights(config: dict, seed: int = 0) -> dict:
    """Random tensors with bfloat16-representable values (float32), sized so that every mechanism matters in the output:
    distance terms and gates of order one, recurrences that neither vanish nor blow up."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(config).items():
        leaf = name.split(".")[-1]
        if name.endswith(("q.norm", "k.norm", "left.out", "right.out")) or name.endswith("right.norm"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.2 * torch.randn(shape, generator=g)
        elif leaf == "talk":
            t = torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "r1":
            t = 0.2 + 0.6 * torch.rand(shape, generator=g)
        elif leaf == "r2":
            t = 0.05 + 0.5 * torch.rand(shape, generator=g)
        elif leaf == "pb":
            t = -1.0 + 0.5 * torch.randn(shape, generator=g)
        elif leaf == "vmix":
            t = 0.2 + 0.5 * torch.rand(shape, generator=g)
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif leaf == "A_log":
            t = -1.0 + 1.5 * torch.rand(shape, generator=g)
        elif leaf == "dt_bias":
            t = -2.0 + 2.0 * torch.rand(shape, generator=g)
        elif leaf == "D":
            t = 0.5 + torch.rand(shape, generator=g)
        elif leaf == "correction":
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "b":
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "router":
            t = 2.0 * torch.randn(shape, generator=g) / shape[1] ** 0.5
        elif leaf == "pos":
            t = 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        else:
            t = torch.randn(shape, generator=g)
        W[name] = t.to(torch.bfloat16).to(torch.float32)
    return W


def write_checkpoint(path: str, config: dict, W: dict):
    """config.json and model.safetensors (bfloat16) in the folder `path`."""
    import json
    import os
    import struct
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config, f)
    header, blobs, off = {}, [], 0
    for name, t in W.items():
        raw = t.to(torch.bfloat16).contiguous().view(torch.int16).numpy().tobytes()
        header[name] = {"dtype": "BF16", "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    head = json.dumps(header).encode()
    head += b" " * (-len(head) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for b in blobs:
            f.write(b)


# ---- configurations for the tests ------------------------------------------------------------------------------------------
def dense_mlp(ff=48):
    return {"kind": "dense", "ff": ff}


def moe_mlp(ff=24, experts=8, top=2, groups=(4, 2), shared=16):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, v_mix=True, scale=None, mlp="dense"):
    return {"type": "attention", "mlp": dense_mlp() if mlp == "dense" else mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "v_mix": v_mix,
                      "scale": scale if scale is not None else dim ** -0.5}}


def parallel_layer(heads=4, kv_heads=2, dim=16, vdim=16, s_heads=3, s_vdim=8, state=12, groups=1, conv=3, norm_groups=1,
                   scale=None, mlp="moe"):
    return {"type": "parallel", "mlp": moe_mlp() if mlp == "moe" else mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "scale": scale if scale is not None else dim ** -0.5},
                      "right": {"heads": s_heads, "vdim": s_vdim, "state": state, "groups": groups, "conv": conv,
                                "norm_groups": norm_groups}}}


def make_config(layers=None, width=40, vocab=61, max_positions=160, eps=1e-5, logit_scale=0.5):
    if layers is None:
        layers = [attention_layer(), parallel_layer(), attention_layer(mlp=moe_mlp()), parallel_layer(mlp=dense_mlp())]
    return {"architecture": "Ratilorn", "vocab": vocab, "width": width, "max_positions": max_positions,
            "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": layers}
