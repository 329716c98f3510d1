"""A plain, slow Rosilix for the tests: one function per mechanism, whole sequences, float64, dense [tokens, tokens] masks.

Nothing here is shared with swiftllm_amd: the product computes the same design with a paged cache and HIP kernels (and, for
the latent attention, with the key up-projection folded into the queries), this file with explicit per-head keys and values
and full score matrices. `W` is a dict name -> tensor with the checkpoint's tensor names, `cfg` the parsed config.json.

Notation: n tokens at positions 0..n-1; H query heads, G key/value heads, d the query/key size, e the value size, r the
latent size, dr the rotated size.
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def rotate_pairs(x, positions, dims, base):
    """x [n, ..., D]: the pairs (2i, 2i + 1), i < dims / 2, turn by the angle position * base^(-2i / dims); the dimensions
    from `dims` on pass unchanged."""
    out = x.clone()
    n = x.shape[0]
    shape = [n] + [1] * (x.dim() - 2)
    for i in range(dims // 2):
        a = positions.to(F64) * float(base) ** (-2.0 * i / dims)
        c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def causal_mask(n):
    i = torch.arange(n)
    return i[None, :] <= i[:, None]


def chunk_mask(n, size):
    """Causal, and only inside the query's own chunk of `size` positions (chunks start at position 0)."""
    i = torch.arange(n)
    return (i[None, :] <= i[:, None]) & ((i[None, :] // size) == (i[:, None] // size))


def softmax_rows(scores, mask, sink=None):
    """Softmax over the visible keys of every row; `sink` (a number) joins the denominator only."""
    s = scores.masked_fill(~mask, -math.inf)
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.as_tensor(float(sink), dtype=F64))
    p = torch.exp(s - m)
    den = p.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(torch.as_tensor(float(sink), dtype=F64) - m)
    return p / den


def diff_lambda(W, pre, diff):
    return float(torch.exp((W[pre + "lq1"] * W[pre + "lk1"]).sum()) - torch.exp((W[pre + "lq2"] * W[pre + "lk2"]).sum())
                 + diff)


def diff_attention_mixer(h, W, pre, mx, eps):
    """Differential attention: two softmax maps per head over the same values, the second subtracted with the layer's
    lambda; per-head unit RMS, (1 - diff), a sigmoid gate per head, output projection."""
    n = h.shape[0]
    H, G, d, e = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    pos = torch.arange(n)
    q = (h @ W[pre + "q"].T).view(n, H, 2, d)
    k = (h @ W[pre + "k"].T).view(n, G, 2, d)
    v = (h @ W[pre + "v"].T).view(n, G, e)
    rot = mx.get("rot")
    if rot:
        q = rotate_pairs(q, pos, rot["dims"], rot["base"])
        k = rotate_pairs(k, pos, rot["dims"], rot["base"])
    size = (mx.get("mask") or {}).get("size")
    mask = chunk_mask(n, size) if size else causal_mask(n)
    lam = diff_lambda(W, pre, mx["diff"])
    gate = torch.sigmoid(h @ W[pre + "g"].T)       # [n, H]
    out = torch.zeros(n, H, e, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, hd, m] @ k[:, g, m].T) * mx["scale"]
            maps.append(softmax_rows(s, mask) @ v[:, g])
        o = maps[0] - lam * maps[1]
        out[:, hd] = unit_rms(o, eps) * (1.0 - mx["diff"]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * e) @ W[pre + "o"].T


def latent_kv(h, W, pre, mx, eps):
    """The cached part of a latent attention layer: (c [n, r] normed latent, kr [n, dr] rotated shared key part)."""
    n = h.shape[0]
    r, dr = mx["kv_rank"], mx["rot_dim"]
    z = h @ W[pre + "dkv"].T
    c = rms_norm(z[:, :r], W[pre + "dkv.norm"], eps)
    kr = rotate_pairs(z[:, r:r + dr], torch.arange(n), mx["rot"]["dims"], mx["rot"]["base"])
    return c, kr


def latent_attention_mixer(h, W, pre, mx, eps, kv):
    """kv = (c, kr) of this layer or of the layer it borrows from. Per head: keys [W_uk c | kr], values W_uv c, softmax with
    the head's sink in the denominator, sigmoid gate, output projection."""
    n = h.shape[0]
    H, d, dr, e, r = mx["heads"], mx["dim"], mx["rot_dim"], mx.get("vdim", mx["dim"]), mx["kv_rank"]
    c, kr = kv
    q = (h @ W[pre + "q"].T).view(n, H, d + dr)
    qn = q[:, :, :d]
    qr = rotate_pairs(q[:, :, d:], torch.arange(n), mx["rot"]["dims"], mx["rot"]["base"])
    kn = (c @ W[pre + "uk"].T).view(n, H, d)
    v = (c @ W[pre + "uv"].T).view(n, H, e)
    gate = torch.sigmoid(h @ W[pre + "g"].T)
    mask = causal_mask(n)
    out = torch.zeros(n, H, e, dtype=F64)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * mx["scale"]
        out[:, hd] = (softmax_rows(s, mask, W[pre + "sink"][hd]) @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * e) @ W[pre + "o"].T


def relu2_ff(h, W, pre):
    return torch.relu(h @ W[pre + "up"].T) ** 2 @ W[pre + "down"].T


def forward(cfg, W, tokens, taps=None):
    """tokens: list of ids of one sequence -> logits [n, vocab] (float64). taps: a list that receives the stream after
    every layer."""
    W = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    cache = {}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        h = rms_norm(x, W[p + "norm1"], eps)
        if layer["type"] == "attention":
            m = diff_attention_mixer(h, W, p + "mix.", mx, eps)
        elif layer["type"] == "latent_attention":
            src = mx.get("kv_from")
            if src is None:
                cache[i] = latent_kv(h, W, p + "mix.", mx, eps)
                src = i
            m = latent_attention_mixer(h, W, p + "mix.", mx, eps, cache[src])
        else:
            raise ValueError(layer["type"])
        x = x + rms_norm(m, W[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = rms_norm(x, W[p + "norm2"], eps)
            x = x + rms_norm(relu2_ff(h, W, p + "mlp."), W[p + "norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T


# ---- making small models -------------------------------------------------------------------------------------------------------
def latent_mixer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=32, base=10000.0, kv_from=None, scale=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
          "rot": {"base": base, "dims": rot_dim}, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": mx}


def diff_mixer(heads=4, kv_heads=2, dim=16, vdim=32, chunk=24, rot_dims=8, base=10000.0, diff=0.25, scale=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
          "scale": scale if scale is not None else dim ** -0.5}
    if rot_dims:
        mx["rot"] = {"base": base, "dims": rot_dims}
    if chunk:
        mx["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": mx}


def make_config(layers, width=64, vocab=96, ff=80, eps=1e-5, embed_scale=4.0, no_mlp=()):
    out = []
    for i, layer in enumerate(layers):
        layer = dict(layer)
        layer["mlp"] = None if i in no_mlp else {"kind": "dense", "ff": ff}
        out.append(layer)
    return {"architecture": "Rosilix", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}, "layers": out}


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    """Random weights with the checkpoint's names and shapes, rounded to `dtype` (what a checkpoint holds)."""
    g = torch.Generator().manual_seed(seed)
    w = cfg["width"]
    W = {}

    def mat(name, rows, cols, gain=1.0):
        W[name] = (torch.randn(rows, cols, generator=g) * gain / math.sqrt(cols)).to(dtype)

    def vec(name, size, mean=1.0, std=0.1):
        W[name] = (mean + std * torch.randn(size, generator=g)).to(dtype)

    mat("embed", cfg["vocab"], w, math.sqrt(w) / cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.get("mlp") else ()):
            vec(p + nm, w)
        if layer["type"] == "attention":
            H, G, d, e = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
            mat(p + "mix.q", H * 2 * d, w, 2.0)
            mat(p + "mix.k", G * 2 * d, w, 2.0)
            mat(p + "mix.v", G * e, w)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                vec(p + "mix." + nm, d, 0.0, 0.2)
            mat(p + "mix.g", H, w)
            mat(p + "mix.o", w, H * e)
        else:
            H, d, dr, e, r = mx["heads"], mx["dim"], mx["rot_dim"], mx.get("vdim", mx["dim"]), mx["kv_rank"]
            mat(p + "mix.q", H * (d + dr), w, 2.0)
            if mx.get("kv_from") is None:
                mat(p + "mix.dkv", r + dr, w, 2.0)
                vec(p + "mix.dkv.norm", r)
            mat(p + "mix.uk", H * d, r, 2.0)
            mat(p + "mix.uv", H * e, r)
            vec(p + "mix.sink", H, 0.0, 1.0)
            mat(p + "mix.g", H, w)
            mat(p + "mix.o", w, H * e)
        if layer.get("mlp"):
            mat(p + "mlp.up", layer["mlp"]["ff"], w)
            mat(p + "mlp.down", w, layer["mlp"]["ff"])
    vec("final.norm", w)
    mat("head", cfg["vocab"], w)
    return W
