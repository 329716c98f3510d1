"""Weight containers and checkpoint reader for Rosilix.

Tensor names are the checkpoint's: `embed`, `final.norm`, `head`, and per layer `l<i>.`: `norm1 / norm1b / norm2 / norm2b`,
the mixer's `mix.*` and the feed-forward's `mlp.up / mlp.down`. Linear weights are [out, in].

What the loader does with them:
  * matrices that multiply the same input are concatenated into one projection, padded with zero rows to a multiple of 8
    rows so that every row of its output starts on a 16-byte boundary:
      differential attention   q | k | v | head gate, with the rows of q and k reordered from [head][map][dim] to
                               [map][head][dim]: the two score maps then are plain attention heads (2 H queries over 2 G keys)
                               whose key head g reads value head g mod G;
      latent attention         q | compressed kv (absent in a layer that reads another layer's cache) | head gate;
  * the latent attention's up-projections are kept per head for batched products: uk [H, dim, kv_rank] (queries are folded
    through it: q_h^T (W_uk,h c) = (W_uk,h^T q_h)^T c) and uv^T [H, kv_rank, vdim] (applied to the attention's output over the
    latent rows);
  * everything that enters fp32 arithmetic — norm weights, the latent's norm weight, the sinks — is kept in fp32 (exact: the
    checkpoint holds bfloat16); the differential attention's lambda, one number per layer, is evaluated here in fp32;
  * rotary frequencies: a float64 table per layer on the device.
Shapes are checked against config.json before anything is used.
"""
import math
from typing import List

import torch

from .kekapel_weight import Getter, _checkpoint_getter
from .kernels.rope_kv import rotary_frequencies


def _pad_rows(t: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    extra = -t.shape[0] % multiple
    if extra:
        t = torch.cat((t, torch.zeros((extra, t.shape[1]), dtype=t.dtype, device=t.device)), dim=0)
    return t.contiguous()


class RosilixLayerWeight:
    def __init__(self, layer_id: int):
        self.layer_id = layer_id

    def load(self, get: Getter, cfg, lcfg, dtype, device):
        w, mx, p = cfg.hidden_size, lcfg.mixer, f"l{self.layer_id}."

        def f32(name, shape):
            return get(p + name, shape).to(device=device, dtype=torch.float32).contiguous()

        def mat(name, shape):
            return get(p + name, shape).to(device=device, dtype=dtype).contiguous()

        for nm in ("norm1", "norm1b") + (("norm2", "norm2b") if lcfg.mlp is not None else ()):
            setattr(self, nm, f32(nm, (w,)))
        H = mx.num_q_heads
        self.freq = rotary_frequencies(mx.rot, device)
        if lcfg.type == "attention":
            G, d = mx.num_kv_heads, mx.head_dim
            q = mat("mix.q", (mx.q_size, w)).view(H, 2, d, w).transpose(0, 1).reshape(mx.q_size, w)
            k = mat("mix.k", (mx.k_size, w)).view(G, 2, d, w).transpose(0, 1).reshape(mx.k_size, w)
            self.proj = _pad_rows(torch.cat((q, k, mat("mix.v", (mx.v_size, w)), mat("mix.g", (H, w))), dim=0))
            self.gate_col = mx.q_size + mx.k_size + mx.v_size
            lam = [get(p + "mix." + nm, (d,)).to(torch.float32) for nm in ("lq1", "lk1", "lq2", "lk2")]
            self.lam = float(torch.exp((lam[0] * lam[1]).sum()) - torch.exp((lam[2] * lam[3]).sum())) + mx.diff
        else:
            parts = [mat("mix.q", (mx.q_size, w))]
            self.dkv_col = -1
            self.c_norm = None
            if mx.kv_from < 0:
                self.dkv_col = mx.q_size
                parts.append(mat("mix.dkv", (mx.dkv_size, w)))
                self.c_norm = f32("mix.dkv.norm", (mx.kv_rank,))
            self.gate_col = sum(t.shape[0] for t in parts)
            parts.append(mat("mix.g", (H, w)))
            self.proj = _pad_rows(torch.cat(parts, dim=0))
            self.uk = mat("mix.uk", (H * mx.head_dim, mx.kv_rank)).view(H, mx.head_dim, mx.kv_rank).contiguous()
            self.uv_t = mat("mix.uv", (H * mx.value_dim, mx.kv_rank)).view(H, mx.value_dim, mx.kv_rank) \
                .transpose(1, 2).contiguous()
            self.sink = f32("mix.sink", (H,))
        self.o = mat("mix.o", (w, mx.o_size))
        if lcfg.mlp is not None:
            self.up = mat("mlp.up", (lcfg.mlp.ffn_inter_dim, w))
            self.down = mat("mlp.down", (w, lcfg.mlp.ffn_inter_dim))


class RosilixWeight:
    def __init__(self, model_config, dtype: torch.dtype):
        self.model_config = model_config
        self.dtype = dtype
        self.layers = [RosilixLayerWeight(i) for i in range(model_config.num_layers)]

    def load(self, get: Getter, device):
        cfg, dtype = self.model_config, self.dtype
        w = cfg.hidden_size
        self.embed = get("embed", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        self.final_norm = get("final.norm", (w,)).to(device=device, dtype=torch.float32).contiguous()
        self.head = get("head", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        for layer, lcfg in zip(self.layers, cfg.layers):
            layer.load(get, cfg, lcfg, dtype, device)

    def projection_tensors(self) -> List[torch.Tensor]:
        """The 2-D matrices a step multiplies through `linear` (candidates for the decode GEMMs' packed copies)."""
        out = [self.head]
        for layer in self.layers:
            for a in ("proj", "o", "up", "down"):
                t = getattr(layer, a, None)
                if t is not None:
                    out.append(t)
        return out


def _dummy_getter(seed: int = 0) -> Getter:
    """Random weights of the checkpoint's shapes (benchmarks, memory profiling): matrices ~ N(0, 1/in), norm weights near
    one, sinks and the lambda vectors small — a stream that stays finite through any depth."""
    g = torch.Generator().manual_seed(seed)

    def get(name: str, shape: tuple) -> torch.Tensor:
        leaf = name.split(".")[-1]
        if len(shape) == 2:
            return torch.randn(shape, generator=g) / math.sqrt(shape[1])
        if leaf in ("lq1", "lk1", "lq2", "lk2"):
            return 0.1 * torch.randn(shape, generator=g)
        if leaf == "sink":
            return 0.5 * torch.randn(shape, generator=g)
        return 1.0 + 0.02 * torch.randn(shape, generator=g)
    return get


def load_rosilix_weights(model_config, dtype: torch.dtype, model_path: str, use_dummy: bool = False,
                         device="cuda") -> RosilixWeight:
    weight = RosilixWeight(model_config, dtype)
    get = _dummy_getter() if use_dummy else _checkpoint_getter(model_path)
    weight.load(get, torch.device(device))
    return weight
