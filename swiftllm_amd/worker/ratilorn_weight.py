"""Weight containers and checkpoint reader for Ratilorn.

Tensor names are the checkpoint's: `embed` (also the output projection), `pos`, `final.norm`, and per layer `l<i>.`: `norm1 /
norm2`, the mixer's `mix.*` (a parallel layer's two mixers under `mix.left.*` / `mix.right.*`) and the feed-forward's `mlp.*`.
Linear weights are [out, in].

What the loader does with them:
  * projection matrices go to the device in the compute dtype; matrices that multiply the same input are concatenated into
    one (attention: q | k | v; a parallel layer: left q | k | v, then the recurrence's input projection, each piece starting
    on a multiple of 8 rows; feed-forwards: gate | up), experts are stacked ([experts, 2 ff, width], [experts, width, ff]);
  * everything that enters fp32 arithmetic — norm weights (the layers' and the model's are stored around zero: kept as 1 + w),
    projection biases, q/k norm weights, the distance terms r1 / r2, the per-head offset, the head-mixing matrix, the
    convolution (stored [channels, taps], kept tap-major [taps, channels]) and its bias, A_log / dt_bias / D, the router and
    its choice correction — is kept in fp32 (exact: the checkpoint holds bfloat16);
  * the value-blend coefficient of a layer becomes a Python float (a kernel argument); the output scale of the logits is
    folded into the model's norm weight.
Shapes are checked against config.json before anything is used.
"""
from typing import List

import torch

from .kekapel_weight import Getter, _checkpoint_getter


def _pad_rows(t: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    extra = -t.shape[0] % multiple
    if extra:
        t = torch.cat((t, torch.zeros((extra, t.shape[1]), dtype=t.dtype, device=t.device)), dim=0)
    return t


class RatilornLayerWeight:
    def __init__(self, layer_id: int):
        self.layer_id = layer_id

    def load(self, get: Getter, cfg, lcfg, dtype, device):
        w, p = cfg.hidden_size, f"l{self.layer_id}."

        def f32(name, shape):
            return get(p + name, shape).to(device=device, dtype=torch.float32).contiguous()

        def one_plus(name, shape):
            return (1.0 + get(p + name, shape).to(torch.float32)).to(device).contiguous()

        def mat(name, shape):
            return get(p + name, shape).to(device=device, dtype=dtype).contiguous()

        def attention(q, mx):
            """-> (q | k | v matrix, their biases)"""
            qkv = torch.cat((mat(q + "q", (mx.q_size, w)), mat(q + "k", (mx.k_size, w)), mat(q + "v", (mx.v_size, w))), dim=0)
            return qkv, f32(q + "q.b", (mx.q_size,)), f32(q + "k.b", (mx.k_size,)), f32(q + "v.b", (mx.v_size,))

        self.norm1 = one_plus("norm1", (w,))
        if lcfg.type == "attention":
            mx = lcfg.mixer
            H = mx.num_q_heads
            qkv, self.q_b, self.k_b, self.v_b = attention("mix.", mx)
            self.qkv = qkv.contiguous()
            self.v_mix = float(get(p + "mix.vmix", ()).to(torch.float32)) if mx.v_mix else 0.0
            self.r1, self.r2, self.pb = f32("mix.r1", (H,)), f32("mix.r2", (H,)), f32("mix.pb", (H,))
            self.talk = f32("mix.talk", (H, H))
            self.o = mat("mix.o", (w, mx.o_size))
        else:
            left, right = lcfg.mixer.left, lcfg.mixer.right
            qkv, self.q_b, self.k_b, self.v_b = attention("mix.left.", left)
            self.q_norm = f32("mix.left.q.norm", (left.head_dim,))
            self.k_norm = f32("mix.left.k.norm", (left.head_dim,))
            qkv = _pad_rows(qkv)
            self.right_col = qkv.shape[0]           # where the recurrence's projection starts inside the fused rows
            self.proj = _pad_rows(torch.cat((qkv, mat("mix.right.in", (right.proj_size, w))), dim=0)).contiguous()
            self.left_o = mat("mix.left.o", (w, left.o_size))
            C, t = right.conv_channels, right.conv_taps
            self.conv = f32("mix.right.conv", (C, t)).t().contiguous()       # tap-major
            self.conv_b = f32("mix.right.conv.b", (C,))
            Hs = right.num_heads
            self.dt_bias, self.a_log, self.d_skip = f32("mix.right.dt_bias", (Hs,)), f32("mix.right.A_log", (Hs,)), \
                f32("mix.right.D", (Hs,))
            self.right_norm = f32("mix.right.norm", (right.inner,))
            self.right_o = mat("mix.right.o", (w, right.inner))
            self.left_out, self.right_out = f32("mix.left.out", (w,)), f32("mix.right.out", (w,))
        mlp = lcfg.mlp
        if mlp is None:
            return
        self.norm2 = one_plus("norm2", (w,))
        ff = mlp.ffn_inter_dim
        if mlp.kind == "dense":
            self.gate_up = torch.cat((mat("mlp.gate", (ff, w)), mat("mlp.up", (ff, w))), dim=0).contiguous()
            self.down = mat("mlp.down", (w, ff))
            return
        self.router = f32("mlp.router", (mlp.num_experts, w))
        self.correction = f32("mlp.correction", (mlp.num_experts,))
        self.gate_up = torch.empty((mlp.num_experts, 2 * ff, w), dtype=dtype, device=device)
        self.down = torch.empty((mlp.num_experts, w, ff), dtype=dtype, device=device)
        for e in range(mlp.num_experts):
            self.gate_up[e, :ff] = mat(f"mlp.e{e}.gate", (ff, w))
            self.gate_up[e, ff:] = mat(f"mlp.e{e}.up", (ff, w))
            self.down[e] = mat(f"mlp.e{e}.down", (w, ff))
        self.shared_gate_up = self.shared_down = None
        if mlp.shared_ffn_inter_dim:
            fs = mlp.shared_ffn_inter_dim
            self.shared_gate_up = torch.cat((mat("mlp.shared.gate", (fs, w)), mat("mlp.shared.up", (fs, w))), dim=0).contiguous()
            self.shared_down = mat("mlp.shared.down", (w, fs))


class RatilornWeight:
    def __init__(self, model_config, dtype: torch.dtype):
        self.model_config = model_config
        self.dtype = dtype
        self.layers = [RatilornLayerWeight(i) for i in range(model_config.num_layers)]

    def load(self, get: Getter, device):
        cfg, dtype = self.model_config, self.dtype
        w = cfg.hidden_size
        self.embed = get("embed", (cfg.vocab_size, w)).to(device=device, dtype=dtype).contiguous()
        self.pos = get("pos", (cfg.max_position_embeddings, w)).to(device=device, dtype=dtype).contiguous()
        # logits = embed (norm(x) * (1 + w)) * logit_scale: the scale rides on the norm weight
        self.final_norm = ((1.0 + get("final.norm", (w,)).to(torch.float32)) * cfg.logit_scale).to(device).contiguous()
        self.head = self.embed
        for layer, lcfg in zip(self.layers, cfg.layers):
            layer.load(get, cfg, lcfg, dtype, device)

    def projection_tensors(self) -> List[torch.Tensor]:
        """The 2-D matrices a step multiplies through `linear` (candidates for the decode GEMMs' packed copies)."""
        out = [self.head]
        for layer in self.layers:
            for a in ("qkv", "proj", "o", "left_o", "right_o", "shared_gate_up", "shared_down"):
                t = getattr(layer, a, None)
                if t is not None:
                    out.append(t)
            for a in ("gate_up", "down"):
                t = getattr(layer, a, None)
                if t is not None and t.dim() == 2:
                    out.append(t)
        return out


def _dummy_getter(seed: int = 0) -> Getter:
    """Random weights of the checkpoint's shapes (benchmarks, memory profiling): matrices ~ N(0, 1/in), weights stored around
    zero and biases small, distance terms and recurrence constants of order one — a stream that stays finite at any depth."""
    g = torch.Generator().manual_seed(seed)

    def get(name: str, shape: tuple) -> torch.Tensor:
        leaf = name.split(".")[-1]
        if leaf == "talk":
            return torch.eye(shape[0]) + 0.1 * torch.randn(shape, generator=g)
        if leaf == "conv":
            return torch.randn(shape, generator=g) / shape[1]
        if len(shape) == 2:
            return torch.randn(shape, generator=g) / shape[1] ** 0.5
        if leaf in ("r1", "r2", "vmix"):
            return 0.1 + 0.5 * torch.rand(shape, generator=g)
        if leaf == "pb":
            return -2.0 + 0.5 * torch.randn(shape, generator=g)
        if leaf in ("A_log", "dt_bias"):
            return 0.5 * torch.randn(shape, generator=g)
        if leaf == "D" or name.endswith(("q.norm", "k.norm", "left.out", "right.out", "right.norm")):
            return 1.0 + 0.02 * torch.randn(shape, generator=g)
        return 0.02 * torch.randn(shape, generator=g)
    return get


def load_ratilorn_weights(model_config, dtype: torch.dtype, model_path: str, use_dummy: bool = False,
                          device="cuda") -> RatilornWeight:
    weight = RatilornWeight(model_config, dtype)
    get = _dummy_getter() if use_dummy else _checkpoint_getter(model_path)
    weight.load(get, torch.device(device))
    return weight
