"""LlamaModelConfig — architecture hyper-parameters read from a HuggingFace `config.json`.

Mirrors swiftllm/model_config.py:5-46 (attribute names, defaults, kv-slot size formula)."""
import json
import os

import torch


class LlamaModelConfig:
    """LLaMA 1/2/3 configuration. Attribute names follow the reference so layer/kernel code and
    user scripts that poke at `model.model_config` keep working."""

    def __init__(self, model_config: dict):
        if model_config["model_type"] != "llama":
            raise AssertionError(f"unsupported model_type {model_config['model_type']!r}")
        if model_config["hidden_act"] != "silu":
            raise AssertionError(f"unsupported hidden_act {model_config['hidden_act']!r}")
        self.num_layers = model_config["num_hidden_layers"]
        self.num_q_heads = model_config["num_attention_heads"]
        self.num_kv_heads = model_config.get("num_key_value_heads", self.num_q_heads)
        self.hidden_size = model_config["hidden_size"]
        self.head_dim = self.hidden_size // self.num_q_heads
        self.vocab_size = model_config["vocab_size"]
        self.max_position_embeddings = model_config["max_position_embeddings"]
        self.ffn_inter_dim = model_config["intermediate_size"]
        self.rope_theta = model_config.get("rope_theta", 10000)
        self.rotary_base = model_config.get("rope_theta", model_config.get("rotary_base", 10000))
        self.rms_norm_eps = model_config["rms_norm_eps"]
        scaling = model_config.get("rope_scaling", 1.0)
        self.rope_scaling = 1.0 if scaling is None else scaling

    def get_kvslot_size(self, dtype: torch.dtype = torch.float16) -> int:
        """Bytes of KV cache one token occupies (K and V, all layers)."""
        return 2 * self.num_layers * self.num_kv_heads * self.head_dim * dtype.itemsize

    @staticmethod
    def load_from_model_path(model_path: str) -> "LlamaModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return LlamaModelConfig(json.load(f))


class KekapelMixerConfig:
    """Sizes and constants of one attention mixer (config `layers[i].mixer`)."""

    def __init__(self, mixer: dict):
        self.num_q_heads = int(mixer["heads"])
        self.num_kv_heads = int(mixer.get("kv_heads", self.num_q_heads))
        self.head_dim = int(mixer["dim"])
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.scale = float(mixer["scale"])
        cap = mixer.get("softcap")
        self.softcap = float(cap) if cap else 0.0           # 0: scores are not capped
        mask = mixer.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 0     # 0: every earlier key is visible
        if self.num_q_heads % self.num_kv_heads:
            raise ValueError(f"heads ({self.num_q_heads}) must be a multiple of kv_heads ({self.num_kv_heads})")

    @property
    def q_size(self) -> int:
        return self.num_q_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim


class KekapelMlpConfig:
    """Feed-forward of one layer: `dense` (PolyNorm activation) or `moe` (router + clamped gated experts)."""

    def __init__(self, mlp: dict):
        self.kind = mlp["kind"]
        if self.kind == "dense":
            self.ffn_inter_dim = int(mlp["ff"])
        elif self.kind == "moe":
            self.ffn_inter_dim = int(mlp["expert"]["ff"])
            self.limit = float(mlp["expert"]["limit"])
            self.num_experts = int(mlp["router"]["experts"])
            self.top_k = int(mlp["router"]["top"])
            if not 0 < self.top_k <= self.num_experts:
                raise ValueError(f"router.top ({self.top_k}) must be in 1..experts ({self.num_experts})")
        else:
            raise ValueError(f"unsupported mlp.kind {self.kind!r}")


class KekapelLayerConfig:
    def __init__(self, layer: dict):
        if layer["type"] != "attention":
            raise ValueError(f"unsupported layer type {layer['type']!r}")
        self.type = layer["type"]
        self.mixer = KekapelMixerConfig(layer["mixer"])
        self.mlp = KekapelMlpConfig(layer["mlp"]) if layer.get("mlp") else None


class LayerRun:
    """One execution of a layer: `layer` indexes the weights, `index` the KV pool slice (a looped layer has one per pass),
    `pass_index` >= 0 on the first layer of a loop pass (where the pass's step vector — and, after the first pass, the
    embedding output — is added to the stream), else -1."""
    __slots__ = ("index", "layer", "pass_index")

    def __init__(self, index: int, layer: int, pass_index: int):
        self.index, self.layer, self.pass_index = index, layer, pass_index


class KekapelModelConfig:
    """Kekapel: a decoder-only model with learned positions, sandwich LayerNorms around every sublayer, sliding-window
    attention with q/k norm, tanh soft-capping and pre-softmax head mixing, dense (PolyNorm) or mixture-of-experts
    feed-forwards, and a span of layers that runs several times with shared weights. Every size and constant is read from
    config.json; layers may differ from one another."""

    def __init__(self, model_config: dict):
        if model_config.get("architecture") != "Kekapel":
            raise AssertionError(f"unsupported architecture {model_config.get('architecture')!r}")
        self.vocab_size = int(model_config["vocab"])
        self.hidden_size = int(model_config["width"])
        self.max_position_embeddings = int(model_config["max_positions"])
        self.norm_eps = float(model_config["norm"]["eps"])
        self.residual_mult = float(model_config.get("residual_mult", 1.0))
        self.embedding_scale = float((model_config.get("embedding") or {}).get("scale", 1.0))
        self.layers = [KekapelLayerConfig(layer) for layer in model_config["layers"]]
        self.num_layers = len(self.layers)
        loop = model_config.get("loop")
        if loop:
            self.loop_start, self.loop_stop, self.loop_times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= self.loop_start < self.loop_stop <= self.num_layers and self.loop_times >= 1):
                raise ValueError(f"bad loop {loop!r} for {self.num_layers} layers")
        else:
            self.loop_start = self.loop_stop = self.loop_times = 0
        self.layer_runs = []
        order = list(range(self.loop_start))
        for t in range(self.loop_times):
            order += [(i, t) for i in range(self.loop_start, self.loop_stop)]
        order += list(range(self.loop_stop, self.num_layers))
        for item in order:
            layer, t = item if isinstance(item, tuple) else (item, -1)
            first = t >= 0 and layer == self.loop_start
            self.layer_runs.append(LayerRun(len(self.layer_runs), layer, t if first else -1))
        self.num_layer_runs = len(self.layer_runs)
        # what the scheduler-facing code reads off any model's configuration
        self.num_q_heads = max(l.mixer.num_q_heads for l in self.layers)
        self.num_kv_heads = max(l.mixer.num_kv_heads for l in self.layers)
        self.head_dim = max(l.mixer.head_dim for l in self.layers)

    def kv_elems_per_token(self) -> int:
        """K and V elements one token occupies over all layer runs."""
        return sum(self.layers[r.layer].mixer.k_size + self.layers[r.layer].mixer.v_size for r in self.layer_runs)

    def get_kvslot_size(self, dtype: torch.dtype = torch.bfloat16) -> int:
        """Bytes of KV cache one token occupies (every layer run has its own keys and values)."""
        return self.kv_elems_per_token() * dtype.itemsize

    @staticmethod
    def load_from_model_path(model_path: str) -> "KekapelModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return KekapelModelConfig(json.load(f))


# ---- Lorulix ---------------------------------------------------------------------------------------------------------------
def distance_bias_rows(table_rows: int, far: float, max_distance: int):
    """Row of a learned distance-bias table for every distance 0 .. max_distance - 1: the first table_rows // 2 distances have
    a row each, beyond that the rows advance in equal steps of log(distance) and the last row is reached at `far`."""
    import math
    half = table_rows // 2
    rows = []
    for dist in range(max_distance):
        if dist < half:
            rows.append(dist)
        else:
            rows.append(min(table_rows - 1,
                            half + int(math.floor(math.log(dist / half) / math.log(far / half) * (table_rows - half)))))
    return rows


class LorulixAttentionConfig:
    """Softmax attention over every earlier key with a whole-projection q/k RMS norm, a position-dependent query
    temperature and a learned bias per (distance bucket, head); optionally on another layer's keys and values."""
    kind = "attention"

    def __init__(self, mixer: dict):
        self.num_q_heads = int(mixer["heads"])
        self.num_kv_heads = int(mixer.get("kv_heads", self.num_q_heads))
        self.head_dim = int(mixer["dim"])
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.scale = float(mixer["scale"])
        self.softcap = 0.0
        self.window = 0
        self.bias_max = float(mixer["bias_max"]) if mixer.get("bias_max") else 0.0     # 0: no distance bias
        temp = mixer.get("q_temp") or {}
        self.q_temp_coef = float(temp.get("coef", 0.0))
        self.q_temp_every = int(temp.get("every", 1))
        self.kv_from = int(mixer["kv_from"]) if mixer.get("kv_from") is not None else -1     # -1: its own keys and values
        if self.num_q_heads % self.num_kv_heads:
            raise ValueError(f"heads ({self.num_q_heads}) must be a multiple of kv_heads ({self.num_kv_heads})")
        if self.q_temp_every < 1:
            raise ValueError(f"q_temp.every must be positive, got {self.q_temp_every}")

    @property
    def q_size(self) -> int:
        return self.num_q_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim


class LorulixDeltaConfig:
    """Gated delta rule: a [dim, vdim] fp32 state per head, short causal convolutions on q, k and v."""
    kind = "delta"

    def __init__(self, mixer: dict):
        self.num_heads = int(mixer["heads"])
        self.num_kv_heads = int(mixer.get("kv_heads", self.num_heads))      # q/k heads
        self.head_dim = int(mixer["dim"])
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.conv_taps = int(mixer.get("conv", 1))
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"heads ({self.num_heads}) must be a multiple of kv_heads ({self.num_kv_heads})")
        if self.conv_taps < 1:
            raise ValueError(f"conv must be positive, got {self.conv_taps}")

    @property
    def qk_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def conv_channels(self) -> int:
        return 2 * self.qk_size + self.v_size

    @property
    def proj_size(self) -> int:
        """Rows of the fused input projection: q | k | v | output gate | beta | decay."""
        return 2 * self.qk_size + 2 * self.v_size + 2 * self.num_heads

    @property
    def state_elems(self) -> int:
        return self.num_heads * self.head_dim * self.value_dim


class LorulixMlpConfig:
    """`dense`: clamped gated unit. `moe`: softmax router over all experts, squared-ReLU experts, optional shared expert."""

    def __init__(self, mlp: dict):
        self.kind = mlp["kind"]
        self.shared_ffn_inter_dim = 0
        if self.kind == "dense":
            self.ffn_inter_dim = int(mlp["ff"])
            self.limit = float(mlp["limit"])
        elif self.kind == "moe":
            self.ffn_inter_dim = int(mlp["expert"]["ff"])
            self.num_experts = int(mlp["router"]["experts"])
            self.top_k = int(mlp["router"]["top"])
            self.router_scale = float(mlp["router"].get("scale", 1.0))
            if mlp.get("shared"):
                self.shared_ffn_inter_dim = int(mlp["shared"]["ff"])
            if not 0 < self.top_k <= self.num_experts:
                raise ValueError(f"router.top ({self.top_k}) must be in 1..experts ({self.num_experts})")
        else:
            raise ValueError(f"unsupported mlp.kind {self.kind!r}")


class LorulixLayerConfig:
    def __init__(self, layer: dict):
        self.type = layer["type"]
        if self.type == "attention":
            self.mixer = LorulixAttentionConfig(layer["mixer"])
        elif self.type == "delta":
            self.mixer = LorulixDeltaConfig(layer["mixer"])
        else:
            raise ValueError(f"unsupported layer type {self.type!r}")
        self.mlp = LorulixMlpConfig(layer["mlp"]) if layer.get("mlp") else None


class LorulixModelConfig:
    """Lorulix: a decoder-only model with learned positions and an fp32 stream; every sublayer reads the RMS-normed stream
    plus a short causal convolution of it, and its result is gated, normed and added. Mixers are gated-delta-rule
    recurrences or distance-biased softmax attention (possibly on an earlier layer's keys and values); feed-forwards are a
    clamped gated unit or a mixture of squared-ReLU experts. Every size and constant is read from config.json."""

    def __init__(self, model_config: dict):
        if model_config.get("architecture") != "Lorulix":
            raise AssertionError(f"unsupported architecture {model_config.get('architecture')!r}")
        self.vocab_size = int(model_config["vocab"])
        self.hidden_size = int(model_config["width"])
        self.max_position_embeddings = int(model_config["max_positions"])
        self.norm_eps = float(model_config["norm"]["eps"])
        self.canon_taps = int((model_config.get("canon") or {}).get("taps", 1))
        if self.canon_taps < 1:
            raise ValueError(f"canon.taps must be positive, got {self.canon_taps}")
        self.layers = [LorulixLayerConfig(layer) for layer in model_config["layers"]]
        self.num_layers = len(self.layers)
        for i, layer in enumerate(self.layers):
            if layer.type != "attention" or layer.mixer.kv_from < 0:
                continue
            j = layer.mixer.kv_from
            src = self.layers[j] if 0 <= j < i else None
            if src is None or src.type != "attention" or src.mixer.kv_from >= 0:
                raise ValueError(f"layer {i}: kv_from {j} must name an earlier attention layer with keys of its own")
            a, b = layer.mixer, src.mixer
            if (a.num_kv_heads, a.head_dim, a.value_dim) != (b.num_kv_heads, b.head_dim, b.value_dim):
                raise ValueError(f"layer {i}: key/value sizes differ from those of layer {j}")
        attn = [l.mixer for l in self.layers if l.type == "attention"] or [None]
        # what the scheduler-facing code reads off any model's configuration
        self.num_q_heads = max((m.num_q_heads for m in attn if m), default=1)
        self.num_kv_heads = max((m.num_kv_heads for m in attn if m), default=1)
        self.head_dim = max((m.head_dim for m in attn if m), default=1)

    def kv_elems_per_token(self) -> int:
        """K and V elements one token occupies over the attention layers that keep their own."""
        return sum(l.mixer.k_size + l.mixer.v_size for l in self.layers if l.type == "attention" and l.mixer.kv_from < 0)

    def get_kvslot_size(self, dtype: torch.dtype = torch.bfloat16) -> int:
        return max(self.kv_elems_per_token(), 1) * dtype.itemsize

    @staticmethod
    def load_from_model_path(model_path: str) -> "LorulixModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return LorulixModelConfig(json.load(f))


# ---- Rosilix ---------------------------------------------------------------------------------------------------------------
class RotaryConfig:
    """Rotary positions on interleaved pairs: dimension 2i of a head turns with dimension 2i + 1 by the angle
    position * base^(-2i / dims), for i < dims / 2; the dimensions from `dims` on pass unchanged."""

    def __init__(self, rot: dict, head_dim: int):
        self.dims = int(rot["dims"]) if rot else 0
        self.base = float(rot["base"]) if rot else 1.0
        if self.dims < 0 or self.dims % 2 or self.dims > head_dim:
            raise ValueError(f"rot.dims ({self.dims}) must be even and at most the head size ({head_dim})")

    def frequencies(self):
        """base^(-2i / dims) for i < dims / 2, in float64."""
        return [self.base ** (-2.0 * i / self.dims) for i in range(self.dims // 2)]


class RosilixDiffAttentionConfig:
    """Differential attention: every head holds two score maps (queries and keys of 2 * dim, laid out [map 1 | map 2]) over
    the same values; the maps' outputs are combined as a1 - lambda * a2, brought to unit RMS per head, scaled by 1 - diff
    and gated per head. Keys are visible inside the query's own chunk of `chunk` positions (0: every earlier key)."""
    kind = "attention"

    def __init__(self, mixer: dict):
        self.num_q_heads = int(mixer["heads"])
        self.num_kv_heads = int(mixer.get("kv_heads", self.num_q_heads))
        self.head_dim = int(mixer["dim"])                       # of one map
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.scale = float(mixer["scale"])
        self.diff = float(mixer["diff"])
        mask = mixer.get("mask") or {}
        self.chunk = int(mask["size"]) if mask.get("size") else 0
        self.rot = RotaryConfig(mixer.get("rot"), self.head_dim)
        self.kv_from = -1
        if self.num_q_heads % self.num_kv_heads:
            raise ValueError(f"heads ({self.num_q_heads}) must be a multiple of kv_heads ({self.num_kv_heads})")
        if self.head_dim % 2:
            raise ValueError(f"dim ({self.head_dim}) must be even")

    @property
    def q_size(self) -> int:
        return 2 * self.num_q_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return 2 * self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def o_size(self) -> int:
        return self.num_q_heads * self.value_dim


class RosilixLatentAttentionConfig:
    """Latent attention: keys and values of all heads are up-projections of one cached latent row of `kv_rank` per token,
    plus one rotated key part of `rot_dim` shared by the heads; a learned sink per head joins the softmax denominator; the
    heads are gated. `kv_from` >= 0: the layer has no compression of its own and reads that layer's cached rows."""
    kind = "latent_attention"

    def __init__(self, mixer: dict):
        self.num_q_heads = int(mixer["heads"])
        self.num_kv_heads = 1
        self.head_dim = int(mixer["dim"])                       # unrotated part of a query / key head
        self.rot_dim = int(mixer["rot_dim"])
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.kv_rank = int(mixer["kv_rank"])
        self.scale = float(mixer["scale"])
        self.rot = RotaryConfig(mixer["rot"], self.rot_dim)
        self.kv_from = int(mixer["kv_from"]) if mixer.get("kv_from") is not None else -1
        if self.rot.dims != self.rot_dim:
            raise ValueError(f"rot.dims ({self.rot.dims}) must equal rot_dim ({self.rot_dim})")

    @property
    def q_size(self) -> int:
        return self.num_q_heads * (self.head_dim + self.rot_dim)

    @property
    def dkv_size(self) -> int:
        return self.kv_rank + self.rot_dim

    @property
    def k_size(self) -> int:
        """Elements of the cached key row: the latent and the shared rotated part."""
        return self.kv_rank + self.rot_dim

    @property
    def v_size(self) -> int:
        """Elements of the cached value row: the latent once more (kept transposed for the value product)."""
        return self.kv_rank

    @property
    def o_size(self) -> int:
        return self.num_q_heads * self.value_dim


class RosilixMlpConfig:
    """`dense`: down(relu(up h)^2)."""

    def __init__(self, mlp: dict):
        self.kind = mlp["kind"]
        if self.kind != "dense":
            raise ValueError(f"unsupported mlp.kind {self.kind!r}")
        self.ffn_inter_dim = int(mlp["ff"])


class RosilixLayerConfig:
    def __init__(self, layer: dict):
        self.type = layer["type"]
        if self.type == "attention":
            self.mixer = RosilixDiffAttentionConfig(layer["mixer"])
        elif self.type == "latent_attention":
            self.mixer = RosilixLatentAttentionConfig(layer["mixer"])
        else:
            raise ValueError(f"unsupported layer type {self.type!r}")
        self.mlp = RosilixMlpConfig(layer["mlp"]) if layer.get("mlp") else None


class RosilixModelConfig:
    """Rosilix: a decoder-only model with an fp32 stream, RMS norms before and after every sublayer, rotary positions on
    interleaved pairs, and two kinds of mixer in any order: chunked differential attention and latent attention with a
    softmax sink (a layer may read an earlier latent layer's cache). Feed-forwards are squared-ReLU. Every size and constant
    is read from config.json. The design has no position table: `max_positions`, if config.json gives it, bounds a sequence;
    otherwise the bound is DEFAULT_MAX_POSITIONS."""
    DEFAULT_MAX_POSITIONS = 1 << 20

    def __init__(self, model_config: dict):
        if model_config.get("architecture") != "Rosilix":
            raise AssertionError(f"unsupported architecture {model_config.get('architecture')!r}")
        self.vocab_size = int(model_config["vocab"])
        self.hidden_size = int(model_config["width"])
        self.max_position_embeddings = int(model_config.get("max_positions") or self.DEFAULT_MAX_POSITIONS)
        self.norm_eps = float(model_config["norm"]["eps"])
        self.embedding_scale = float((model_config.get("embedding") or {}).get("scale", 1.0))
        self.layers = [RosilixLayerConfig(layer) for layer in model_config["layers"]]
        self.num_layers = len(self.layers)
        for i, layer in enumerate(self.layers):
            j = layer.mixer.kv_from
            if j < 0:
                continue
            src = self.layers[j] if 0 <= j < i else None
            if src is None or src.type != "latent_attention" or src.mixer.kv_from >= 0:
                raise ValueError(f"layer {i}: kv_from {j} must name an earlier latent attention layer with a cache of its own")
            a, b = layer.mixer, src.mixer
            if (a.kv_rank, a.rot_dim, a.rot.base) != (b.kv_rank, b.rot_dim, b.rot.base):
                raise ValueError(f"layer {i}: latent size or rotation differ from those of layer {j}")
        # what the scheduler-facing code reads off any model's configuration
        self.num_q_heads = max(l.mixer.num_q_heads for l in self.layers)
        self.num_kv_heads = max(l.mixer.num_kv_heads for l in self.layers)
        self.head_dim = max(l.mixer.head_dim for l in self.layers)

    def kv_elems_per_token(self) -> int:
        """Cached elements per token over the layers that keep a cache of their own."""
        return sum(l.mixer.k_size + l.mixer.v_size for l in self.layers if l.mixer.kv_from < 0)

    def get_kvslot_size(self, dtype: torch.dtype = torch.bfloat16) -> int:
        return max(self.kv_elems_per_token(), 1) * dtype.itemsize

    @staticmethod
    def load_from_model_path(model_path: str) -> "RosilixModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return RosilixModelConfig(json.load(f))


# ---- Ratilorn --------------------------------------------------------------------------------------------------------------
class RatilornAttentionConfig:
    """Attention with biased projections. `sigmoid` = True: keys and queries of unit RMS per head, every visible key weighted by
    a sigmoid of its score minus a logarithmic distance term, the heads' weights mixed afterwards, values optionally blended
    with those of the first such layer (`v_mix`). `sigmoid` = False: softmax attention with a weighted q/k norm and no
    positional term at all."""

    def __init__(self, mixer: dict, sigmoid: bool):
        self.kind = "sigmoid_attention" if sigmoid else "attention"
        self.sigmoid = sigmoid
        self.num_q_heads = int(mixer["heads"])
        self.num_kv_heads = int(mixer.get("kv_heads", self.num_q_heads))
        self.head_dim = int(mixer["dim"])
        self.value_dim = int(mixer.get("vdim", self.head_dim))
        self.scale = float(mixer["scale"])
        self.v_mix = bool(mixer.get("v_mix", False)) if sigmoid else False
        self.softcap = 0.0
        self.window = 0         # every earlier key is visible
        if self.num_q_heads % self.num_kv_heads:
            raise ValueError(f"heads ({self.num_q_heads}) must be a multiple of kv_heads ({self.num_kv_heads})")

    @property
    def q_size(self) -> int:
        return self.num_q_heads * self.head_dim

    @property
    def k_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_size(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def o_size(self) -> int:
        return self.num_q_heads * self.value_dim


class StateSpaceConfig:
    """A state-space recurrence with a scalar decay per head: `heads` heads of `vdim` inputs, a state [state, vdim] per head,
    B and C shared by the heads of each of `groups` groups, a causal convolution of `conv` taps on x | B | C, and a gated RMS
    norm of the result in `norm_groups` equal parts."""
    kind = "state_space"

    def __init__(self, mixer: dict):
        self.num_heads = int(mixer["heads"])
        self.value_dim = int(mixer["vdim"])
        self.state_dim = int(mixer["state"])
        self.groups = int(mixer.get("groups", 1))
        self.conv_taps = int(mixer.get("conv", 1))
        self.norm_groups = int(mixer.get("norm_groups", 1))
        if self.groups < 1 or self.num_heads % self.groups:
            raise ValueError(f"heads ({self.num_heads}) must be a multiple of groups ({self.groups})")
        if self.conv_taps < 1:
            raise ValueError(f"conv must be positive, got {self.conv_taps}")
        if self.norm_groups < 1 or self.inner % self.norm_groups:
            raise ValueError(f"heads * vdim ({self.inner}) must be a multiple of norm_groups ({self.norm_groups})")

    @property
    def inner(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state_dim

    @property
    def proj_size(self) -> int:
        """Rows of the input projection: z | x | B | C | dt."""
        return self.inner + self.conv_channels + self.num_heads

    @property
    def state_elems(self) -> int:
        return self.num_heads * self.state_dim * self.value_dim


class RatilornParallelConfig:
    """Two mixers side by side on the same input: softmax attention (`left`) and a state-space recurrence (`right`); the layer
    takes half the sum of their separately normed results."""
    kind = "parallel"

    def __init__(self, mixer: dict):
        self.left = RatilornAttentionConfig(mixer["left"], sigmoid=False)
        self.right = StateSpaceConfig(mixer["right"])


class RatilornMlpConfig:
    """`dense`: down(silu(gate h) * up h). `moe`: the same unit as experts behind a sigmoid router with a choice correction and
    group-limited top-k, plus an optional shared expert."""

    def __init__(self, mlp: dict):
        self.kind = mlp["kind"]
        self.shared_ffn_inter_dim = 0
        if self.kind == "dense":
            self.ffn_inter_dim = int(mlp["ff"])
        elif self.kind == "moe":
            router = mlp["router"]
            self.ffn_inter_dim = int(mlp["expert"]["ff"])
            self.num_experts = int(router["experts"])
            self.top_k = int(router["top"])
            groups = router.get("groups") or {}
            self.group_count = int(groups.get("count", 1))
            self.group_keep = int(groups.get("keep", self.group_count))
            if mlp.get("shared"):
                self.shared_ffn_inter_dim = int(mlp["shared"]["ff"])
            if not 0 < self.top_k <= self.num_experts:
                raise ValueError(f"router.top ({self.top_k}) must be in 1..experts ({self.num_experts})")
            if self.group_count < 1 or self.num_experts % self.group_count or not 0 < self.group_keep <= self.group_count:
                raise ValueError(f"bad router groups {groups!r} for {self.num_experts} experts")
            if self.group_keep * (self.num_experts // self.group_count) < self.top_k:
                raise ValueError(f"router groups {groups!r} leave fewer than top ({self.top_k}) experts to choose from")
        else:
            raise ValueError(f"unsupported mlp.kind {self.kind!r}")


class RatilornLayerConfig:
    def __init__(self, layer: dict):
        self.type = layer["type"]
        if self.type == "attention":
            self.mixer = RatilornAttentionConfig(layer["mixer"], sigmoid=True)
        elif self.type == "parallel":
            self.mixer = RatilornParallelConfig(layer["mixer"])
        else:
            raise ValueError(f"unsupported layer type {self.type!r}")
        self.mlp = RatilornMlpConfig(layer["mlp"]) if layer.get("mlp") else None

    @property
    def attention(self) -> RatilornAttentionConfig:
        """The layer's attention (the one whose keys and values the block pool holds)."""
        return self.mixer if self.type == "attention" else self.mixer.left


class RatilornModelConfig:
    """Ratilorn: a decoder-only model with learned positions and an fp32 stream that every sublayer reads as it is; a
    sublayer's RESULT is RMS-normed (weight stored around zero) and added. Mixers are sigmoid attention with a logarithmic
    distance penalty and post-sigmoid head mixing, or softmax attention beside a state-space recurrence; feed-forwards are a
    SiLU gated unit, dense or as a mixture of experts. The embedding table is the output projection too. Every size and
    constant is read from config.json; layers may differ from one another."""

    def __init__(self, model_config: dict):
        if model_config.get("architecture") != "Ratilorn":
            raise AssertionError(f"unsupported architecture {model_config.get('architecture')!r}")
        self.vocab_size = int(model_config["vocab"])
        self.hidden_size = int(model_config["width"])
        self.max_position_embeddings = int(model_config["max_positions"])
        self.norm_eps = float(model_config["norm"]["eps"])
        self.logit_scale = float(model_config.get("logit_scale", 1.0))
        self.layers = [RatilornLayerConfig(layer) for layer in model_config["layers"]]
        self.num_layers = len(self.layers)
        # the layers whose values are blended with those of the first of them
        self.v_mix_layers = [i for i, l in enumerate(self.layers) if l.type == "attention" and l.mixer.v_mix]
        for i in self.v_mix_layers[1:]:
            a, b = self.layers[i].mixer, self.layers[self.v_mix_layers[0]].mixer
            if a.v_size != b.v_size:
                raise ValueError(f"layer {i}: v_mix needs values of the size of layer {self.v_mix_layers[0]}'s "
                                 f"({a.v_size} vs {b.v_size})")
        attn = [l.attention for l in self.layers]
        # what the scheduler-facing code reads off any model's configuration
        self.num_q_heads = max(m.num_q_heads for m in attn)
        self.num_kv_heads = max(m.num_kv_heads for m in attn)
        self.head_dim = max(m.head_dim for m in attn)

    @property
    def has_state(self) -> bool:
        return any(l.type == "parallel" for l in self.layers)

    def kv_elems_per_token(self) -> int:
        """K and V elements one token occupies over all layers (every layer has one attention)."""
        return sum(l.attention.k_size + l.attention.v_size for l in self.layers)

    def get_kvslot_size(self, dtype: torch.dtype = torch.bfloat16) -> int:
        return max(self.kv_elems_per_token(), 1) * dtype.itemsize

    @staticmethod
    def load_from_model_path(model_path: str) -> "RatilornModelConfig":
        with open(os.path.join(model_path, "config.json"), "r", encoding="utf-8") as f:
            return RatilornModelConfig(json.load(f))
