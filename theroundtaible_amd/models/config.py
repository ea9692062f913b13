"""Model architecture presets (SURVEY §2.4.1 shape table)."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, replace
from typing import Callable, Dict, Optional, Tuple


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Sizes and constants of one latent-attention mixer (low-rank queries; keys and values
    from one cached latent plus a rotated key part shared by all heads; a softmax sink per head)."""
    heads: int
    dim: int              # unrotated query / key dims per head
    rot_dim: int          # rotated query / key dims per head (the key part is shared by the heads)
    vdim: int             # value dims per head
    kv_rank: int          # width of the cached latent
    q_rank: int           # width of the query latent
    rot_base: float
    rot_dims: int         # leading entries of the rotated part that take the rotation
    scale: float

    @property
    def cache_row(self) -> int:
        """Cached numbers per token: the latent and the rotated key part."""
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer of a per-layer-configured model: its mixer, its feed-forward (``ff`` 0 =
    none) and ``source``, the layer whose tensors it uses (itself unless its weights are shared)."""
    mixer_type: str
    mixer: LatentAttentionSpec
    ff: int
    ff_kind: str
    source: int


@dataclass(frozen=True)
class ModelConfig:
    name: str
    arch: str                 # "llama" (Llama-3 / Mistral / Qwen2) | "gpt2"
    n_layers: int
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    ffn: int
    vocab: int
    max_pos: int
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    tie_embeddings: bool = False
    qkv_bias: bool = False    # Qwen2 / Qwen2.5: biased q/k/v projections (added before RoPE)
    # checkpoint RoPE scaling (ops/reference.py rope_inv_freq): ("linear", f) | ("llama3", f, low,
    # high, original_max_pos) | ("yarn", f, original_max_pos, beta_fast, beta_slow, attention_factor)
    rope_scaling: Optional[tuple] = None
    # per-layer-configured architectures ("mupulorn"): the layers, the taps of the causal input
    # convolution ahead of every sublayer, and the output scaling / soft cap of the logits
    layers: Optional[Tuple[LayerSpec, ...]] = None
    canon_taps: int = 0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0

    @property
    def q_size(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.n_heads // self.n_kv_heads

    def n_params(self) -> int:
        h, f, v, L = self.hidden, self.ffn, self.vocab, self.n_layers
        if self.layers is not None:
            n = 2 * v * h + 1
            for i, ls in enumerate(self.layers):
                if ls.source != i:
                    continue
                m = ls.mixer
                n += h * (m.q_rank + m.cache_row + m.heads * m.vdim) + m.q_rank + m.kv_rank + m.heads
                n += m.q_rank * m.heads * (m.dim + m.rot_dim) + m.kv_rank * m.heads * (m.dim + m.vdim)
                n += m.heads * m.vdim * h + 2 + self.canon_taps * h
                if ls.ff:
                    n += 2 * h * ls.ff + 6 + self.canon_taps * h
            return n
        if self.arch == "gpt2":
            per = 4 * h * h + 2 * h * f + 9 * h + f
            return L * per + v * h + self.max_pos * h + 2 * h
        per = h * (self.q_size + 2 * self.kv_size) + self.q_size * h + 3 * h * f + 2 * h
        if self.qkv_bias:
            per += self.q_size + 2 * self.kv_size
        emb = v * h * (1 if self.tie_embeddings else 2)
        return L * per + emb + h

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.layers is not None:
            return sum(ls.mixer.cache_row for ls in self.layers) * dtype_bytes
        return 2 * self.n_layers * self.n_kv_heads * self.head_dim * dtype_bytes


PRESETS: Dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig("llama3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 131072, 500000.0, 1e-5),
    # Llama 3.1 / 3.2: the same blocks with rope_type "llama3" scaling (3.2: tied embeddings;
    # 3.2-3B has GQA group 3)
    "llama3.1-8b": ModelConfig("llama3.1-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 131072, 500000.0, 1e-5,
                               False, False, ("llama3", 8.0, 1.0, 4.0, 8192)),
    "llama3.2-1b": ModelConfig("llama3.2-1b", "llama", 16, 2048, 32, 8, 64, 8192, 128256, 131072, 500000.0, 1e-5,
                               True, False, ("llama3", 32.0, 1.0, 4.0, 8192)),
    "llama3.2-3b": ModelConfig("llama3.2-3b", "llama", 28, 3072, 24, 8, 128, 8192, 128256, 131072, 500000.0, 1e-5,
                               True, False, ("llama3", 32.0, 1.0, 4.0, 8192)),
    "llama3-70b": ModelConfig("llama3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256, 131072, 500000.0, 1e-5),
    "mistral-7b": ModelConfig("mistral-7b", "llama", 32, 4096, 32, 8, 128, 14336, 32000, 32768, 1000000.0, 1e-5),
    # Qwen2.5 (HF model_type "qwen2"): the Llama block with q/k/v biases; 7B: GQA 28 / 4 heads,
    # 0.5B: head_dim 64, tied embeddings (the family most local coding setups run)
    "qwen2.5-7b": ModelConfig("qwen2.5-7b", "llama", 28, 3584, 28, 4, 128, 18944, 152064, 32768, 1000000.0, 1e-6,
                              False, True),
    "qwen2.5-14b": ModelConfig("qwen2.5-14b", "llama", 48, 5120, 40, 8, 128, 13824, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-32b": ModelConfig("qwen2.5-32b", "llama", 64, 5120, 40, 8, 128, 27648, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-72b": ModelConfig("qwen2.5-72b", "llama", 80, 8192, 64, 8, 128, 29568, 152064, 32768, 1000000.0, 1e-6,
                               False, True),
    "qwen2.5-0.5b": ModelConfig("qwen2.5-0.5b", "llama", 24, 896, 14, 2, 64, 4864, 151936, 32768, 1000000.0, 1e-6,
                                True, True),
    # GPT-2-small: random init allows n_positions beyond 1024 (SURVEY §7.3 hard part 3).
    "gpt2-small": ModelConfig("gpt2-small", "gpt2", 12, 768, 12, 12, 64, 3072, 50257, 8192, 0.0, 1e-5, True),
    # test-sized models (CPU unit tests, GPU smoke)
    "tiny-llama": ModelConfig("tiny-llama", "llama", 2, 256, 4, 2, 64, 512, 32000, 4096, 10000.0, 1e-5),
    "tiny-llama-128": ModelConfig("tiny-llama-128", "llama", 2, 512, 4, 1, 128, 1024, 32000, 8192, 500000.0, 1e-5),
    "tiny-qwen": ModelConfig("tiny-qwen", "llama", 2, 256, 4, 2, 64, 512, 32000, 4096, 1000000.0, 1e-6, True, True),
    "tiny-qwen-128": ModelConfig("tiny-qwen-128", "llama", 2, 512, 4, 1, 128, 1024, 32000, 8192, 1000000.0, 1e-6,
                                 False, True),
    "tiny-gpt2": ModelConfig("tiny-gpt2", "gpt2", 2, 128, 2, 2, 64, 512, 32000, 2048, 0.0, 1e-5, True),
}


def parse_mupulorn(d: dict, name: str = "mupulorn") -> ModelConfig:
    """``config.json`` of a Mupulorn checkpoint -> :class:`ModelConfig`. Every size and every
    per-model constant comes from the file; a layer with ``weights_of`` runs another layer's tensors."""
    raw = d["layers"]
    specs = []
    for i, e in enumerate(raw):
        if e["type"] != "latent_attention":
            raise ValueError(f"{name}: layer {i}: unknown mixer type '{e['type']}'")
        src, seen = i, set()
        while "weights_of" in raw[src] and raw[src]["weights_of"] is not None:
            if src in seen:
                raise ValueError(f"{name}: layer {i}: weights_of forms a cycle")
            seen.add(src)
            src = int(raw[src]["weights_of"])
        mx = e["mixer"]
        rot = mx["rot"]
        m = LatentAttentionSpec(int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]),
                                int(mx["kv_rank"]), int(mx["q_rank"]), float(rot["base"]), int(rot["dims"]),
                                float(mx["scale"]))
        if m.rot_dims > m.rot_dim or m.rot_dims % 2:
            raise ValueError(f"{name}: layer {i}: rot.dims {m.rot_dims} does not fit rot_dim {m.rot_dim}")
        mlp = raw[src].get("mlp") if e.get("mlp", "absent") == "absent" else e.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"{name}: layer {i}: unknown feed-forward kind '{mlp['kind']}'")
        specs.append(LayerSpec("latent_attention", m, int(mlp["ff"]) if mlp is not None else 0, "dense", src))
    top = max(specs, key=lambda s: s.mixer.heads).mixer
    return ModelConfig(name, "mupulorn", len(specs), int(d["width"]), top.heads, 1, top.dim + top.rot_dim,
                       max(s.ff for s in specs), int(d["vocab"]), int(d.get("max_pos", 1 << 17)),
                       specs[0].mixer.rot_base, float(d["norm"]["eps"]), layers=tuple(specs),
                       canon_taps=int(d["canon"]["taps"]), logit_scale=float(d["logit_scale"]),
                       logit_softcap=float(d["logit_softcap"]))


def mupulorn_config(name: str, n_layers: int, width: int, heads: int, dim: int, rot_dim: int, vdim: int,
                    kv_rank: int, q_rank: int, ff: int, vocab: int, taps: int = 4, shared_every: int = 0,
                    rot_base: float = 10000.0, max_pos: int = 1 << 17) -> ModelConfig:
    """A uniform Mupulorn stack from a few sizes (benchmarks and presets). ``shared_every`` n > 0:
    layers n*k+1 .. n*k+n-1 run layer n*k's weights."""
    layer = {"type": "latent_attention",
             "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                       "q_rank": q_rank, "rot": {"base": rot_base, "dims": rot_dim},
                       "scale": (dim + rot_dim) ** -0.5},
             "mlp": {"kind": "dense", "ff": ff} if ff else None}
    layers = []
    for i in range(n_layers):
        e = dict(layer)
        if shared_every > 0 and i % shared_every:
            e["weights_of"] = i - i % shared_every
        layers.append(e)
    return parse_mupulorn({"architecture": "Mupulorn", "canon": {"taps": taps}, "layers": layers,
                           "logit_scale": 1.0, "logit_softcap": 30.0, "norm": {"eps": 1e-5}, "vocab": vocab,
                           "width": width, "max_pos": max_pos}, name)


# config.json "architecture" -> parser (checkpoint directories name their own model class)
ARCHITECTURES: Dict[str, Callable[[dict, str], ModelConfig]] = {"Mupulorn": parse_mupulorn}

PRESETS.update({
    # Mupulorn (latent attention + input convolutions + PolyNorm feed-forward), random-init sizes:
    # a test-sized stack and three whose layers have the shapes of 1B / 3B / 8B-class models
    "tiny-mupulorn": mupulorn_config("tiny-mupulorn", 3, 128, 4, 32, 16, 32, 64, 48, 256, 32000, taps=4,
                                     shared_every=2),
    # (the two-matrix feed-forward is 1.5x as wide as the gated three-matrix one of the Llama preset
    # of the same class, so a layer holds about the same weights)
    "mupulorn-1b": mupulorn_config("mupulorn-1b", 16, 2048, 16, 128, 64, 128, 512, 768, 12288, 128256),
    "mupulorn-3b": mupulorn_config("mupulorn-3b", 28, 3072, 24, 128, 64, 128, 256, 1024, 12288, 128256),
    "mupulorn-8b": mupulorn_config("mupulorn-8b", 32, 4096, 32, 128, 64, 128, 512, 1536, 21504, 128256),
})


def config_from_dir(path: str) -> ModelConfig:
    """The model a checkpoint directory declares in its ``config.json`` (key ``architecture``)."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch not in ARCHITECTURES:
        raise KeyError(f"{path}/config.json: unknown architecture {arch!r} (known: {', '.join(ARCHITECTURES)})")
    return ARCHITECTURES[arch](d, os.path.basename(os.path.normpath(path)) or arch.lower())


def get_config(name: str, **overrides) -> ModelConfig:
    if name not in PRESETS and os.path.isfile(os.path.join(name, "config.json")):
        cfg = config_from_dir(name)
        return replace(cfg, **overrides) if overrides else cfg
    if name not in PRESETS:
        raise KeyError(f"unknown model preset '{name}' (known: {', '.join(PRESETS)})")
    cfg = PRESETS[name]
    if isinstance(overrides.get("rope_scaling"), list):   # from a JSON config
        overrides = dict(overrides, rope_scaling=tuple(overrides["rope_scaling"]))
    return replace(cfg, **overrides) if overrides else cfg
