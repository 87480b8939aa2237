"""Model architecture presets (public HF configs; SURVEY.md §2.4 'Model constants').

The reference has no model code at all — its model is remote (`/root/reference/app.py:117`).
These are the architectures BASELINE.json names for the on-node engine, plus tiny variants of the
same shape family used by CPU tests and GPU numerics tests.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Dict, Optional, Tuple


@dataclasses.dataclass(frozen=True)
class ModelConfig:
    name: str
    family: str                 # "llama" | "mixtral"
    num_layers: int
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate: int
    vocab_size: int
    rope_theta: float
    norm_eps: float = 1e-5
    max_position: int = 8192
    num_experts: int = 0        # mixtral
    top_k: int = 0
    tie_embeddings: bool = False
    tokenizer: str = "llama3"   # "llama3" | "llama2"

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    def num_params(self) -> int:
        h, i, v = self.hidden, self.intermediate, self.vocab_size
        attn = h * self.qkv_size + self.q_size * h
        mlp = 3 * h * i * (self.num_experts if self.is_moe else 1) + (h * self.num_experts if self.is_moe else 0)
        per_layer = attn + mlp + 2 * h
        return self.num_layers * per_layer + v * h * (1 if self.tie_embeddings else 2) + h

    def default_step_tokens(self) -> int:
        """Engine token budget per step when MAX_NUM_BATCHED_TOKENS is 0 (auto).  Each step streams
        every weight once, so a step has a fixed cost that grows with the model: for an 8B model a
        256-request wave's ~8k prompt tokens are best split over ~3 mixed steps that also carry the
        running decodes (4096: 1243-1273 vs 1109-1122 req/s at 16384), while Mixtral-8x7B and
        Llama-3-70B do better with the wave's prompt in one step (16384: 269 vs 252 and 102 vs 91
        req/s; profiles/r2/budget/)."""
        return 4096 if self.num_params() * 2 < (40 << 30) else 16384

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return self.num_layers * 2 * self.kv_size * dtype_bytes


@dataclasses.dataclass(frozen=True)
class AttentionSpec:
    """One attention mixer of a per-layer-configured model (the `mixer` entry of a Vivepel layer)."""
    heads: int
    kv_heads: int
    dim: int                    # per-head query / key size
    vdim: int                   # per-head value size (the values are the projected keys: vdim == dim)
    chunk: int                  # chunked causal mask: position p sees floor(p / chunk) * chunk .. p (0: all of 0 .. p)
    rot_dims: int               # rotary positions on the first rot_dims entries of each head
    rot_base: float
    scale: float
    softcap: float

    @classmethod
    def from_dict(cls, m: dict) -> "AttentionSpec":
        mask, rot, cap = m.get("mask"), m.get("rot"), m.get("softcap")
        spec = cls(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                   chunk=int(mask["size"]) if mask else 0,            # no mask entry: plain causal
                   rot_dims=int(rot["dims"]) if rot else 0,           # no rot entry: no rotary positions
                   rot_base=float(rot["base"]) if rot else 1.0,
                   scale=float(m["scale"]), softcap=float(cap) if cap else 0.0)   # no softcap: scores as they are
        if spec.heads % spec.kv_heads:
            raise ValueError(f"heads {spec.heads} must be a multiple of kv_heads {spec.kv_heads}")
        if spec.vdim != spec.dim:
            raise ValueError(f"vdim {spec.vdim} != dim {spec.dim}: the values are the projected keys")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim or spec.chunk < 0:
            raise ValueError(f"bad rotary dims {spec.rot_dims} / chunk {spec.chunk} for head size {spec.dim}")
        return spec


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    mixer: AttentionSpec
    ff: int = 0                 # dense feed-forward width; 0: the layer has no feed-forward


@dataclasses.dataclass(frozen=True)
class VivepelConfig:
    """Vivepel: a decoder whose layers are listed one by one in its config.json.  Every layer is
    x += ls1 * gnorm(mixer(gnorm(x))), then (if it has one) x += ls2 * gnorm(ff(gnorm(x))), with RMS
    norms in `norm_groups` groups; the mixer is chunk-masked attention (AttentionSpec), the
    feed-forward is up -> PolyNorm -> down.  The residual stream is fp32."""
    name: str
    vocab_size: int
    hidden: int
    norm_eps: float
    norm_groups: int
    layers: Tuple[LayerSpec, ...]
    max_position: int = 1 << 20
    tokenizer: str = "llama3"
    family: str = "vivepel"
    tie_embeddings: bool = False
    is_moe: bool = False

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, name: str = "vivepel") -> "VivepelConfig":
        layers = []
        for i, L in enumerate(d["layers"]):
            if L["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerSpec(AttentionSpec.from_dict(L["mixer"]), int(mlp["ff"]) if mlp is not None else 0))
        cfg = cls(name=name, vocab_size=int(d["vocab"]), hidden=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  norm_groups=int(d["norm"]["groups"]), layers=tuple(layers))
        if cfg.hidden % cfg.norm_groups:
            raise ValueError(f"width {cfg.hidden} is not a multiple of norm groups {cfg.norm_groups}")
        return cfg

    def to_dict(self) -> dict:
        """The config.json form (what `from_dict` reads)."""
        return {"architecture": "Vivepel", "vocab": self.vocab_size, "width": self.hidden,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                "layers": [{"type": "attention",
                            "mixer": {"heads": L.mixer.heads, "kv_heads": L.mixer.kv_heads, "dim": L.mixer.dim,
                                      "vdim": L.mixer.vdim, "mask": {"size": L.mixer.chunk} if L.mixer.chunk else None,
                                      "rot": {"base": L.mixer.rot_base, "dims": L.mixer.rot_dims},
                                      "scale": L.mixer.scale, "softcap": L.mixer.softcap},
                            "mlp": {"kind": "dense", "ff": L.ff} if L.ff else None} for L in self.layers]}

    def num_params(self) -> int:
        h = self.hidden
        n = 2 * self.vocab_size * h + h
        for L in self.layers:
            m = L.mixer
            n += (m.heads + m.kv_heads) * m.dim * (h + 1) + m.heads * m.vdim * h + m.heads * m.heads + 2 * m.dim + 3 * h
            if L.ff:
                n += 2 * h * L.ff + 4 + 3 * h
        return n

    def default_step_tokens(self) -> int:
        """16384: the tile attention kernel runs one workgroup per 16 query rows and CU, longest first; a
        step needs several times 256 of them for the causal tiles' unequal lengths to even out."""
        return 16384

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(2 * L.mixer.kv_heads * L.mixer.dim * dtype_bytes for L in self.layers)


def vivepel_uniform(name: str, layers: int, hidden: int, heads: int, kv_heads: int, dim: int, ff: int, vocab: int,
                    chunk: int = 1024, rot_dims: Optional[int] = None, groups: int = 4) -> VivepelConfig:
    """A Vivepel configuration whose layers are all alike (benchmarks, tests)."""
    spec = AttentionSpec(heads, kv_heads, dim, dim, chunk, rot_dims if rot_dims is not None else dim // 2, 10000.0,
                         dim ** -0.5, 30.0)
    return VivepelConfig(name, vocab, hidden, 1e-6, groups, tuple(LayerSpec(spec, ff) for _ in range(layers)))


# config.json "architecture" -> parser of the file's dict
ARCHITECTURES = {"Vivepel": VivepelConfig.from_dict}


def load_config_dir(path: str):
    """The configuration of a checkpoint folder (config.json + model.safetensors), by its architecture."""
    with open(os.path.join(path, "config.json")) as f:
        d = json.load(f)
    arch = d.get("architecture")
    if arch not in ARCHITECTURES:
        raise ValueError(f"{path}/config.json: unknown architecture {arch!r}; known: {sorted(ARCHITECTURES)}")
    return ARCHITECTURES[arch](d, name=os.path.basename(os.path.normpath(path)) or arch.lower())


PRESETS: Dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig("llama3-8b", "llama", 32, 4096, 32, 8, 128, 14336, 128256, 500000.0),
    "llama3-70b": ModelConfig("llama3-70b", "llama", 80, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    "mixtral-8x7b": ModelConfig("mixtral-8x7b", "mixtral", 32, 4096, 32, 8, 128, 14336, 32000, 1e6,
                                max_position=32768, num_experts=8, top_k=2, tokenizer="llama2"),
    # Same shape family, small enough for CPU tests (fp32 reference) and quick GPU numerics.
    "tiny-llama": ModelConfig("tiny-llama", "llama", 2, 256, 4, 2, 64, 512, 128256, 500000.0),
    "tiny-mixtral": ModelConfig("tiny-mixtral", "mixtral", 2, 256, 4, 2, 64, 384, 32000, 1e6, num_experts=4,
                                top_k=2, tokenizer="llama2"),
    # GPU test model with the real head geometry (head_dim 128, GQA 4) but few layers.
    "llama3-8b-2l": ModelConfig("llama3-8b-2l", "llama", 2, 4096, 32, 8, 128, 14336, 128256, 500000.0),
    # Llama-3-70B geometry (8 KV heads: 1 per rank at TP = 8, GQA group 8) with 2 layers: TP = 4 / 8
    # numerics on one GPU (tests/virtual_tp.py, tests/test_tp_single_gpu.py)
    "llama3-70b-2l": ModelConfig("llama3-70b-2l", "llama", 2, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    # 8 layers of Llama-3-70B: timing a TP group's decode step on one GPU (scripts/bench_tp_persistent_2rank.py)
    "llama3-70b-8l": ModelConfig("llama3-70b-8l", "llama", 8, 8192, 64, 8, 128, 28672, 128256, 500000.0),
    # Llama-3-70B head layout (64 q / 8 kv heads: GQA 8, one KV head per rank at TP = 8) on small
    # layers: CPU multi-process TP = 8 serving tests (gloo), where the 8192-wide layers would not fit
    "llama3-70b-tiny": ModelConfig("llama3-70b-tiny", "llama", 2, 2048, 64, 8, 32, 1024, 128256, 500000.0),
    "mixtral-2l": ModelConfig("mixtral-2l", "mixtral", 2, 4096, 32, 8, 128, 14336, 32000, 1e6, max_position=32768,
                              num_experts=8, top_k=2, tokenizer="llama2"),
    # Vivepel at small sizes (CPU tests) and at the layer sizes of Llama-3-8B (bench.py --arch-compare)
    "tiny-vivepel": vivepel_uniform("tiny-vivepel", 2, 128, 4, 2, 32, 192, 384, chunk=16, rot_dims=12, groups=2),
    "vivepel-8b-2l": vivepel_uniform("vivepel-8b-2l", 2, 4096, 32, 8, 128, 14336, 128256),
    "vivepel-8b": vivepel_uniform("vivepel-8b", 32, 4096, 32, 8, 128, 14336, 128256),
}


def get_config(name: str):
    """A preset by name, or a checkpoint folder (its config.json names the architecture)."""
    if name in PRESETS:
        return PRESETS[name]
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return load_config_dir(name)
    raise ValueError(f"unknown MODEL {name!r}; choose from {sorted(PRESETS)} or give a checkpoint folder")
