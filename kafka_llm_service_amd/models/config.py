"""Model architecture configs (public HF configs of the benchmark models; random-init weights)."""
from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field
from pathlib import Path


@dataclass
class ModelConfig:
    name: str
    arch: str = "llama"  # "llama" | "mixtral"
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    # MoE
    num_experts: int = 0
    num_experts_per_tok: int = 0
    # special tokens (Llama-3 family ids; Mixtral uses its own)
    bos_token_id: int = 128000
    eos_token_ids: list[int] = field(default_factory=lambda: [128001, 128008, 128009])

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        d, f, L, V = self.hidden_size, self.intermediate_size, self.num_layers, self.vocab_size
        attn = d * (self.q_size + 2 * self.kv_size) + self.q_size * d
        if self.num_experts:
            mlp = self.num_experts * 3 * d * f + d * self.num_experts
        else:
            mlp = 3 * d * f
        emb = V * d * (1 if self.tie_word_embeddings else 2)
        return L * (attn + mlp + 2 * d) + emb + d

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    def to_json(self) -> str:
        return json.dumps(asdict(self))

    @staticmethod
    def from_hf(path: str | Path) -> "ModelConfig":
        """Build from a HF ``config.json`` (for loading real safetensors checkpoints when available)."""
        c = json.loads(Path(path).read_text())
        arch = "mixtral" if c.get("num_local_experts") else "llama"
        eos = c.get("eos_token_id", 2)
        return ModelConfig(
            name=c.get("_name_or_path", Path(path).parent.name), arch=arch, hidden_size=c["hidden_size"],
            intermediate_size=c["intermediate_size"], num_layers=c["num_hidden_layers"],
            num_heads=c["num_attention_heads"], num_kv_heads=c.get("num_key_value_heads", c["num_attention_heads"]),
            head_dim=c.get("head_dim", c["hidden_size"] // c["num_attention_heads"]), vocab_size=c["vocab_size"],
            rms_norm_eps=c.get("rms_norm_eps", 1e-5), rope_theta=c.get("rope_theta", 10000.0),
            rope_scaling=c.get("rope_scaling"), max_position_embeddings=c.get("max_position_embeddings", 8192),
            tie_word_embeddings=c.get("tie_word_embeddings", False), num_experts=c.get("num_local_experts", 0),
            num_experts_per_tok=c.get("num_experts_per_tok", 0), bos_token_id=c.get("bos_token_id", 1),
            eos_token_ids=eos if isinstance(eos, list) else [eos])


LLAMA31_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                   "original_max_position_embeddings": 8192}

PRESETS: dict[str, ModelConfig] = {
    # Llama-3-8B shapes with Llama-3.1 RoPE scaling: the ~18k-token Kafka prompt exceeds 8k.
    "llama3-8b": ModelConfig(name="llama3-8b", rope_scaling=LLAMA31_SCALING, max_position_embeddings=131072),
    "llama3-8b-8k": ModelConfig(name="llama3-8b-8k"),
    "llama3-70b": ModelConfig(name="llama3-70b", hidden_size=8192, intermediate_size=28672, num_layers=80,
                              num_heads=64, num_kv_heads=8, rope_scaling=LLAMA31_SCALING,
                              max_position_embeddings=131072),
    "mixtral-8x7b": ModelConfig(name="mixtral-8x7b", arch="mixtral", vocab_size=32000, rope_theta=1e6,
                                max_position_embeddings=32768, num_experts=8, num_experts_per_tok=2,
                                bos_token_id=1, eos_token_ids=[2]),
    # small configs with the same head geometry (head_dim 128, GQA) for tests and smoke runs
    "tiny-llama": ModelConfig(name="tiny-llama", hidden_size=512, intermediate_size=1024, num_layers=2,
                              num_heads=8, num_kv_heads=2, vocab_size=128256, max_position_embeddings=131072,
                              rope_scaling=LLAMA31_SCALING),
    "tiny-mixtral": ModelConfig(name="tiny-mixtral", arch="mixtral", hidden_size=512, intermediate_size=512,
                                num_layers=2, num_heads=8, num_kv_heads=2, vocab_size=32000, rope_theta=1e6,
                                max_position_embeddings=32768, num_experts=4, num_experts_per_tok=2,
                                bos_token_id=1, eos_token_ids=[2]),
    "small-llama": ModelConfig(name="small-llama", hidden_size=1024, intermediate_size=3584, num_layers=4,
                               num_heads=16, num_kv_heads=4, max_position_embeddings=131072,
                               rope_scaling=LLAMA31_SCALING),
}


def _budurax(width: int, heads: int, n_layers: int, vocab: int, ff: int, attn_every: int = 3) -> dict:
    """A Budurax config dict at transformer-like sizes: 128-dim heads with a 64-dim rotary part, latent rank 4 x the
    head size, every ``attn_every``-th layer latent attention (later ones borrow the first's cache), the rest Mamba-2."""
    rot = {"base": 500000.0, "dims": 64, "scaling": {"factor": 8.0, "original": 8192, "fast": 32.0, "slow": 1.0}}
    layers = []
    for i in range(n_layers):
        if i % attn_every == 0:
            m = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "rot": rot,
                 "scale": (128 + 64) ** -0.5}
            if i:
                m["kv_from"] = 0
            layers.append({"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff}})
        else:
            layers.append({"type": "mamba2", "mixer": {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 8,
                                                       "norm_groups": 8, "conv": 4},
                           "mlp": {"kind": "dense", "ff": ff}})
    return {"architecture": "Budurax", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": 1e-6},
            "token_side": {"dim": 64}}


BUDURAX_PRESETS: dict[str, dict] = {
    # sizes of the Llama presets below (same width, heads, depth, vocabulary and feed-forward), random init
    "budurax-8b-shape": _budurax(4096, 32, 32, 128256, 14336),
    "budurax-small": _budurax(1024, 16, 4, 128256, 3584),
    "budurax-tiny": _budurax(512, 8, 3, 32000, 1024),
}


def _lisorax(width: int, heads: int, kv_heads: int, n_layers: int, vocab: int, ff: int, experts: int = 8,
             top: int = 2) -> dict:
    """A Lisorax config dict at transformer-like sizes: 128-dim heads; layers cycle attention, rglru, attention that
    borrows the first attention layer's keys and values, mlstm; every layer with routed experts of ``ff`` rows."""
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    layers = []
    for i in range(n_layers):
        kind = i % 4
        if kind in (0, 2):
            m = {"heads": heads, "kv_heads": kv_heads, "dim": 128, "vdim": 128, "conv": 4, "scale": 128 ** -0.5,
                 "softcap": 50.0, "q_temp": {"coef": 0.25, "every": 4096}}
            if kind == 2:
                m["kv_from"] = i - 2
            layers.append({"type": "attention", "mixer": m, "mlp": moe})
        elif kind == 1:
            layers.append({"type": "rglru", "mixer": {"width": width, "blocks": max(1, width // 256), "conv": 4},
                           "mlp": moe})
        else:
            layers.append({"type": "mlstm", "mixer": {"heads": max(1, width // 256), "dim": 128, "vdim": 256,
                                                      "gate_cap": 10.0}, "mlp": moe})
    return {"architecture": "Lisorax", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "canon": {"taps": 4}}


LISORAX_PRESETS: dict[str, dict] = {
    # widths, heads and vocabularies of the Llama presets above; 8 experts of ff / 4 rows, top 2 (random init)
    "lisorax-small": _lisorax(1024, 16, 4, 4, 128256, 896),
    "lisorax-tiny": _lisorax(512, 8, 2, 4, 32000, 256, experts=4),
}


def _mozidra(width: int, heads: int, kv_heads: int, n_layers: int, vocab: int, ff: int, experts: int = 8,
             top: int = 2, streams: int = 4, attn_every: int = 3, window: int = 1024) -> dict:
    """A Mozidra config dict at transformer-like sizes: 128-dim heads; every ``attn_every``-th layer grouped-query
    attention with a full rotation and value mixing, the others latent attention (rank 512); sliding windows; every
    layer with group-routed experts of ``ff`` rows (4 groups, 2 kept) and a shared expert of the same size."""
    moe = {"kind": "moe", "expert": {"ff": ff, "limit": 7.0},
           "router": {"experts": experts, "top": top, "groups": {"count": 4 if experts % 4 == 0 else 1,
                                                                 "keep": 2 if experts % 4 == 0 else 1}},
           "shared": {"ff": ff, "limit": 7.0}}
    layers = []
    for i in range(n_layers):
        if i % attn_every == attn_every - 1:
            m = {"heads": heads, "kv_heads": kv_heads, "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                 "mask": {"size": 2 * window}, "rot": {"base": 500000.0, "dims": 128}, "v_mix": True}
            layers.append({"type": "attention", "mixer": m, "mlp": moe})
        else:
            m = {"heads": heads, "dim": 128, "vdim": 128, "kv_rank": 512, "scale": 128 ** -0.5,
                 "mask": {"size": window}}
            layers.append({"type": "latent_attention", "mixer": m, "mlp": moe})
    return {"architecture": "Mozidra", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": 1e-6},
            "streams": streams}


MOZIDRA_PRESETS: dict[str, dict] = {
    # widths, heads and vocabularies of the Llama presets above; 8 experts of ff / 4 rows, top 2 (random init)
    "mozidra-small": _mozidra(1024, 16, 4, 6, 128256, 896),
    "mozidra-tiny": _mozidra(512, 8, 2, 3, 32000, 256, experts=4, window=64),
}


def _magedra(width: int, heads: int, kv_heads: int, n_layers: int, vocab: int, ff: int, streams: int = 4,
             head_dim: int = 128) -> dict:
    """A Magedra config dict at transformer-like sizes: layers cycle latent attention (rank 512, rotated part 64,
    query rank 3 x the latent's), minGRU (as wide as the model), parallel (grouped-query attention with a head mix
    beside HGRN2 with ``width / 128`` heads of 64 x 128) and minGRU; every layer with a clamped dense feed-forward;
    the second half of the depth runs the first half's tensors when the depth is a multiple of 8."""
    mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
    kinds = []
    for i in range(n_layers):
        k = i % 4
        if k == 0:
            m = {"heads": heads, "dim": 128, "rot_dim": 64, "vdim": 128, "kv_rank": 512, "q_rank": 1536,
                 "rot": {"base": 500000.0, "dims": 64}, "scale": (128 + 64) ** -0.5}
            kinds.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
        elif k == 2:
            left = {"heads": heads, "kv_heads": kv_heads, "dim": head_dim, "vdim": head_dim,
                    "rot": {"base": 100000.0, "dims": head_dim // 2}, "scale": head_dim ** -0.5}
            right = {"heads": max(1, width // 128), "dim": 64, "vdim": 128}
            kinds.append({"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 0.7,
                                                        "right_scale": 0.6}, "mlp": mlp})
        else:
            kinds.append({"type": "mingru", "mixer": {"width": width}, "mlp": mlp})
    if n_layers % 8 == 0:
        half = n_layers // 2
        kinds = kinds[:half] + [dict(kinds[j], weights_of=j) for j in range(half)]
    return {"architecture": "Magedra", "vocab": vocab, "width": width, "layers": kinds, "norm": {"eps": 1e-6},
            "streams": streams, "residual_mult": 0.5, "logit_scale": 0.5}


MAGEDRA_PRESETS: dict[str, dict] = {
    # widths, heads and vocabularies of the Llama presets above (random init)
    "magedra-small": _magedra(1024, 16, 2, 8, 128256, 3584),
    "magedra-tiny": _magedra(512, 8, 2, 4, 32000, 1024, streams=2, head_dim=64),
}


def _budurax_config(c: dict, name: str):
    from kafka_llm_service_amd.models.budurax import BuduraxConfig

    return BuduraxConfig.from_dict(c, name=name)


def _lisorax_config(c: dict, name: str):
    from kafka_llm_service_amd.models.lisorax import LisoraxConfig

    return LisoraxConfig.from_dict(c, name=name)


def _mozidra_config(c: dict, name: str):
    from kafka_llm_service_amd.models.mozidra import MozidraConfig

    return MozidraConfig.from_dict(c, name=name)


def _magedra_config(c: dict, name: str):
    from kafka_llm_service_amd.models.magedra import MagedraConfig

    return MagedraConfig.from_dict(c, name=name)


# config.json "architecture" (lower case) -> config class of a model family that names itself there
ARCH_CONFIGS = {"budurax": _budurax_config, "lisorax": _lisorax_config, "mozidra": _mozidra_config,
                "magedra": _magedra_config}
# model families whose kernels are built for float32 as well as bfloat16 (EngineConfig.dtype)
FP32_ARCHS = ("budurax", "lisorax", "mozidra", "magedra")


def _from_json(path: Path):
    """A config.json names its model class: ``"architecture": "Budurax"`` (models/budurax.py), ``"Lisorax"``
    (models/lisorax.py), ``"Mozidra"`` (models/mozidra.py), ``"Magedra"`` (models/magedra.py), else HF Llama /
    Mixtral."""
    c = json.loads(path.read_text())
    make = ARCH_CONFIGS.get(str(c.get("architecture", "")).lower())
    if make is not None:
        return make(c, path.parent.name)
    return ModelConfig.from_hf(path)


def get_config(name: str):
    if name in PRESETS:
        return PRESETS[name]
    if name in BUDURAX_PRESETS:
        return _budurax_config(BUDURAX_PRESETS[name], name)
    if name in LISORAX_PRESETS:
        return _lisorax_config(LISORAX_PRESETS[name], name)
    if name in MOZIDRA_PRESETS:
        return _mozidra_config(MOZIDRA_PRESETS[name], name)
    if name in MAGEDRA_PRESETS:
        return _magedra_config(MAGEDRA_PRESETS[name], name)
    p = Path(name)
    if p.is_dir() and (p / "config.json").exists():
        return _from_json(p / "config.json")
    if p.suffix == ".json" and p.exists():
        return _from_json(p)
    raise KeyError(f"unknown model {name!r}; presets: {sorted(PRESETS) + sorted(BUDURAX_PRESETS) + sorted(LISORAX_PRESETS) + sorted(MOZIDRA_PRESETS) + sorted(MAGEDRA_PRESETS)}")
