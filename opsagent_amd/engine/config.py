"""Model architecture registry.

Llama-3 family dims (8B / 70B per BASELINE.json configs #2-#4), a tiny config
for CPU tests, and DeepSeek-V3-style MoE configs (BASELINE config #5). Random
initialization is the benchmark mode (no network for checkpoints); safetensors
loading is supported for real weights.
"""

from __future__ import annotations

import dataclasses
from typing import List, Optional


@dataclasses.dataclass
class ModelSpec:
    name: str
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    rope_theta: float = 500000.0
    rms_eps: float = 1e-5
    max_seq_len: int = 8192
    tie_embeddings: bool = False
    # MoE (None => dense MLP)
    moe_num_experts: Optional[int] = None
    moe_top_k: int = 2
    moe_intermediate_size: Optional[int] = None
    moe_shared_experts: int = 0
    moe_dtype: str = "bf16"  # "fp8" enables the CDNA4 fp8 expert GEMM path

    is_hybrid = False

    @property
    def is_moe(self) -> bool:
        return self.moe_num_experts is not None


MODEL_REGISTRY = {
    # Llama-3 8B (BASELINE configs #2/#3)
    "llama3-8b": ModelSpec(
        name="llama3-8b",
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=32,
        num_heads=32,
        num_kv_heads=8,
    ),
    # Llama-3 70B (BASELINE config #4, TP=8)
    "llama3-70b": ModelSpec(
        name="llama3-70b",
        hidden_size=8192,
        intermediate_size=28672,
        num_layers=80,
        num_heads=64,
        num_kv_heads=8,
    ),
    # tiny model for CPU tests (vocab covers the byte tokenizer's ~260 ids)
    "llama3-tiny": ModelSpec(
        name="llama3-tiny",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=32,
        max_seq_len=512,
    ),
    # tiny model whose head/vocab geometry divides by 4 (CPU world=4 TP tests)
    "llama3-tiny-w4": ModelSpec(
        name="llama3-tiny-w4",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=8,
        num_kv_heads=4,
        head_dim=16,
        max_seq_len=512,
    ),
    # GPU-smoke-sized model (real head_dim for the HIP kernels)
    "llama3-micro": ModelSpec(
        name="llama3-micro",
        vocab_size=2048,
        hidden_size=1024,
        intermediate_size=2816,
        num_layers=4,
        num_heads=8,
        num_kv_heads=2,
        head_dim=128,
        max_seq_len=4096,
    ),
    # 8B-class projection shapes at 2 layers: exercises the K=4096 MFMA
    # GEMV paths (fp8 and bf16) end-to-end without an 8B weight build
    "llama3-2l4k": ModelSpec(
        name="llama3-2l4k",
        vocab_size=2048,
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=2,
        num_heads=32,
        num_kv_heads=8,
        head_dim=128,
        max_seq_len=4096,
    ),
    # tiny MoE for CPU tests
    "moe-tiny": ModelSpec(
        name="moe-tiny",
        vocab_size=512,
        hidden_size=128,
        intermediate_size=256,
        num_layers=2,
        num_heads=4,
        num_kv_heads=2,
        head_dim=32,
        max_seq_len=512,
        moe_num_experts=8,
        moe_top_k=2,
        moe_intermediate_size=64,
        moe_shared_experts=1,
    ),
    # GPU-smoke-sized MoE (real head_dim, fp8-capable expert shapes)
    "moe-micro": ModelSpec(
        name="moe-micro",
        vocab_size=2048,
        hidden_size=1024,
        intermediate_size=2816,
        num_layers=4,
        num_heads=8,
        num_kv_heads=2,
        head_dim=128,
        max_seq_len=4096,
        moe_num_experts=16,
        moe_top_k=4,
        moe_intermediate_size=512,
        moe_shared_experts=1,
    ),
    # DeepSeek-V3-style MoE, scaled down to fit one MI355X comfortably
    # (BASELINE config #5: fp8 experts on CDNA4 MFMA)
    "deepseek-moe-small": ModelSpec(
        name="deepseek-moe-small",
        vocab_size=128256,
        hidden_size=2048,
        intermediate_size=8192,       # dense MLP for the first layer(s)
        num_layers=12,
        num_heads=16,
        num_kv_heads=4,
        moe_num_experts=64,
        moe_top_k=6,
        moe_intermediate_size=1408,
        moe_shared_experts=2,
    ),
    "deepseek-moe": ModelSpec(
        name="deepseek-moe",
        vocab_size=128256,
        hidden_size=4096,
        intermediate_size=14336,
        num_layers=28,
        num_heads=32,
        num_kv_heads=8,
        moe_num_experts=128,
        moe_top_k=8,
        moe_intermediate_size=2048,
        moe_shared_experts=1,
    ),
}


def get_model_spec(name):
    """A registry name, a checkpoint folder, or an already-built spec."""
    import os

    if not isinstance(name, str):
        return name
    if name in HYBRID_REGISTRY:
        return povazen_spec_from_dict(HYBRID_REGISTRY[name](), name=name)
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return load_spec_from_dir(name)
    if name not in MODEL_REGISTRY:
        raise KeyError(f"unknown model {name!r}; known: {sorted(MODEL_REGISTRY)}")
    return MODEL_REGISTRY[name]


# ---------------------------------------------------------------------------
# Hybrid designs: a per-layer list of mixers (softmax attention, recurrent
# delta rule, ...) read from a checkpoint folder's config.json. Every size
# and every constant that can differ between checkpoints lives in the spec;
# nothing is taken from a particular checkpoint.


@dataclasses.dataclass
class MixerSpec:
    """One layer's token mixer. kind: "attention" | "channel_delta"."""

    kind: str
    heads: int
    kv_heads: int
    dim: int                      # per-head query/key size
    vdim: int                     # per-head value size
    scale: Optional[float] = None  # attention score scale
    conv: int = 0                 # short-convolution taps (recurrent mixers)
    # inner sizes of the low-rank decay / output-gate projections; only the
    # checkpoint's tensor shapes give them (None => the mixer's default)
    decay_rank: Optional[int] = None
    gate_rank: Optional[int] = None

    @property
    def has_kv(self) -> bool:
        return self.kind == "attention"

    @property
    def has_state(self) -> bool:
        return self.kind == "channel_delta"


@dataclasses.dataclass
class HybridLayerSpec:
    mixer: MixerSpec
    mlp_kind: Optional[str] = None   # None => the layer has no feed-forward
    mlp_ff: int = 0


@dataclasses.dataclass
class HybridSpec:
    """Architecture of a hybrid decoder (the Povazen design)."""

    name: str
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: List[HybridLayerSpec]
    norm_eps: float
    norm_groups: int
    canon_taps: int
    logit_softcap: float
    max_seq_len: int = 1 << 20
    weights_path: Optional[str] = None

    is_moe = False
    is_hybrid = True

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def povazen_spec_from_dict(cfg: dict, name: str = "povazen") -> HybridSpec:
    """Parse a Povazen config.json dict."""
    layers = []
    for entry in cfg["layers"]:
        m = entry["mixer"]
        kind = entry["type"]
        if kind not in ("attention", "channel_delta"):
            raise ValueError(f"unknown Povazen layer type {kind!r}")
        mixer = MixerSpec(
            kind=kind,
            heads=int(m["heads"]),
            kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]),
            vdim=int(m["vdim"]),
            scale=float(m["scale"]) if "scale" in m else None,
            conv=int(m.get("conv", 0)),
        )
        if mixer.heads % mixer.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind") != "dense":
            raise ValueError(f"unknown Povazen feed-forward kind {mlp.get('kind')!r}")
        layers.append(
            HybridLayerSpec(
                mixer=mixer,
                mlp_kind=None if mlp is None else "dense",
                mlp_ff=0 if mlp is None else int(mlp["ff"]),
            )
        )
    width = int(cfg["width"])
    groups = int(cfg["norm"]["groups"])
    if width % groups:
        raise ValueError("width must be a multiple of norm.groups")
    return HybridSpec(
        name=name,
        architecture="Povazen",
        vocab_size=int(cfg["vocab"]),
        hidden_size=width,
        layers=layers,
        norm_eps=float(cfg["norm"]["eps"]),
        norm_groups=groups,
        canon_taps=int(cfg["canon"]["taps"]),
        logit_softcap=float(cfg["logit_softcap"]),
    )


def povazen_config_dict(
    vocab: int, width: int, pattern: str, heads: int, kv_heads: int, dim: int,
    vdim: int, ff: int, delta_heads: Optional[int] = None, conv: int = 4,
    taps: int = 3, groups: int = 4, eps: float = 1e-6, softcap: float = 30.0,
) -> dict:
    """A Povazen config.json dict from a layer pattern: 'D' = channel_delta
    layer without feed-forward, 'd' = with one, 'A'/'a' likewise attention."""
    layers = []
    for ch in pattern:
        mlp = {"kind": "dense", "ff": ff} if ch.islower() else None
        if ch in "Aa":
            mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                     "vdim": vdim, "scale": dim ** -0.5}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        else:
            dh = delta_heads or heads
            mixer = {"heads": dh, "kv_heads": dh, "dim": dim, "vdim": vdim, "conv": conv}
            layers.append({"type": "channel_delta", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Povazen", "canon": {"taps": taps}, "layers": layers,
            "logit_softcap": softcap, "norm": {"eps": eps, "groups": groups},
            "vocab": vocab, "width": width}


# config.json "architecture" -> parser
ARCHITECTURE_PARSERS = {"Povazen": povazen_spec_from_dict}

# named hybrid configurations (random-weight benchmarking and tests)
HYBRID_REGISTRY = {
    # CPU-test size
    "povazen-tiny": lambda: povazen_config_dict(
        vocab=512, width=64, pattern="Dad", heads=4, kv_heads=2, dim=16, vdim=8,
        ff=128, delta_heads=2),
    # GPU-smoke size
    "povazen-micro": lambda: povazen_config_dict(
        vocab=2048, width=1024, pattern="DdaD", heads=8, kv_heads=2, dim=128,
        vdim=128, ff=2816, delta_heads=8),
    # layer shapes of an ~8B-class model at 4 layers (speed measurements
    # beside llama3 layers of equal width)
    "povazen-4l4k": lambda: povazen_config_dict(
        vocab=2048, width=4096, pattern="dada", heads=32, kv_heads=8, dim=128,
        vdim=128, ff=14336, delta_heads=32),
}


def load_spec_from_dir(path: str):
    """Model spec from a checkpoint folder (config.json + model.safetensors);
    the model class follows config.json's "architecture"."""
    import json
    import os

    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    arch = cfg.get("architecture")
    if arch not in ARCHITECTURE_PARSERS:
        raise KeyError(
            f"unknown architecture {arch!r} in {path}/config.json; "
            f"known: {sorted(ARCHITECTURE_PARSERS)}"
        )
    spec = ARCHITECTURE_PARSERS[arch](cfg, name=os.path.basename(os.path.normpath(path)))
    spec.weights_path = os.path.join(path, "model.safetensors")
    if os.path.exists(spec.weights_path):
        apply_tensor_shapes(spec, safetensors_shapes(spec.weights_path))
    return spec


def apply_tensor_shapes(spec: HybridSpec, shapes: dict) -> HybridSpec:
    """Fill the sizes that only tensor shapes give (name -> shape): the inner
    ranks of the low-rank decay and output-gate projections."""
    for i, layer in enumerate(spec.layers):
        a1, g1 = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.g1")
        if a1 is not None:
            layer.mixer.decay_rank = int(a1[0])
        if g1 is not None:
            layer.mixer.gate_rank = int(g1[0])
    return spec


def safetensors_shapes(path: str) -> dict:
    """name -> shape from a safetensors header (8-byte little-endian length,
    then that many bytes of JSON); reads no tensor data."""
    import json
    import struct

    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
    return {k: tuple(v["shape"]) for k, v in header.items() if k != "__metadata__"}
