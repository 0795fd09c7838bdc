"""The typed configuration of the Katenex decoder, read from its own config.json.

config.json gives every size and every constant that differs between models of the design: `vocab`, `width`,
`streams` (copies of the residual stream that the layers read from and write to through learned weights),
`embedding.scale`, `norm.eps`, and `layers`: per layer its `type` ("parallel": softmax attention beside a gated
linear recurrence; "channel_delta": the gated delta rule with a decay per key channel), the `mixer`'s sizes and
its `mlp` (a mixture of experts, or null for none).  Nothing here has a default but what may be absent.
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, ClassVar

from .model import ArchitectureConfig, ConfigError, KeyReader


@dataclass(frozen=True)
class KatenexRotary:
    base: float
    dims: int
    factor: float | None  # linear scaling: every frequency divided by it


@dataclass(frozen=True)
class KatenexAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: KatenexRotary | None


@dataclass(frozen=True)
class KatenexRecurrence:
    width: int
    blocks: int
    conv: int


@dataclass(frozen=True)
class KatenexParallelMixer:
    left: KatenexAttention
    right: KatenexRecurrence
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class KatenexDeltaMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    # the inner sizes of the two low-rank products (decay and output gate): config.json may give them; when it does
    # not, they are the shapes of the folder's `a1` and `g1` tensors
    decay_rank: int | None = None
    gate_rank: int | None = None


@dataclass(frozen=True)
class KatenexExperts:
    experts: int
    top: int
    scale: float
    groups: int
    keep: int
    expert_ff: int
    shared_ff: int | None


@dataclass(frozen=True)
class KatenexLayer:
    type: str  # "parallel" | "channel_delta"
    mixer: KatenexParallelMixer | KatenexDeltaMixer
    mlp: KatenexExperts | None


def _mapping(value: Any, where: str) -> dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"{where} must be a mapping, got {value!r}")
    return value


def _read_attention(values: dict[str, Any], where: str) -> KatenexAttention:
    reader = KeyReader(values, where)
    heads = reader.integer("heads")
    rot = None
    if values.get("rot"):
        rot_reader = KeyReader(_mapping(values["rot"], f"{where}.rot"), f"{where}.rot")
        factor = None
        if rot_reader.optional("scaling"):
            scaling = KeyReader(_mapping(values["rot"]["scaling"], f"{where}.rot.scaling"), f"{where}.rot.scaling")
            factor = scaling.number("factor")
        rot = KatenexRotary(rot_reader.number("base"), rot_reader.integer("dims", minimum=2), factor)
    dim = reader.integer("dim")
    return KatenexAttention(
        heads=heads, kv_heads=reader.integer("kv_heads", default=heads), dim=dim, vdim=reader.integer("vdim", default=dim),
        scale=reader.number("scale"), rot=rot,
    )


def _read_mixer(kind: str, values: dict[str, Any], where: str):
    reader = KeyReader(values, where)
    if kind == "parallel":
        right = KeyReader(_mapping(values.get("right"), f"{where}.right"), f"{where}.right")
        return KatenexParallelMixer(
            left=_read_attention(_mapping(values.get("left"), f"{where}.left"), f"{where}.left"),
            right=KatenexRecurrence(right.integer("width"), right.integer("blocks"), right.integer("conv")),
            left_scale=reader.number("left_scale"), right_scale=reader.number("right_scale"),
        )
    heads = reader.integer("heads")
    return KatenexDeltaMixer(
        heads=heads, kv_heads=reader.integer("kv_heads", default=heads), dim=reader.integer("dim"), vdim=reader.integer("vdim"),
        conv=reader.integer("conv"), decay_rank=reader.integer("decay_rank", default=None) if values.get("decay_rank") is not None else None,
        gate_rank=reader.integer("gate_rank", default=None) if values.get("gate_rank") is not None else None,
    )


def _read_mlp(values: Any, where: str) -> KatenexExperts | None:
    if values is None:
        return None
    reader = KeyReader(_mapping(values, where), where)
    reader.choice("kind", choices=("moe",), default="moe")
    router = KeyReader(_mapping(values.get("router"), f"{where}.router"), f"{where}.router")
    expert = KeyReader(_mapping(values.get("expert"), f"{where}.expert"), f"{where}.expert")
    groups, keep = 1, 1
    if router.optional("groups"):
        grouping = KeyReader(_mapping(values["router"]["groups"], f"{where}.router.groups"), f"{where}.router.groups")
        groups, keep = grouping.integer("count"), grouping.integer("keep")
    shared = values.get("shared")
    shared_ff = KeyReader(_mapping(shared, f"{where}.shared"), f"{where}.shared").integer("ff") if shared else None
    return KatenexExperts(
        experts=router.integer("experts"), top=router.integer("top"), scale=router.number("scale"), groups=groups, keep=keep,
        expert_ff=expert.integer("ff"), shared_ff=shared_ff,
    )


@dataclass(frozen=True)
class KatenexConfig(ArchitectureConfig):
    architecture: ClassVar[str] = "Katenex"

    vocab: int
    width: int
    streams: int | None  # copies of the residual stream; None: one stream with the plain residual sum (no link tensors)
    embedding_scale: float
    norm_eps: float
    layers: tuple[KatenexLayer, ...]

    def __post_init__(self) -> None:
        if not self.layers:
            raise ConfigError("Katenex config: no layers")
        for index, layer in enumerate(self.layers):
            where = f"Katenex config: layer {index}"
            mixer = layer.mixer
            if isinstance(mixer, KatenexDeltaMixer) and mixer.heads % mixer.kv_heads:
                raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
            if isinstance(mixer, KatenexParallelMixer):
                left, right = mixer.left, mixer.right
                if left.heads % left.kv_heads:
                    raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
                if left.rot is not None and (left.rot.dims % 2 or left.rot.dims > left.dim):
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
                if right.width % right.blocks:
                    raise ConfigError(f"{where}: the recurrence's width must be a multiple of its blocks")
            mlp = layer.mlp
            if mlp is not None:
                if mlp.experts % mlp.groups or not 0 < mlp.keep <= mlp.groups:
                    raise ConfigError(f"{where}: the experts form equal groups, of which between one and all are kept")
                if mlp.top > mlp.keep * (mlp.experts // mlp.groups):
                    raise ConfigError(f"{where}: more experts a token than the kept groups hold")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "KatenexConfig":
        reader = KeyReader(values, "Katenex config")
        norm = KeyReader(_mapping(values.get("norm"), "Katenex config: norm"), "Katenex config: norm")
        embedding = KeyReader(_mapping(values.get("embedding") or {}, "Katenex config: embedding"), "Katenex config: embedding")
        entries = values.get("layers")
        if not isinstance(entries, list):
            raise ConfigError("Katenex config: 'layers' must be a list")
        layers = []
        for index, entry in enumerate(entries):
            where = f"Katenex config: layers[{index}]"
            entry = _mapping(entry, where)
            kind = KeyReader(entry, where).choice("type", choices=("parallel", "channel_delta"))
            mixer = _read_mixer(kind, _mapping(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer")
            layers.append(KatenexLayer(kind, mixer, _read_mlp(entry.get("mlp"), f"{where}.mlp")))
        return cls(
            vocab=reader.integer("vocab"), width=reader.integer("width"), streams=reader.integer("streams", minimum=1) if values.get("streams") is not None else None,
            embedding_scale=embedding.number("scale", default=1.0), norm_eps=norm.number("eps"), layers=tuple(layers),
        )

    def with_sizes_of(self, shapes: dict[str, tuple[int, ...]]) -> "KatenexConfig":
        """The sizes that config.json leaves to the tensors' shapes, read from `shapes` (name -> shape)."""
        layers = []
        for index, layer in enumerate(self.layers):
            mixer = layer.mixer
            if isinstance(mixer, KatenexDeltaMixer):
                decay, gate = shapes.get(f"l{index}.mix.a1"), shapes.get(f"l{index}.mix.g1")
                mixer = replace(
                    mixer,
                    decay_rank=mixer.decay_rank if mixer.decay_rank is not None or decay is None else int(decay[0]),
                    gate_rank=mixer.gate_rank if mixer.gate_rank is not None or gate is None else int(gate[0]),
                )
            layers.append(replace(layer, mixer=mixer))
        return replace(self, layers=tuple(layers))

    def to_config_json(self) -> dict[str, Any]:
        layers = []
        for layer in self.layers:
            mixer = layer.mixer
            if isinstance(mixer, KatenexParallelMixer):
                left: dict[str, Any] = {"heads": mixer.left.heads, "kv_heads": mixer.left.kv_heads, "dim": mixer.left.dim,
                                        "vdim": mixer.left.vdim, "scale": mixer.left.scale}
                if mixer.left.rot is not None:
                    left["rot"] = {"base": mixer.left.rot.base, "dims": mixer.left.rot.dims}
                    if mixer.left.rot.factor is not None:
                        left["rot"]["scaling"] = {"factor": mixer.left.rot.factor}
                described: dict[str, Any] = {
                    "left": left, "left_scale": mixer.left_scale, "right_scale": mixer.right_scale,
                    "right": {"width": mixer.right.width, "blocks": mixer.right.blocks, "conv": mixer.right.conv},
                }
            else:
                described = {"heads": mixer.heads, "kv_heads": mixer.kv_heads, "dim": mixer.dim, "vdim": mixer.vdim, "conv": mixer.conv}
                if mixer.decay_rank is not None:
                    described["decay_rank"] = mixer.decay_rank
                if mixer.gate_rank is not None:
                    described["gate_rank"] = mixer.gate_rank
            mlp = layer.mlp
            feed: Any = None
            if mlp is not None:
                router: dict[str, Any] = {"experts": mlp.experts, "top": mlp.top, "scale": mlp.scale}
                if mlp.groups > 1:
                    router["groups"] = {"count": mlp.groups, "keep": mlp.keep}
                feed = {"kind": "moe", "expert": {"ff": mlp.expert_ff}, "router": router}
                if mlp.shared_ff is not None:
                    feed["shared"] = {"ff": mlp.shared_ff}
            layers.append({"type": layer.type, "mixer": described, "mlp": feed})
        described = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                     "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.streams is not None:
            described["streams"] = self.streams
        return described
