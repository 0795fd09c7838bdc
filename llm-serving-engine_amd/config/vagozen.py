"""The typed configuration of the Vagozen decoder, read from its own config.json.

config.json gives every size and every constant that differs between models of the design: `vocab`, `width`,
`norm.eps`, `logit_scale`, `layers` (per layer its `type`, the `mixer`'s sizes and its `mlp`, or null for none)
and `loop` (layers `start` .. `stop - 1` run `times` times in a row).  Nothing here has a default but what may
be absent: `kv_heads` (as many as heads), `mask` (every earlier token is seen), `mask.keep_first` (0), `rot`
(positions do not enter), `rot.scaling`, `mlp`, `loop`, `logit_scale` (1).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .model import ArchitectureConfig, ConfigError, KeyReader

LAYER_TYPES = ("attention", "retention", "latent_attention")


@dataclass(frozen=True)
class VagozenRotary:
    base: float
    dims: int
    scaling: tuple[float, float, float, float] | None = None  # factor, original, fast, slow


@dataclass(frozen=True)
class VagozenAttentionMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None
    keep_first: int
    rot: VagozenRotary | None


@dataclass(frozen=True)
class VagozenRetentionMixer:
    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]
    rot: VagozenRotary | None


@dataclass(frozen=True)
class VagozenLatentMixer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: VagozenRotary


@dataclass(frozen=True)
class VagozenDenseMLP:
    ff: int
    limit: float


@dataclass(frozen=True)
class VagozenExpertsMLP:
    experts: int
    top: int
    expert_ff: int
    limit: float


@dataclass(frozen=True)
class VagozenLayer:
    type: str
    mixer: VagozenAttentionMixer | VagozenRetentionMixer | VagozenLatentMixer
    mlp: VagozenDenseMLP | VagozenExpertsMLP | None


@dataclass(frozen=True)
class VagozenLoop:
    start: int
    stop: int
    times: int


def _mapping(value: Any, where: str) -> dict[str, Any]:
    if not isinstance(value, dict):
        raise ConfigError(f"{where} must be a mapping, got {value!r}")
    return value


def _read_rotary(values: Any, where: str, default_dims: int | None = None) -> VagozenRotary | None:
    if values is None:
        return None
    reader = KeyReader(_mapping(values, where), where)
    scaling = None
    if reader.optional("scaling"):
        scale_reader = KeyReader(_mapping(values["scaling"], f"{where}.scaling"), f"{where}.scaling")
        scaling = tuple(scale_reader.number(name) for name in ("factor", "original", "fast", "slow"))
    if default_dims is None:
        dims = reader.integer("dims", minimum=2)
    else:
        dims = reader.integer("dims", default=default_dims, minimum=2)
    return VagozenRotary(reader.number("base"), dims, scaling)


def _read_mixer(kind: str, values: dict[str, Any], where: str):
    reader = KeyReader(values, where)
    heads = reader.integer("heads")
    if kind == "attention":
        window, keep_first = None, 0
        if values.get("mask") is not None:
            mask = KeyReader(_mapping(values["mask"], f"{where}.mask"), f"{where}.mask")
            window = mask.integer("size")
            keep_first = mask.integer("keep_first", default=0, minimum=0)
        return VagozenAttentionMixer(
            heads=heads, kv_heads=reader.integer("kv_heads", default=heads), dim=reader.integer("dim"), vdim=reader.integer("vdim"),
            scale=reader.number("scale"), window=window, keep_first=keep_first, rot=_read_rotary(values.get("rot"), f"{where}.rot"),
        )
    if kind == "retention":
        decay = values.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"{where}: 'decay' must list one number a head")
        return VagozenRetentionMixer(
            heads=heads, dim=reader.integer("dim"), vdim=reader.integer("vdim"), decay=tuple(float(d) for d in decay),
            rot=_read_rotary(values.get("rot"), f"{where}.rot"),
        )
    rot_dim = reader.integer("rot_dim")
    return VagozenLatentMixer(
        heads=heads, dim=reader.integer("dim"), rot_dim=rot_dim, vdim=reader.integer("vdim"), q_rank=reader.integer("q_rank"),
        kv_rank=reader.integer("kv_rank"), scale=reader.number("scale"),
        rot=_read_rotary(_mapping(values.get("rot"), f"{where}.rot"), f"{where}.rot", default_dims=rot_dim),
    )


def _read_mlp(values: Any, where: str):
    if values is None:
        return None
    reader = KeyReader(_mapping(values, where), where)
    kind = reader.choice("kind", choices=("dense", "moe"))
    if kind == "dense":
        return VagozenDenseMLP(reader.integer("ff"), reader.number("limit"))
    router = KeyReader(_mapping(values.get("router"), f"{where}.router"), f"{where}.router")
    expert = KeyReader(_mapping(values.get("expert"), f"{where}.expert"), f"{where}.expert")
    return VagozenExpertsMLP(experts=router.integer("experts"), top=router.integer("top"), expert_ff=expert.integer("ff"), limit=expert.number("limit"))


@dataclass(frozen=True)
class VagozenConfig(ArchitectureConfig):
    architecture: ClassVar[str] = "Vagozen"

    vocab: int
    width: int
    norm_eps: float
    layers: tuple[VagozenLayer, ...]
    loop: VagozenLoop | None = None
    logit_scale: float = 1.0

    def __post_init__(self) -> None:
        if not self.layers:
            raise ConfigError("Vagozen config: no layers")
        for index, layer in enumerate(self.layers):
            mixer, where = layer.mixer, f"Vagozen config: layer {index}"
            if isinstance(mixer, VagozenAttentionMixer):
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
                if mixer.rot is not None and (mixer.rot.dims % 2 or mixer.rot.dims > mixer.dim):
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
            elif isinstance(mixer, VagozenRetentionMixer):
                if any(not 0.0 < d <= 1.0 for d in mixer.decay):
                    raise ConfigError(f"{where}: a decay lies in (0, 1]")
                if mixer.rot is not None and (mixer.rot.dims % 2 or mixer.rot.dims > mixer.dim):
                    raise ConfigError(f"{where}: rot.dims must be even and at most dim")
            elif mixer.rot.dims % 2 or mixer.rot.dims > mixer.rot_dim:
                raise ConfigError(f"{where}: rot.dims must be even and at most rot_dim")
            if isinstance(layer.mlp, (VagozenDenseMLP, VagozenExpertsMLP)) and not layer.mlp.limit > 0:
                raise ConfigError(f"{where}: the feed-forward's limit must be positive")
            if isinstance(layer.mlp, VagozenExpertsMLP) and layer.mlp.top > layer.mlp.experts:
                raise ConfigError(f"{where}: more experts a token than there are")
        if self.loop is not None and not 0 <= self.loop.start < self.loop.stop <= len(self.layers):
            raise ConfigError("Vagozen config: loop must name layers start < stop within the model")

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, values: dict[str, Any]) -> "VagozenConfig":
        reader = KeyReader(values, "Vagozen config")
        norm = KeyReader(_mapping(values.get("norm"), "Vagozen config: norm"), "Vagozen config: norm")
        entries = values.get("layers")
        if not isinstance(entries, list):
            raise ConfigError("Vagozen config: 'layers' must be a list")
        layers = []
        for index, entry in enumerate(entries):
            where = f"Vagozen config: layers[{index}]"
            entry = _mapping(entry, where)
            kind = KeyReader(entry, where).choice("type", choices=LAYER_TYPES)
            mixer = _read_mixer(kind, _mapping(entry.get("mixer"), f"{where}.mixer"), f"{where}.mixer")
            layers.append(VagozenLayer(kind, mixer, _read_mlp(entry.get("mlp"), f"{where}.mlp")))
        loop = None
        if values.get("loop"):
            loop_reader = KeyReader(_mapping(values["loop"], "Vagozen config: loop"), "Vagozen config: loop")
            loop = VagozenLoop(loop_reader.integer("start", minimum=0), loop_reader.integer("stop"), loop_reader.integer("times"))
        return cls(
            vocab=reader.integer("vocab"), width=reader.integer("width"), norm_eps=norm.number("eps"), layers=tuple(layers), loop=loop,
            logit_scale=reader.number("logit_scale", default=1.0),
        )

    def to_config_json(self) -> dict[str, Any]:
        def rotary(rot: VagozenRotary | None):
            if rot is None:
                return None
            described: dict[str, Any] = {"base": rot.base, "dims": rot.dims}
            if rot.scaling is not None:
                described["scaling"] = dict(zip(("factor", "original", "fast", "slow"), rot.scaling))
            return described

        layers = []
        for layer in self.layers:
            mixer = layer.mixer
            if isinstance(mixer, VagozenAttentionMixer):
                described: dict[str, Any] = {"heads": mixer.heads, "kv_heads": mixer.kv_heads, "dim": mixer.dim, "vdim": mixer.vdim, "scale": mixer.scale}
                if mixer.window is not None:
                    described["mask"] = {"size": mixer.window, "keep_first": mixer.keep_first}
            elif isinstance(mixer, VagozenRetentionMixer):
                described = {"heads": mixer.heads, "dim": mixer.dim, "vdim": mixer.vdim, "decay": list(mixer.decay)}
            else:
                described = {"heads": mixer.heads, "dim": mixer.dim, "rot_dim": mixer.rot_dim, "vdim": mixer.vdim, "q_rank": mixer.q_rank,
                             "kv_rank": mixer.kv_rank, "scale": mixer.scale}
            if mixer.rot is not None:
                described["rot"] = rotary(mixer.rot)
            mlp = layer.mlp
            if isinstance(mlp, VagozenDenseMLP):
                feed: Any = {"kind": "dense", "ff": mlp.ff, "limit": mlp.limit}
            elif isinstance(mlp, VagozenExpertsMLP):
                feed = {"kind": "moe", "expert": {"ff": mlp.expert_ff, "limit": mlp.limit}, "router": {"experts": mlp.experts, "top": mlp.top}}
            else:
                feed = None
            layers.append({"type": layer.type, "mixer": described, "mlp": feed})
        values: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                                  "norm": {"eps": self.norm_eps}, "layers": layers, "logit_scale": self.logit_scale}
        if self.loop is not None:
            values["loop"] = {"start": self.loop.start, "stop": self.loop.stop, "times": self.loop.times}
        return values
