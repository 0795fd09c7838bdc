"""Small Katenex models for the tests: configurations as config.json mappings, random tensors that make every
mechanism count, and model folders.

The sizes differ from layer to layer and avoid coincidences (dim != vdim, one to three query or value heads a
key head, rot.dims below and equal to dim, one to four taps, groups of one to three experts of which some or all
are kept, a layer without a feed-forward or without a shared expert, one to four copies of the stream)."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from llmserve_amd.weights import read_config
from tests.dafutar_cases import run_steps, tokens_of  # noqa: F401  (the schedules' helper is the same)


def attention(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.31, dims=8, base=500.0, factor=2.0):
    found = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        found["rot"] = {"base": base, "dims": dims}
        if factor is not None:
            found["rot"]["scaling"] = {"factor": factor}
    return found


def recurrence(width=40, blocks=5, conv=3):
    return {"width": width, "blocks": blocks, "conv": conv}


def parallel(left=None, right=None, left_scale=0.8, right_scale=1.3):
    return {"type": "parallel", "mixer": {"left": left or attention(), "right": right or recurrence(), "left_scale": left_scale,
                                           "right_scale": right_scale}}


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, decay_rank=6, gate_rank=5):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                                "decay_rank": decay_rank, "gate_rank": gate_rank}}


def moe(experts=6, top=2, scale=1.25, ff=12, shared=20, groups=(3, 2)):
    router = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    found = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        found["shared"] = {"ff": shared}
    return found


def config_of(layers, streams=3, vocab=67, width=32, eps=1e-5, scale=3.0):
    """`layers`: [(mixer entry, mlp or None)]."""
    found = {"architecture": "Katenex", "vocab": vocab, "width": width, "streams": streams, "embedding": {"scale": scale},
             "norm": {"eps": eps}, "layers": [dict(mixer, mlp=mlp) for mixer, mlp in layers]}
    if streams is None:  # the plain residual sum
        del found["streams"]
    return found


# A model with both kinds of layer and sizes that differ wherever they can.
MIXED = config_of(
    [
        (delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3), moe(6, 2, 1.25, 12, 20, (3, 2))),
        (parallel(attention(4, 2, 16, 24, 0.31, 8), recurrence(40, 5, 3)), moe(8, 3, 0.75, 8, None, (4, 2))),
        (delta(heads=3, kv_heads=3, dim=24, vdim=8, conv=2, decay_rank=3, gate_rank=7), None),
        (parallel(attention(3, 1, 8, 8, 0.5, 8, factor=None), recurrence(24, 1, 4), 1.5, 0.4), moe(4, 1, 2.0, 16, 8, None)),
        (delta(heads=6, kv_heads=2, dim=8, vdim=16, conv=4), moe(6, 4, 1.0, 16, 8, (2, 2))),
    ],
    streams=3,
)


def with_every_expert(values: dict) -> dict:
    """The same model with every expert of a layer used by every token (all groups kept): the router still weighs
    them, but chooses nothing, so no rounding can turn a choice."""
    values = json.loads(json.dumps(values))
    for layer in values["layers"]:
        if layer["mlp"] is not None:
            router = layer["mlp"]["router"]
            router["top"] = router["experts"]
            if "groups" in router:
                router["groups"]["keep"] = router["groups"]["count"]
    return values


def random_tensors(values: dict, seed: int, *, sharp: bool = False) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by the model's own list of names and shapes.  Matrices are drawn so that activations stay
    of order one; norms, biases, decays and the links between the copies of the stream are far enough from one and
    zero to matter.  `sharp`: decays near one (the state remembers far back)."""
    from llmserve_amd.registry import resolve_architecture

    architecture = resolve_architecture(values)
    spec = architecture.build_spec(architecture.config_class.from_dict(values))
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, wanted in spec.tensors().items():
        shape = wanted.shape
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            value = torch.randn(shape, generator=generator)
        elif last == "A_log":
            value = torch.randn(shape, generator=generator) * 0.5 + (-5.0 if sharp else -1.0)
        elif last == "dt_bias":
            value = torch.randn(shape, generator=generator)
        elif last == "lam":
            value = torch.randn(shape, generator=generator) * 0.5 + (-6.0 if sharp else -1.5)
        elif last == "conv":
            value = torch.randn(shape, generator=generator) / shape[1] ** 0.5
        elif ".hc" in name and last == "mix":
            value = torch.eye(shape[0]) + 0.25 * torch.randn(shape, generator=generator)
        elif ".hc" in name:  # in, out
            value = 0.7 + 0.3 * torch.randn(shape, generator=generator)
        elif last == "b" and len(shape) <= 2 and wanted.role == "bias":
            value = 0.3 * torch.randn(shape, generator=generator)
        elif wanted.role == "norm":
            value = 1.0 + 0.3 * torch.randn(shape, generator=generator)
        elif last in ("router", "a2", "g2"):
            value = 2.0 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        else:
            value = 1.4 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(folder: Path, values: dict, seed: int = 1, *, sharp: bool = False, tensors: dict | None = None, drop_ranks: bool = False) -> Path:
    """`drop_ranks`: config.json leaves the low-rank products' inner sizes to the tensors' shapes."""
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    tensors = tensors if tensors is not None else random_tensors(values, seed, sharp=sharp)
    written = json.loads(json.dumps(values))
    if drop_ranks:
        for layer in written["layers"]:
            layer["mixer"].pop("decay_rank", None)
            layer["mixer"].pop("gate_rank", None)
    (folder / "config.json").write_text(json.dumps(written, indent=1))
    save_file({name: value.contiguous() for name, value in tensors.items()}, str(folder / "model.safetensors"))
    read_config(folder)  # the folder is one the engine accepts
    return folder


def read_folder(folder: Path):
    """(config.json as a mapping, the folder's tensors in float64) for the plain implementation."""
    from safetensors.torch import load_file

    folder = Path(folder)
    return json.loads((folder / "config.json").read_text()), {name: value.double() for name, value in load_file(str(folder / "model.safetensors")).items()}
