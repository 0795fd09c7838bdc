"""Small Vagozen models for the tests: configurations as config.json mappings, random tensors that make every
mechanism count, and model folders.

The sizes differ from layer to layer and avoid coincidences (dim != vdim, heads / kv_heads of 1, 2 and 3, rot.dims
below dim, windows and kept first tokens that are no multiple of a page, scales that are no power of dim, decays that
differ from head to head, latents of sizes of their own, one to all experts a token, a layer without a feed-forward,
loops from the first layer, of one pass, with layers behind them, and none)."""

from __future__ import annotations

from pathlib import Path

import torch

from tests.dafutar_cases import run_steps, tokens_of, write_folder as _write_folder  # noqa: F401  (generic helpers)

YARN = {"factor": 3.0, "original": 48, "fast": 8.0, "slow": 1.0}


def attention(heads=6, kv_heads=2, dim=24, vdim=40, window=13, keep_first=3, scale=0.31, dims=10, scaling=YARN, base=500.0):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(scaling)
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window, "keep_first": keep_first}
    return {"type": "attention", "mixer": mixer}


def retention(heads=3, dim=16, vdim=24, decay=(0.7, 0.95, 0.995), dims=8, base=300.0):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": {"base": base, "dims": dims}}}


def latent(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=24, scale=0.2, base=1000.0):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                                                  "scale": scale, "rot": {"base": base, "dims": rot_dim}}}


def dense(ff=56, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts=5, top=2, ff=24, limit=2.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config_of(layers, vocab=67, width=40, eps=1e-4, loop=None, logit_scale=0.7):
    """`layers`: [(mixer entry, mlp or None)]; `loop`: (start, stop, times)."""
    values = {"architecture": "Vagozen", "vocab": vocab, "width": width, "norm": {"eps": eps},
              "layers": [dict(mixer, mlp=mlp) for mixer, mlp in layers], "logit_scale": logit_scale}
    if loop is not None:
        values["loop"] = dict(zip(("start", "stop", "times"), loop))
    return values


# A model with every kind of layer, in an order of its own, sizes that differ wherever they can, and a loop in the middle.
MIXED = config_of(
    [
        (retention(heads=3, dim=16, vdim=24), moe(experts=5, top=2, ff=24)),
        (attention(heads=6, kv_heads=2, dim=24, vdim=40, window=13, keep_first=3), dense(56)),
        (latent(heads=3, dim=16, rot_dim=8, vdim=24), None),
        (attention(heads=2, kv_heads=1, dim=40, vdim=8, window=30, keep_first=9, dims=40, scaling=None), moe(experts=3, top=3, ff=16, limit=1.0)),
        (retention(heads=2, dim=32, vdim=16, decay=(1.0, 0.5), dims=32), dense(16, limit=0.75)),
        (latent(heads=2, dim=8, rot_dim=16, vdim=8, q_rank=12, kv_rank=32, scale=0.4), dense(72, limit=4.0)),
    ],
    loop=(1, 4, 3),
)


def random_tensors(values: dict, seed: int, *, sharp: bool = False) -> dict[str, torch.Tensor]:
    """bfloat16 tensors (the precision model folders hold) by the model's own list of names and shapes.  Matrices are
    drawn so that activations stay of order one; norms, vectors on results, biases and the passes' vectors are far
    enough from one and zero to matter.  `sharp`: the attention's queries and keys are large, so that a softmax looks
    at one key."""
    from llmserve_amd.registry import resolve_architecture

    architecture = resolve_architecture(values)
    spec = architecture.build_spec(architecture.config_class.from_dict(values))
    generator = torch.Generator().manual_seed(seed)
    kinds = [layer["type"] for layer in values["layers"]]
    tensors = {}
    for name, wanted in spec.tensors().items():
        shape = wanted.shape
        last = name.rsplit(".", 1)[-1]
        if name == "embed":
            value = torch.randn(shape, generator=generator)
        elif name == "loop.step":
            value = 0.5 * torch.randn(shape, generator=generator)
        elif name.endswith("router.b"):
            value = 0.7 * torch.randn(shape, generator=generator)
        elif last == "b":
            value = 0.3 * torch.randn(shape, generator=generator)
        elif wanted.role == "norm":  # (the vectors on the sublayers' results too)
            value = 1.0 + 0.3 * torch.randn(shape, generator=generator)
        elif last in ("router", "g"):
            value = 2.0 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
        else:
            value = 1.4 * torch.randn(shape, generator=generator) / shape[-1] ** 0.5
            if sharp and name.endswith((".mix.q", ".mix.k")) and kinds[int(name[1:name.index(".")])] == "attention":
                value = 2.2 * value
        tensors[name] = value.to(torch.bfloat16)
    return tensors


def write_folder(folder: Path, values: dict, seed: int = 1, *, sharp: bool = False, tensors: dict | None = None) -> Path:
    return _write_folder(folder, values, seed, tensors=tensors if tensors is not None else random_tensors(values, seed, sharp=sharp))
