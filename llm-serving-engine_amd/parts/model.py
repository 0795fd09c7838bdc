"""A decoder as data: an embedding, layer definitions, the order in which they
run, a final norm and an output head.  `DecoderModel` runs any such list."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import BLOCKS, LOGIT_PARTS, NORMS, PASS_PARTS, STREAM_PARTS, CacheNeed, TensorSpec, prefixed, under


@dataclass(frozen=True)
class LayerDefinition:
    prefix: str  # e.g. "model.layers.3."
    block: Any  # spec of a block


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order.  `layer` indexes `ModelSpec.layers`; a layer
    may be named by several entries (its tensors are shared, each run has a
    cache cell of its own).  With `reads` set, the run uses the cell of that
    earlier entry of the run order instead, and stores nothing.  With `enters` set, the run is
    the first of a pass (its number: 0, 1, ...) through layers that the model walks several times, and
    the model's `pass_entry` part acts on the stream before it."""

    layer: int
    reads: int | None = None
    enters: int | None = None


@dataclass(frozen=True)
class NamedPart:
    """A part outside the layers: the prefix of its tensors and its spec."""

    prefix: str
    spec: Any


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerDefinition, ...]
    run_order: tuple[LayerRun, ...]
    final_norm: Any
    tie_embeddings: bool
    embedding_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm."
    head_name: str = "lm_head.weight"
    # parts that act on the embedded rows before the first layer (kinds of STREAM_PARTS), and on the
    # logits after the head (kinds of LOGIT_PARTS), in order; Qwen2 has none
    input_parts: tuple[NamedPart, ...] = ()
    output_parts: tuple[NamedPart, ...] = ()
    # the part that stands before every run with `enters` set (a kind of PASS_PARTS)
    pass_entry: NamedPart | None = None
    # tensors that a model folder may hold and the model does not use
    ignored_tensors: tuple[str, ...] = ()

    def __post_init__(self) -> None:
        if self.pass_entry is None and any(run.enters is not None for run in self.run_order):
            raise ValueError("a run begins a pass, and the model has no part for that")
        for index, run in enumerate(self.run_order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run {index} names layer {run.layer}, which does not exist")
            if run.reads is not None:
                if not 0 <= run.reads < index:
                    raise ValueError(f"run {index} reads the cache of run {run.reads}, which is not earlier")
                if self.run_order[run.reads].reads is not None:
                    raise ValueError(f"run {index} reads run {run.reads}, which owns no cache")
                if self.cell_need(run.reads) != self.cell_need(index):
                    raise ValueError(f"run {index} and run {run.reads} need different caches")

    def cell_need(self, run_index: int) -> CacheNeed:
        block = self.layers[self.run_order[run_index].layer].block
        return BLOCKS.cache_need(block)

    def tensors(self) -> dict[str, TensorSpec]:
        """Every tensor of the model by its name in the model folder."""
        found = {self.embedding_name: TensorSpec((self.vocab_size, self.hidden_size), role="embedding")}
        for layer in self.layers:
            found.update(prefixed(BLOCKS.tensors(layer.block), layer.prefix))
        found.update(prefixed(NORMS.tensors(self.final_norm), self.final_norm_name))
        for part in self.input_parts:
            found.update(prefixed(STREAM_PARTS.tensors(part.spec), part.prefix))
        for part in self.output_parts:
            found.update(prefixed(LOGIT_PARTS.tensors(part.spec), part.prefix))
        if self.pass_entry is not None:
            found.update(prefixed(PASS_PARTS.tensors(self.pass_entry.spec), self.pass_entry.prefix))
        if not self.tie_embeddings:
            found[self.head_name] = TensorSpec((self.vocab_size, self.hidden_size))
        return found


class DecoderModel:
    """Runs a `ModelSpec`: embedding, the layers in run order, final norm and
    head on the wanted rows only (the reference computes the head on every row,
    `model.py:309`).  Architecture-agnostic: everything specific sits in the spec."""

    def __init__(self, spec: ModelSpec, tensors: dict[str, torch.Tensor], kernels) -> None:
        self.spec = spec
        self.kernels = kernels
        self.embedding = tensors[spec.embedding_name]
        self.layers = [
            BLOCKS.build(layer.block, under(tensors, layer.prefix), kernels) for layer in spec.layers
        ]
        self.final_norm = NORMS.build(spec.final_norm, under(tensors, spec.final_norm_name), kernels)
        head = self.embedding if spec.tie_embeddings else tensors[spec.head_name]
        self.head = kernels.prepare_linear([head], None)
        self.input_parts = [STREAM_PARTS.build(part.spec, under(tensors, part.prefix), kernels) for part in spec.input_parts]
        self.output_parts = [LOGIT_PARTS.build(part.spec, under(tensors, part.prefix), kernels) for part in spec.output_parts]
        self.pass_entry = None
        if spec.pass_entry is not None:
            self.pass_entry = PASS_PARTS.build(spec.pass_entry.spec, under(tensors, spec.pass_entry.prefix), kernels)
        every = [*self.layers, self.final_norm, *self.input_parts, *self.output_parts]
        every += [self.pass_entry] if self.pass_entry is not None else []
        self.replayable = all(part.replayable for part in every)
        # Called, if set, after every run of the run order with (index of the run, the float32 stream, what the
        # run still has to add to it: None, [T, hidden] or partial sums [parts, T, hidden]): tests and
        # debugging look at the stream layer by layer through it (with a runner that replays no graphs).
        self.observer = None

    def _run_layers(self, batch, cells: list):
        hidden = self.kernels.embedding(self.embedding, batch.token_ids)
        for part in self.input_parts:  # (in place, or a new stream of another shape: copies side by side)
            changed = part.forward(hidden, batch)
            hidden = hidden if changed is None else changed
        embedded = hidden.clone() if self.pass_entry is not None else None  # the layers add into `hidden` in place
        delta = None
        for index, (run, cell) in enumerate(zip(self.spec.run_order, cells)):
            layer = self.layers[run.layer]
            # what a block left to do in a form of its own (a result that is normed before it is added) is done here
            # unless the next block takes it as it is
            if hasattr(delta, "settle") and (run.enters is not None or not getattr(layer, "accepts_pending_normed", False)):
                delta = delta.settle(hidden)
            if run.enters is not None:
                hidden, delta = self.pass_entry.forward(hidden, delta, embedded, batch, run.enters), None
            delta = layer.forward(hidden, delta, batch, cell)
            if self.observer is not None:
                if hasattr(delta, "settle"):
                    delta = delta.settle(hidden)
                self.observer(index, hidden, delta)
        if hasattr(delta, "settle"):
            delta = delta.settle(hidden)
        return hidden, delta

    def forward_without_logits(self, batch, cells: list) -> None:
        """Runs the layers only: the step fills the cache and no logits are wanted."""
        self._run_layers(batch, cells)

    def forward(self, batch, cells: list) -> torch.Tensor:
        """Logits [R, vocab] float32 at `batch.logit_rows`.  `cells[i]` is the
        cache cell of run i."""
        hidden, delta = self._run_layers(batch, cells)
        if getattr(batch, "every_row_wanted", False):  # the final norm adds the last layer's delta itself
            normed = self.final_norm.forward(hidden, delta)
        elif hasattr(self.final_norm, "forward_rows"):  # a norm that reads the wanted rows of the stream itself
            normed = self.final_norm.forward_rows(hidden, delta, batch.logit_rows)
        else:
            rows = self.kernels.gather_rows(hidden, delta, batch.logit_rows)
            normed = self.final_norm.forward(rows, None)
        logits = self.kernels.linear(normed, self.head, out_dtype=torch.float32)
        for part in self.output_parts:
            logits = part.forward(logits, batch)
        return logits


@dataclass(frozen=True)
class JoinedPassSpec:
    """x <- W [x; x0] + step[t] at the start of pass t, x0 the embedded stream; `passes` is how many
    there are.  `weight_name` [hidden, 2 hidden] and `step_name` [passes, hidden] below the part's prefix."""

    hidden_size: int
    passes: int
    weight_name: str = "in"
    step_name: str = "step"
    kind: str = "joined_pass"


@PASS_PARTS.register("joined_pass")
class JoinedPass:
    """The stream that enters a pass is a product of the stream so far beside the embedded one, plus a
    vector of the pass.  The product's operand is the two streams side by side in the run dtype; its result
    (with the pass's vector as the product's bias) is the new float32 stream."""

    replayable = True

    @classmethod
    def tensors(cls, spec: JoinedPassSpec) -> dict[str, TensorSpec]:
        return {
            spec.weight_name: TensorSpec((spec.hidden_size, 2 * spec.hidden_size)),
            spec.step_name: TensorSpec((spec.passes, spec.hidden_size), role="bias"),
        }

    @classmethod
    def cache_need(cls, spec: JoinedPassSpec) -> None:
        return None

    def __init__(self, spec: JoinedPassSpec, tensors, kernels) -> None:
        self.spec = spec
        self.kernels = kernels
        weight, steps = tensors[spec.weight_name], tensors[spec.step_name]
        self.products = [kernels.prepare_linear([weight], [steps[index].contiguous()]) for index in range(spec.passes)]

    def forward(self, hidden, delta, embedded, batch, number: int):
        both = self.kernels.join_rows(hidden, delta, embedded)  # [T, 2 hidden] in the run dtype
        return self.kernels.linear(both, self.products[number], out_dtype=torch.float32)


@dataclass(frozen=True)
class AddedPassSpec:
    """x <- x + x0 (every pass but the first) + step[t] at the start of pass t, x0 the embedded stream; `passes` is how
    many there are.  `step_name` [passes, hidden] below the part's prefix."""

    hidden_size: int
    passes: int
    step_name: str = "step"
    kind: str = "added_pass"


@PASS_PARTS.register("added_pass")
class AddedPass:
    """The stream that enters a pass is the stream so far plus a vector of the pass and, from the second pass on, plus
    the embedded stream: one kernel, in place, in float32."""

    replayable = True

    @classmethod
    def tensors(cls, spec: AddedPassSpec) -> dict[str, TensorSpec]:
        return {spec.step_name: TensorSpec((spec.passes, spec.hidden_size), role="bias")}

    @classmethod
    def cache_need(cls, spec: AddedPassSpec) -> None:
        return None

    def __init__(self, spec: AddedPassSpec, tensors, kernels) -> None:
        self.spec = spec
        self.kernels = kernels
        steps = tensors[spec.step_name]
        self.steps = [steps[index].float().contiguous() for index in range(spec.passes)]

    def forward(self, hidden, delta, embedded, batch, number: int):
        return self.kernels.add_rows(hidden, delta, embedded if number > 0 else None, self.steps[number])


@dataclass(frozen=True)
class SoftCapSpec:
    cap: float
    kind: str = "soft_cap"


@LOGIT_PARTS.register("soft_cap")
class SoftCap:
    """logits <- cap * tanh(logits / cap), in place on the wanted rows."""

    replayable = True

    @classmethod
    def tensors(cls, spec: SoftCapSpec) -> dict[str, TensorSpec]:
        return {}

    @classmethod
    def cache_need(cls, spec: SoftCapSpec) -> None:
        return None

    def __init__(self, spec: SoftCapSpec, tensors, kernels) -> None:
        if not spec.cap > 0:
            raise ValueError("soft cap: the cap is positive")
        self.spec = spec
        self.kernels = kernels

    def forward(self, logits, batch):
        return self.kernels.soft_cap(logits, self.spec.cap)
