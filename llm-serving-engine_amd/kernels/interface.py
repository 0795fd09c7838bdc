"""The operations the parts call.  The product has one implementation, the HIP
library in `hip.py`; the interface is spelled out so that tests can check parts,
cache and step function with a stand-in of their own on a machine without a GPU.

Conventions: the residual stream and every value added to it are float32 in
every run dtype; activations between kernels are in the run dtype (bfloat16 or
float32); products accumulate in float32; logits are float32.
"""

from __future__ import annotations

from typing import Any, Protocol

import torch


class Kernels(Protocol):
    device: torch.device
    dtype: torch.dtype

    def to_device(self, tensor: torch.Tensor) -> torch.Tensor: ...

    def queued_to_device(self, tensor: torch.Tensor) -> torch.Tensor:
        """As `to_device`, for small per-step inputs: the host does not wait for work queued before."""

    def embedding(self, table: torch.Tensor, token_ids: torch.Tensor) -> torch.Tensor:
        """float32 rows [T, hidden] of `table` at `token_ids`."""

    def add_rms_norm(
        self, hidden: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float
    ) -> torch.Tensor:
        """`hidden += delta` in place (float32), then rows * rsqrt(mean(rows^2) + eps) * weight in the run dtype."""

    def prepare_linear(self, weights: list[torch.Tensor], biases: list[torch.Tensor] | None) -> Any:
        """Concatenates [N_i, K] weights (and biases) along N into whatever layout `linear` wants."""

    def prepare_gated_linear(self, gate: torch.Tensor, up: torch.Tensor, activation: str = "silu", limit: float | None = None) -> Any:
        """Gate and up weights [I, K] in whatever layout `gated_linear` wants; `activation` is the gate's
        (silu, gelu, gelu_tanh, relu), and one the library has no kernel for is refused here, by name.
        "limited_swish" is a function of gate and up both and has a `limit`: g = min(gate, limit), u = clamp(up,
        -limit, limit), and the result is g * sigmoid(1.702 g) * (u + 1)."""

    def linear(
        self, x: torch.Tensor, weights: Any, out_dtype: torch.dtype | None = None, *, partial: bool = False
    ) -> torch.Tensor:
        """x [T, K] @ W^T + bias -> [T, N] in `out_dtype` (the run dtype if None).  With
        `partial`, a float32 result may be [parts, T, N] partial sums for the reader to add."""

    def gated_linear(self, x: torch.Tensor, weights: Any) -> torch.Tensor:
        """act(x Wg^T) * (x Wu^T) -> [T, I] in the run dtype."""

    def rotate_and_store(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any,
        inverse_frequencies: torch.Tensor | None, pairing: str,
    ) -> None:
        """Rotary on the q and k heads of `qkv` in place; k and v into the cell's pages if it is writable."""

    def paged_attention(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any, scale: float, window: int | None, *,
        score_slopes: torch.Tensor | None = None, soft_cap: float | None = None, sinks: torch.Tensor | None = None,
        keep_first: int = 0,
    ) -> torch.Tensor:
        """Attention of the q heads of `qkv` over the cell's pages -> [T, heads * head_dim].
        Before the softmax a score s of a query at position p for a key at position k may be changed,
        for encodings and models that want it (Qwen2 wants neither): with `soft_cap`, to
        soft_cap * tanh(s / soft_cap); with `score_slopes` (float32, one per query head), by
        - slope * (p - k) after that.  With `sinks` (float32, one per query head) the softmax's denominator
        has exp(sink) more, once, with no value to it.  With `keep_first` (and a window) a query at p sees the keys at
        k <= p with p - k < window or k < keep_first: a sequence's first keys stay visible, at their own positions (the
        cell's need says the same, so their pages are never given back).  A library refuses what it cannot compute."""

    def rotate_store_attend(
        self, qkv: torch.Tensor, layout: Any, batch: Any, cell: Any,
        inverse_frequencies: torch.Tensor | None, pairing: str, scale: float, window: int | None,
        project: Any = None,
    ) -> torch.Tensor:
        """`rotate_and_store` followed by `paged_attention` (a library may fuse them); with `project` (what
        `prepare_linear` returned), followed by `linear(that, project, float32, partial=True)`, whose result
        is returned instead (a library may let that product finish what the attention left undone)."""

    # ------------------------------------------------------------------ layer norm, runs of columns, products per head

    def add_layer_norm(
        self, hidden: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, bias: torch.Tensor, eps: float
    ) -> torch.Tensor:
        """`hidden += delta` in place (float32), then (rows - mean) * rsqrt(var + eps) * weight + bias in the run dtype."""

    def new_rows(self, rows: int, width: int) -> torch.Tensor:
        """An uninitialised [rows, width] tensor in the run dtype for operations that write runs of its columns."""

    def rms_norm_columns(
        self, x: torch.Tensor, first: int, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None,
        out_first: int = 0, copies: int = 1, copy_stride: int = 0,
    ) -> torch.Tensor:
        """RMS norm (float32) of the columns [first, first + len(weight)) of x's rows, times weight; written to a new
        tensor, or to `copies` places of `out`'s rows, `copy_stride` columns apart, from column `out_first`."""

    def rotary_table(self, batch: Any, frequencies: torch.Tensor, magnitude: float = 1.0) -> torch.Tensor:
        """float32 [T, len(frequencies), 2]: magnitude * (cos, sin) of position * frequency for the step's tokens."""

    def rotate_columns(
        self, x: torch.Tensor, first: int, head_stride: int, heads: int, width: int, table: torch.Tensor, dims: int,
        out: torch.Tensor, out_first: int, out_head_stride: int,
    ) -> torch.Tensor:
        """For every head h: `width` columns of x from first + h * head_stride to out from out_first + h *
        out_head_stride; the first `dims` of them rotated in adjacent pairs by the token's table row, the rest copied."""

    def prepare_headwise_linear(self, weight: torch.Tensor) -> Any:
        """[heads, N, K] weights in whatever layout `headwise_linear` wants."""

    def headwise_linear(
        self, x: torch.Tensor, first: int, head_stride: int, weights: Any, out: torch.Tensor | None = None,
        out_first: int = 0, out_head_stride: int | None = None,
    ) -> torch.Tensor:
        """For every head h: x[:, first + h * head_stride : + K] @ W_h^T -> out[:, out_first + h * out_head_stride : + N]
        (a new [T, heads * N] tensor if `out` is None), run dtype, float32 sums."""

    def join_rows(self, hidden: torch.Tensor, delta: torch.Tensor | None, embedded: torch.Tensor) -> torch.Tensor:
        """[hidden + delta | embedded] in the run dtype, [T, 2 hidden]."""

    def activate(self, x: torch.Tensor, activation: str) -> torch.Tensor:
        """act(x) elementwise (silu, gelu, gelu_tanh, relu), in x's type."""

    def add_gated_rows(self, target: torch.Tensor, rows: torch.Tensor, gates: torch.Tensor, column: int, squash: str) -> torch.Tensor:
        """target += squash(gates[:, column]) * rows, float32, in place."""

    # ------------------------------------------------------------------ the gated delta rule

    def causal_conv(
        self, x: torch.Tensor, channels: int, taps: torch.Tensor, activation: str, batch: Any, window: torch.Tensor | None,
        bias: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """act (silu, or "none") of the causal convolution per channel (plus `bias`, float32 [channels]) over each request's
        tokens, of the first `channels` columns of x; taps float32 [channels, width], the last column the current token's.  `window` float32 [slots, width - 1,
        channels] holds each request's last inputs (zeros at its start) and is moved on."""

    def gated_delta_rule(
        self, mixed: torch.Tensor, controls: torch.Tensor, rate: torch.Tensor, step_bias: torch.Tensor, heads: int,
        kv_heads: int, dim: int, vdim: int, batch: Any, state: torch.Tensor, channel_steps: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """With `channel_steps` (float32 [T, heads * dim or more columns]) the decay is one a head and key channel,
        g = exp(-exp(rate_h) softplus(channel_steps + step_bias)) with step_bias [heads * dim], row r of S scaled by g[r], and
        controls is [T, b] alone.  Otherwise:
        mixed [T, q | k | v], controls float32 [T, b | a]; q, k to unit length (q times dim^-1/2), beta = sigmoid(b),
        g = exp(-exp(rate) softplus(a + step_bias)); per request and head, token by token: S = g S; u = beta (v - S^T k);
        S += k u^T; o = S^T q.  `state` float32 [slots, heads, vdim, dim] holds S^T and is updated.  -> float32 [T, heads * vdim]."""

    def conv_gated_delta_rule(
        self, projected: torch.Tensor, channels: int, taps: torch.Tensor, activation: str, controls: torch.Tensor,
        rate: torch.Tensor, step_bias: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int, batch: Any,
        window: torch.Tensor | None, state: torch.Tensor, channel_steps: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """`causal_conv` followed by `gated_delta_rule` (a library may fuse them and keep what lies between in float32)."""

    def gated_head_norm(
        self, read: torch.Tensor, gates: torch.Tensor, gate_first: int, weight: torch.Tensor, eps: float, heads: int,
        vdim: int, activation: str,
    ) -> torch.Tensor:
        """Per head: read / rms(read) * weight * act(gates[:, gate_first + h * vdim : + vdim]) -> run dtype [T, heads * vdim];
        act silu or sigmoid; weight of vdim for every head; the gates in the run dtype or float32."""

    # ------------------------------------------------------------------ norms on results, heads put together, linear attention

    def stream_rows(self, hidden: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        """`hidden += delta` in place (float32), then the rows in the run dtype (in a float32 run the stream itself)."""

    def add_normed(self, hidden: torch.Tensor, update: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
        """`hidden += u * rsqrt(mean(u^2) + eps) * weight` in place, u the float32 rows of `update` (its parts added
        first); -> the new rows in the run dtype (in a float32 run the stream itself)."""

    def add_normed_norm(
        self, hidden: torch.Tensor, update: torch.Tensor, weight: torch.Tensor, eps: float, next_weight: torch.Tensor, next_eps: float,
    ) -> torch.Tensor:
        """`add_normed`, and then the norm before the next sublayer in the same pass over the row: -> the new rows *
        rsqrt(mean(new rows^2) + next_eps) * next_weight in the run dtype."""

    def rotate_heads(
        self, x: torch.Tensor, first: int, head_stride: int, heads: int, table: torch.Tensor | None, dims: int, pairing: str, scale: float = 1.0,
        scale_from: int = 0,
    ) -> torch.Tensor:
        """In place, for `heads` heads of `head_stride` columns from column `first` of x's rows (float32 or the run
        dtype): the first `dims` columns of a head turn in pairs (`pairing` "adjacent": (2i, 2i + 1); "half": (i, i +
        dims / 2)) by the token's row of `table` (float32 [T, dims / 2, 2], cos and sin), and every head from head `scale_from`
        on is multiplied by `scale` (queries and keys side by side in one call, the keys scaled); float32 arithmetic."""

    def add_rows(self, hidden: torch.Tensor, delta: torch.Tensor | None, other: torch.Tensor | None, vector: torch.Tensor | None) -> torch.Tensor:
        """`hidden += delta (its parts added in order) + other + vector` in place, float32: `other` rows of the stream's
        shape, `vector` one row for all; any of the three may be None.  -> hidden."""

    def assemble_heads(
        self, x: torch.Tensor, q_first: int, k_first: int, v_first: int, heads: int, kv_heads: int, dim: int, vdim: int,
        width: int, norm: str | None, q_weight: torch.Tensor | None, k_weight: torch.Tensor | None, eps: float,
        table: torch.Tensor | None, rot_dims: int, other: torch.Tensor | None = None, other_first: int = 0, blend: float = 0.0,
        batch: Any = None, cell: Any = None, pairing: str = "adjacent",
    ) -> torch.Tensor:
        """From rows that hold `heads` queries and `kv_heads` keys of `dim` and `kv_heads` values of `vdim` (from the
        columns q_first, k_first, v_first): rows [T, (heads + 2 kv_heads) * width] of queries, keys and values of
        `width`, zeros beyond a head's own size.  Queries and keys are RMS-normed (`norm` "head": every head by
        itself, weights of dim; "row": all query heads together and all key heads together, weights as long as
        they; None), then their first `rot_dims` dimensions turned in pairs (`pairing` "adjacent": (2i, 2i + 1); "half":
        (i, i + rot_dims / 2)) by the token's row of `table`
        (float32 [T, rot_dims / 2, 2], cos and sin).  With `other`: v <- (1 - blend) v + blend * other[:, other_first : + kv_heads * vdim].
        With a writable `cell` (and the step's `batch`) the keys and values are also stored in the cell's pages, as
        `rotate_and_store` without a rotation would store them."""

    def scale_heads(self, x: torch.Tensor, heads: int, width: int, gates: torch.Tensor, gate_first: int, squash: str) -> torch.Tensor:
        """x[:, h * width : (h + 1) * width] *= squash(gates[:, gate_first + h]) for every head, in place."""

    def decay_attention(
        self, x: torch.Tensor, q_first: int, k_first: int, v_first: int, heads: int, dim: int, vdim: int, decays: torch.Tensor,
        activation: str, batch: Any, state: torch.Tensor,
    ) -> torch.Tensor:
        """q, k (heads of dim) and v (heads of vdim) are act of x's columns from q_first, k_first, v_first.  Per request
        and head, token by token: S = decay_h S + k v^T; o = S^T q.  `state` float32 [slots, heads, dim, vdim] holds S
        and is updated; decays float32 [heads]; act is "silu" or "none"; x in the run dtype or float32.  -> float32 [T, heads * vdim]."""

    def soft_cap(self, logits: torch.Tensor, cap: float) -> torch.Tensor:
        """cap * tanh(logits / cap), in place (float32)."""

    # ------------------------------------------------------------------ routed experts

    def route(
        self, scores: torch.Tensor, experts: int, correction: torch.Tensor | None, top: int, scale: float, scoring: str,
        groups: int = 1, keep_groups: int = 1, renormalise: bool = False,
    ):
        """s = squash(scores[:, :experts]) (sigmoid of each, or softmax over all); the `top` largest of s + correction (None:
        of s) choose (the lower index among equals), among the experts of the `keep_groups` best of `groups` equal groups of
        neighbours (a group's score is its largest); -> (int32 [T, top] experts, float32 [T, top] weights = scale * s of the
        chosen, with `renormalise` scale * s / (sum of the chosen s + 1e-20))."""

    def prepare_experts(
        self, ups: list[torch.Tensor], downs: list[torch.Tensor], activation: str, gates: list[torch.Tensor] | None = None, limit: float | None = None,
    ) -> Any:
        """With `gates` an expert is down(act(gate x) * (up x)), else down(act(up x)); "limited_swish" (with `gates` and a
        `limit`) is the function of gate and up that `prepare_gated_linear` describes."""

    def expert_feed_forward(
        self, x: torch.Tensor, experts: Any, chosen: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor | None = None,
        gates: torch.Tensor | None = None, gate_column: int = 0,
    ) -> torch.Tensor:
        """sum over a token's chosen experts of weight * down_e(act(up_e x)) (+ sigmoid(gates[:, gate_column]) * shared, or
        + shared where no gates are given), float32 [T, hidden]; the inner rows are rounded to the run dtype between the
        two products."""

    # ------------------------------------------------------------------ copies of the stream, a diagonal recurrence, weighted sums

    def stream_copies(self, hidden: torch.Tensor, copies: int, scale: float) -> torch.Tensor:
        """float32 [T, copies * width]: the rows times `scale`, `copies` times side by side."""

    def stream_norm(
        self, streams: torch.Tensor, pending: Any, read: torch.Tensor, weight: torch.Tensor, eps: float, rows: torch.Tensor | None = None,
    ) -> torch.Tensor:
        """`streams` float32 [T, copies * width].  With `pending` (`.result` float32 [T, width] or partial sums of it, `.mix`
        float32 [copies, copies] from -> to, `.out` float32 [copies]): x_t <- sum_s mix[s, t] x_s + out[t] * result, in place.
        Then u = sum_s read[s] x_s and u * rsqrt(mean(u^2) + eps) * weight in the run dtype.  With `rows` (int32 token rows)
        only those rows are computed and returned, and the copies stay as they are."""

    def gated_recurrence(
        self, u: torch.Tensor, gates: torch.Tensor, gate_bias: torch.Tensor, rates: torch.Tensor, branch: torch.Tensor, branch_first: int,
        activation: str, blocks: int, batch: Any, state: torch.Tensor,
    ) -> torch.Tensor:
        """u [T, width]; gates [T, blocks * (r part | i part)] before their bias (float32, the same layout) and sigmoid;
        a = exp(rates * r); per request, token by token: S <- a S + sqrt(1 - a^2) i u; -> S * act(branch[:, branch_first : +
        width]) in the run dtype.  `state` float32 [slots, width] holds S and is updated."""

    def add_scaled(self, a: torch.Tensor, a_scale: float, b: torch.Tensor | None, b_scale: float) -> torch.Tensor:
        """float32 [T, width]: a_scale * a + b_scale * b, where a and b are float32 results or partial sums [parts, T, width]."""

    def gather_rows(self, hidden: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor) -> torch.Tensor:
        """float32 (hidden + delta)[rows]."""

    def argmax(self, logits: torch.Tensor) -> torch.Tensor: ...

    def sample(
        self, logits: torch.Tensor, temperatures: torch.Tensor, top_ps: torch.Tensor, uniforms: torch.Tensor,
        with_top_p: bool = True,
    ) -> torch.Tensor:
        """One token per row.  `with_top_p=False` promises that no row with a temperature has top_p < 1
        (a library may then leave the search for the kept set out)."""
