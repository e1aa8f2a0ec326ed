"""Attention over a sliding window that also keeps the first tokens of the sequence, with a sink.

q = h Wq^T, k = h Wk^T, v = h Wv^T without biases; keys are `key_dim` wide, values `value_dim` (they may
differ); query head h reads kv head h // (heads / kv_heads).  Position i sees position j when j <= i and
(i - j < window or j < keep_first); window = 0 means every earlier position.  With `sink` the softmax has one
more term in its denominator, a key of score 0 that carries no value: p_j = e^(s_j) / (1 + sum e^(s_j)), so a
query may look at nothing (Xiao, Tian, Chen, Han, Lewis: "Efficient Streaming Language Models with Attention
Sinks" keeps first tokens for the same purpose).  `sink="learned"`: the term is e^(b_h) with a stored number b_h for
every query head (`<prefix>.sink`), which is not scaled: p_j = e^(s_j) / (e^(b_h) + sum e^(s_j)).  With `head_gate` every head's result is multiplied by the
sigmoid of one more projection of h, a number per head.  Scores, probabilities and the sums over values are
32-bit whatever the run's dtype.  A position encoding is optional (`position=None`: positions do not enter
the scores).

`rotary` (a mapping: `dims`, `base`, optionally `scaling` as `rope.rotary_frequencies` takes it and `pairing`,
"interleaved" or "half") rotates the first `dims` entries of every query and key head by the position, the rest
pass; `qk_norm_eps` then divides every query and key head by its root mean square over key_dim (no weight).  Both
are taken in 32-bit on the product's 32-bit result, by one kernel that also leaves q, k and v in the dtype of the
cache.

`probabilities="bfloat16"` says that a design lets the softmax's weights be rounded to bfloat16 as operands of their
product with the values (the sums stay 32-bit): plain causal attention with keys and values of one size then runs, in
a bfloat16 run, on the causal kernel of the matrix cores, several times as fast over a prompt.  The default keeps the
weights 32-bit through that product.

All projections of h are one matrix product ([q | k | v | gate]).
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import (MIXERS, POSITION_ENCODINGS, VECTOR32, BuildEnv, KVNeed, LayerCache, Mixer, PartSpec, StepContext,
                   TensorSpec, build_part, product_weight, project)
from .rope import rotary_frequencies, rotary_magnitude


def split_scratch(ctx: StepContext, dtype, heads: int, kv_heads: int, key_dim: int, value_dim: int, block_size: int,
                  window: int, keep_first: int) -> Dict[str, object]:
    """The keywords with which `sink_attention` may share a decoding step's keys out over several workgroups a tile:
    the step's bound of the lengths and the scratch that the kernel object asks for (nothing where it asks for none)."""
    ask = getattr(ctx.kernels, "sink_attention_workspace", None)
    if ask is None or not ctx.decode:
        return {}
    need = ask(dtype, ctx.rows, ctx.batch, heads, kv_heads, key_dim, value_dim, block_size, window, keep_first, ctx.max_len)
    return dict(max_len=ctx.max_len, workspace=ctx.ws.alloc((need,), torch.float32)) if need else {}


@MIXERS.register("sink_window_attention")
class SinkWindowAttention(Mixer):
    takes_out = True

    def __init__(self, width: int, heads: int, kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 prefix: str, window: int = 0, keep_first: int = 0, sink=True, head_gate: bool = False,
                 position: Optional[PartSpec] = None, rotary: Optional[Mapping] = None,
                 qk_norm_eps: Optional[float] = None, names: Optional[Mapping[str, str]] = None,
                 probabilities: str = "float32") -> None:
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} heads cannot share {kv_heads} kv heads evenly")
        self.rot_dims, self.rot_interleaved, self.rot_magnitude, self.freq_table = 0, False, 1.0, []
        if rotary is not None:
            if position is not None:
                raise ValueError("a position encoding part or the `rotary` parameters, not both")
            self.rot_dims = int(rotary["dims"])
            pairing = rotary.get("pairing", "interleaved")
            if pairing not in ("half", "interleaved"):
                raise ValueError(f"rotary pairing {pairing!r} is not known (known: 'half', 'interleaved')")
            if self.rot_dims % 2 or not 2 <= self.rot_dims <= int(key_dim):
                raise ValueError(f"{self.rot_dims} rotated entries do not fit a head of {key_dim}")
            scaling = dict(rotary["scaling"]) if rotary.get("scaling") else None
            self.rot_interleaved = pairing == "interleaved"
            self.freq_table = rotary_frequencies(self.rot_dims, float(rotary["base"]), scaling)
            self.rot_magnitude = rotary_magnitude(scaling)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.prepared = rotary is not None or qk_norm_eps is not None  # q, k and v pass the kernel named above
        if self.prepared and head_gate:
            raise ValueError("a gate per head and a rotation or norm of q and k are not combined")
        if window < 0 or keep_first < 0:
            raise ValueError("window and keep_first must not be negative")
        self.width, self.heads, self.kv_heads = int(width), int(heads), int(kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.window, self.keep_first = float(scale), int(window), int(keep_first)
        if sink not in (True, False, "learned"):
            raise ValueError(f"the sink is True (a score of 0), False or 'learned' (a stored score a head), found {sink!r}")
        self.sink, self.head_gate, self.learned_sink = bool(sink), bool(head_gate), sink == "learned"
        self.sink_w: Optional[torch.Tensor] = None
        if probabilities not in ("float32", "bfloat16"):
            raise ValueError(f"probabilities are 'float32' or 'bfloat16', found {probabilities!r}")
        self.probabilities = probabilities
        n = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "sink": "sink"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.position = build_part(POSITION_ENCODINGS, position) if position is not None else None
        self.q_width = self.heads * self.key_dim
        self.k_width = self.kv_heads * self.key_dim
        self.v_width = self.kv_heads * self.value_dim
        self.o_width = self.heads * self.value_dim
        self.w_in: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    @property
    def graph_safe(self) -> bool:
        return self.position is None or self.position.graph_safe

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [
            TensorSpec(self.names["q"], (self.q_width, self.width)),
            TensorSpec(self.names["k"], (self.k_width, self.width)),
            TensorSpec(self.names["v"], (self.v_width, self.width)),
        ]
        if self.head_gate:
            specs.append(TensorSpec(self.names["gate"], (self.heads, self.width)))
        if self.learned_sink:
            specs.append(TensorSpec(self.names["sink"], (self.heads,), kind=VECTOR32))
        specs.append(TensorSpec(self.names["o"], (self.width, self.o_width)))
        return specs + (self.position.tensor_specs() if self.position is not None else [])

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        mats = [tensors[self.names[key]] for key in ("q", "k", "v") + (("gate",) if self.head_gate else ())]
        if len({m.dtype for m in mats}) != 1:
            raise ValueError(f"{self.names['q']}: the projections of one input are stored in different dtypes")
        self.w_in = product_weight(env, torch.cat(mats, dim=0))
        self.w_o = product_weight(env, tensors[self.names["o"]])
        if self.learned_sink:
            self.sink_w = tensors[self.names["sink"]].contiguous()
        if self.position is not None:
            self.position.bind(tensors, env)
        self.freqs = torch.tensor(self.freq_table, dtype=torch.float64, device=env.device) if self.rot_dims else None

    def cache_need(self) -> KVNeed:
        # a window that keeps first tokens still gives its middle blocks back
        return KVNeed(self.kv_heads, self.key_dim, self.window, self.value_dim, self.keep_first if self.window else 0)

    def lengths_uneven(self, kernels, lengths) -> bool:
        ask = getattr(kernels, "decode_lengths_uneven", None)
        plain = not (self.sink or self.head_gate or self.keep_first or self.window) and self.key_dim == self.value_dim \
            and self.probabilities == "bfloat16"
        return bool(ask(lengths)) if ask is not None and plain else False

    def _plain_causal(self, kn, ctx: StepContext, cache: LayerCache) -> bool:
        """Whether this step's attention is the causal kernel's (`attention`): the design lets the probabilities be
        rounded to bfloat16 for their product with the values (that kernel's way; the general kernel keeps them
        32-bit), the mask and softmax are plain, and the kernel object runs the shape on its matrix cores."""
        if self.probabilities != "bfloat16" or self.sink or self.head_gate or self.keep_first \
                or self.key_dim != self.value_dim:
            return False
        ask = getattr(kn, "attention_on_matrix_cores", None)
        return ask is not None and bool(ask(ctx.dtype, self.heads, self.kv_heads, self.key_dim, cache.block_size))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache],
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cache is None or cache.k is None:
            raise RuntimeError("attention needs a key/value cache")
        kn = ctx.kernels
        rows = h.shape[0]
        total = self.q_width + self.k_width + self.v_width + (self.heads if self.head_gate else 0)
        total_padded = (total + 3) // 4 * 4  # rows of the product start on 16 bytes
        if self.prepared:
            # the product's 32-bit result is rotated and normed in 32-bit, then rounded to what the cache holds
            proj = ctx.ws.alloc((rows, total_padded), torch.float32)[:, :total]
            project(kn, ctx, h, self.w_in, proj)
            q = ctx.ws.alloc((rows, self.q_width), ctx.dtype)
            k = ctx.ws.alloc((rows, self.k_width), ctx.dtype)
            v = ctx.ws.alloc((rows, self.v_width), ctx.dtype)
            gate = None
            kn.rotary_qkv(proj, q, k, v, self.heads, self.kv_heads, self.key_dim, self.value_dim, self.rot_dims,
                          self.rot_interleaved, self.freqs, self.rot_magnitude, self.qk_norm_eps, ctx.row_pos)
        else:
            # q, k and v in the run's dtype (what the cache holds); the gate's logits ride in the same product
            proj = ctx.ws.alloc((rows, total_padded), ctx.dtype)[:, :total]
            project(kn, ctx, h, self.w_in, proj)
            q = proj[:, : self.q_width]
            k = proj[:, self.q_width : self.q_width + self.k_width]
            v = proj[:, self.q_width + self.k_width : self.q_width + self.k_width + self.v_width]
            gate = proj[:, self.q_width + self.k_width + self.v_width :] if self.head_gate else None
            if self.position is not None:
                self.position.apply(q, k, ctx)
        if cache.write:
            kn.kv_store(k, v, self.kv_heads, self.key_dim, self.value_dim, ctx.row_pos, ctx.row_seq, ctx.seq_slot,
                        cache.block_table, cache.k, cache.v, cache.block_size)
        att = ctx.ws.alloc((rows, self.o_width), ctx.dtype)
        if self._plain_causal(kn, ctx, cache):
            # no sink, gate or kept first tokens, keys and values of one size: the causal kernel on the matrix cores
            need = kn.attention_workspace(ctx.dtype, rows, self.heads, self.kv_heads, self.key_dim, cache.block_size,
                                          ctx.decode, ctx.max_len)
            kn.attention(q, att, self.heads, self.kv_heads, self.key_dim, ctx.row_pos, ctx.row_seq, ctx.seq_slot,
                         ctx.cu_rows, cache.block_table, cache.k, cache.v, cache.block_size, self.scale, self.window,
                         decode=ctx.decode, max_len=ctx.max_len,
                         workspace=ctx.ws.alloc((need,), torch.float32) if need else None, uneven=ctx.uneven)
            if out is None:
                out = ctx.ws.alloc((rows, self.width), torch.float32)
            project(kn, ctx, att, self.w_o, out)
            return out
        kn.sink_attention(q, att, self.heads, self.kv_heads, self.key_dim, self.value_dim, ctx.row_pos, ctx.row_seq,
                          ctx.seq_slot, cache.block_table, cache.k, cache.v, cache.block_size, self.scale,
                          window=self.window, keep_first=self.keep_first, sink=self.sink, gate=gate,
                          decode=ctx.decode, **({"sink_values": self.sink_w} if self.learned_sink else {}),
                          **split_scratch(ctx, q.dtype, self.heads, self.kv_heads, self.key_dim,
                                                             self.value_dim, cache.block_size, self.window,
                                                             self.keep_first))
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, att, self.w_o, out)
        return out
