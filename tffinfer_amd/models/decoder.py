"""The model skeleton every decoder architecture shares: embedding, a list of
blocks run in the order the configuration gives, final norm, output head.

What a layer is made of and in which order layers run is data from the typed
configuration (``layer_specs``, ``layer_schedule``); this file holds no size
and no constant of any architecture.  The reference wires the same sequence as
graph nodes in src/core/model/qwen3/QWen3Creator.cpp:43-165.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from ..config.base import ModelConfig
from ..parts.base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Part, WeightSpec
from ..parts.embedding import Embedding, OutputHead
from ..weights.loader import check_weights, normalize_stored
from ..weights.random_init import random_tensor


@dataclass
class TensorNames:
    """How an architecture's files name the tensors of the skeleton's parts."""
    embedding: str = "model.embed_tokens"
    layer: str = "model.layers.{i}"
    final_norm: str = "model.norm"
    head: str = "lm_head"
    #: the block's children by the name the files use
    children: dict = field(default_factory=dict)
    #: tensors a file may hold that the model has no use for
    ignorable: tuple = ()


def _leaves(prefix: str, part: Part, rename: dict):
    """(global name prefix, part) for a part and all its sub-parts."""
    yield prefix, part
    for child_name, child in part.children().items():
        yield from _leaves(f"{prefix}.{rename.get(child_name, child_name)}", child, rename)


class DecoderModel:
    def __init__(self, config: ModelConfig, names: TensorNames):
        self.config = config
        self.names = names
        self.dtype = None
        self.device = None
        H, V = config.hidden_size, config.vocab_size
        self.embedding = Embedding(V, H)
        self.blocks = []
        for spec in config.layer_specs():
            mixer = MIXERS.build(spec.mixer)
            ffn = FEED_FORWARDS.build(spec.feed_forward)
            norm_spec = spec.norm
            block = BLOCKS.build(spec.block, mixer=mixer, feed_forward=ffn,
                                 make_norm=lambda s=norm_spec: NORMS.build(s))
            self.blocks.append(block)
        self.schedule = list(config.layer_schedule())
        for call in self.schedule:
            if not 0 <= call.layer < len(self.blocks):
                raise ValueError(f"layer schedule names layer {call.layer}, the model has {len(self.blocks)}")
        self.final_norm = NORMS.build(config.final_norm_spec())
        self.head = OutputHead(V, H, self.embedding if config.tie_word_embeddings else None)

    # ---- weights ---------------------------------------------------------
    def _weighted_parts(self):
        yield self.names.embedding, self.embedding
        for i, block in enumerate(self.blocks):
            yield from _leaves(self.names.layer.format(i=i), block, self.names.children)
        yield self.names.final_norm, self.final_norm
        yield self.names.head, self.head

    def expected_tensors(self) -> dict[str, WeightSpec]:
        out = {}
        for prefix, part in self._weighted_parts():
            for local, spec in part.weight_specs().items():
                out[f"{prefix}.{local}"] = spec
        return out

    def load_tensors(self, found: dict[str, torch.Tensor], dtype: torch.dtype, device,
                     where: str = "") -> None:
        """Checks ``found`` against what the parts expect (one error for all
        that is wrong) and hands every part its tensors."""
        ignorable = set(self.names.ignorable)
        if self.config.tie_word_embeddings:
            head = f"{self.names.head}.weight"
            ignorable.add(head)
            if head in found:
                from .. import log
                log.warning("%s: '%s' is stored but the configuration ties the head to the embedding; "
                            "the stored copy is not used", where or "weights", head)
        check_weights(self.expected_tensors(), found, ignorable, where)
        self.dtype, self.device = dtype, torch.device(device)
        for prefix, part in self._weighted_parts():
            specs = part.weight_specs()
            if specs:
                part.load_weights({local: normalize_stored(found[f"{prefix}.{local}"]) for local in specs},
                                  dtype, self.device)

    def init_random(self, seed: int, dtype: torch.dtype, device, on_device: bool = False) -> None:
        """Seeded random weights without a file.  ``on_device`` draws on the GPU
        (another stream of numbers than the host's, for large models)."""
        self.dtype, self.device = dtype, torch.device(device)
        gen_dev = self.device if on_device else "cpu"
        for prefix, part in self._weighted_parts():
            specs = part.weight_specs()
            if specs:
                ws = {}
                for local, spec in specs.items():
                    t = random_tensor(spec, seed, f"{prefix}.{local}", device=gen_dev)
                    ws[local] = t if spec.init == "norm" else t.to(torch.bfloat16)
                part.load_weights(ws, dtype, self.device)

    def graph_safe(self) -> bool:
        """True if every part launches only kernels that read the step's sizes
        from device tables, so a whole decode step can be captured in one HIP graph."""
        pieces = self.graph_pieces()
        return pieces is not None and len(pieces) == 1

    def _item_graph_safe(self, item) -> bool:
        if item == "embed":
            parts = [self.embedding]
        elif item == "finish":
            parts = [self.final_norm, self.head]
        else:
            parts = [p for _, p in _leaves("", self.blocks[self.schedule[item].layer], {})]
        return all(getattr(p, "graph_safe", False) for p in parts)

    def graph_pieces(self):
        """The step as a list of pieces ``(capturable, items)``: items are "embed", the
        indices of the run order, and "finish" (final norm and head), in order; consecutive
        items that can all be captured in a HIP graph (or that all cannot: a part that loops
        on the host over the step's entries) form a piece.  None when nothing is gained:
        the embedding cannot be captured, or no layer call can."""
        items = ["embed"] + list(range(len(self.schedule))) + ["finish"]
        if not self._item_graph_safe("embed") or not any(self._item_graph_safe(i) for i in items[1:-1]):
            return None
        pieces = []
        for it in items:
            safe = self._item_graph_safe(it)
            if pieces and pieces[-1][0] == safe:
                pieces[-1][1].append(it)
            else:
                pieces.append((safe, [it]))
        return pieces

    # ---- cache needs -----------------------------------------------------
    def call_requirements(self):
        """For every entry of the run order: (cache id, writes, KVCacheSpec or
        None, StateSpec or None)."""
        out = []
        for call in self.schedule:
            mixer = self.blocks[call.layer].mixer
            out.append((call.cache, call.writes_cache, mixer.cache_spec(), mixer.state_spec()))
        return out

    # ---- one step --------------------------------------------------------
    def forward(self, ctx) -> torch.Tensor:
        """Runs the tokens of ``ctx.batch`` and returns float32 logits
        [len(logit_rows), vocab]."""
        items = ["embed"] + list(range(len(self.schedule))) + ["finish"]
        _, _, logits = self.run_items(ctx, items, None, None)
        return logits

    def run_items(self, ctx, items, resid, pending):
        """Runs some consecutive items of the step (see ``graph_pieces``) and returns
        (residual stream, pending term, logits or None).  The residual stream is one float32
        tensor from the embedding on, added to in place; the pending term is what the last
        block returned for the next norm to add."""
        b = ctx.batch
        logits = None
        for it in items:
            if it == "embed":
                resid, pending = self.embedding.forward(ctx, b.token_ids), None
            elif it == "finish":
                if b.num_logit_rows == 0:
                    logits = torch.empty(0, self.config.vocab_size, dtype=torch.float32, device=resid.device)
                else:
                    y = self.final_norm.forward(ctx, resid, pending, rows=b.logit_rows)
                    logits = self.head.forward(ctx, y)
            else:
                call = self.schedule[it]
                pending = self.blocks[call.layer].forward(ctx.for_call(it), resid, pending)
        return resid, pending, logits
