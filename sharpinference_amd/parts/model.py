"""The whole decoder: embedding, a list of blocks, the order they run in, final norm, head."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..ops.profile import section
from .base import LayerCache, ParamSpec, Part, ResidualStream, StepContext, TensorSource
from .norm import RMSNorm


@dataclass(frozen=True)
class Run:
    """One entry of the execution order: run `layer` with cache slot `cache`.

    A layer may appear in several entries (its weights are used again; give each entry its own
    cache slot unless sharing is meant).  ``write=False`` makes the entry read the keys and
    values that the slot's owner stored earlier in the same step and store nothing."""

    layer: int
    cache: int
    write: bool = True


class DecoderModel(Part):
    """tokens -> embedding rows (times ``embedding_scale``; 1 for this architecture; reference:
    src/SharpInference.Engine/ForwardPass.cs:1478-1483) -> blocks in the order of ``schedule`` ->
    final norm -> logits through the head, which is the embedding table when tied
    (ForwardPass.cs:1741-1747, 410-413), times ``logit_scale`` and softly capped at
    ``logit_softcap`` (cap * tanh(x / cap), reference: src/SharpInference.Cpu/SimdKernels.cs:4490-4530)
    where an architecture has them."""

    def __init__(self, vocab_size: int, hidden: int, blocks: Sequence[Part], final_norm: RMSNorm,
                 schedule: Optional[Sequence[Run]] = None, tie_embeddings: bool = False, config=None,
                 layer_prefix: str = "model.layers.", embed_name: str = "model.embed_tokens.weight",
                 norm_prefix: str = "model.norm.", head_name: str = "lm_head.weight", embedding_scale: float = 1.0,
                 logit_scale: float = 1.0, logit_softcap: Optional[float] = None):
        self.vocab_size, self.hidden = int(vocab_size), int(hidden)
        self.blocks = list(blocks)
        self.final_norm = final_norm
        self.schedule: List[Run] = list(schedule) if schedule is not None else [Run(i, i) for i in range(len(self.blocks))]
        self.tie_embeddings = bool(tie_embeddings)
        self.embedding_scale, self.logit_scale = float(embedding_scale), float(logit_scale)
        self.logit_softcap = float(logit_softcap) if logit_softcap else 0.0
        if self.logit_softcap < 0:
            raise ValueError("logit_softcap must be positive (or None)")
        self.config = config
        self.layer_prefix, self.embed_name, self.norm_prefix, self.head_name = layer_prefix, embed_name, norm_prefix, head_name
        self.embed: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self._check_schedule()

    def _check_schedule(self) -> None:
        n_slots = self.num_cache_slots()
        owner: Dict[int, int] = {}
        for r in self.schedule:
            if not 0 <= r.layer < len(self.blocks):
                raise ValueError(f"schedule names layer {r.layer}; the model has {len(self.blocks)}")
            if not 0 <= r.cache < n_slots:
                raise ValueError(f"schedule names cache slot {r.cache} out of range")
            spec = self.blocks[r.layer].cache_spec()
            if r.write:
                if r.cache in owner:
                    raise ValueError(f"cache slot {r.cache} is written by two entries of the schedule")
                owner[r.cache] = r.layer
            else:
                if r.cache not in owner:
                    raise ValueError(f"cache slot {r.cache} is read before any entry has written it")
                if self.blocks[owner[r.cache]].cache_spec() != spec:
                    raise ValueError(f"layer {r.layer} reads the cache of layer {owner[r.cache]}, whose shape differs")

    # -- cache ------------------------------------------------------------------
    def num_cache_slots(self) -> int:
        return 1 + max((r.cache for r in self.schedule), default=-1)

    def cache_specs(self) -> list:
        """Per cache slot, what its owner asks of the cache manager."""
        specs = [None] * self.num_cache_slots()
        for r in self.schedule:
            if r.write:
                specs[r.cache] = self.blocks[r.layer].cache_spec()
        return specs

    def decode_graph_safe(self) -> bool:
        return all(getattr(b, "decode_graph_safe", lambda: True)() for b in self.blocks)

    def step_planners(self):
        """The planners of the parts in the order they first appear, one per key."""
        out: dict = {}
        for b in self.blocks:
            for pl in getattr(b, "step_planners", tuple)():
                if not pl.key:
                    raise ValueError(f"{type(pl).__name__}: a step planner needs a key")
                out.setdefault(pl.key, pl)
        return list(out.values())

    # -- weights ------------------------------------------------------------------
    def param_specs(self, prefix: str = "") -> Dict[str, ParamSpec]:
        out = {self.embed_name: ParamSpec((self.vocab_size, self.hidden))}
        for i, b in enumerate(self.blocks):
            out.update(b.param_specs(f"{self.layer_prefix}{i}."))
        out.update(self.final_norm.param_specs(self.norm_prefix))
        if not self.tie_embeddings:
            out[self.head_name] = ParamSpec((self.vocab_size, self.hidden))
        return out

    def load_weights(self, source: TensorSource) -> None:
        self.embed = source.get(self.embed_name)
        for i, b in enumerate(self.blocks):
            b.load(f"{self.layer_prefix}{i}.", source)
        self.final_norm.load(self.norm_prefix, source)
        # the head also in the order the few-rows kernel streams it (the rows stay for many-row steps
        # and, when tied, for the embedding gather)
        self.head = ops.pack_weight(self.embed if self.tie_embeddings else source.get(self.head_name))

    # -- compute ------------------------------------------------------------------
    def forward(self, ctx: StepContext, caches: Sequence[LayerCache], logit_rows: Optional[torch.Tensor],
                select: Optional[str] = None) -> Optional[torch.Tensor]:
        """Run the step's tokens through every entry of the schedule.  Returns float32 logits
        [len(logit_rows), vocab], or None if no row is wanted.  With ``select="argmax"`` the
        largest logit's index per wanted row is returned instead (int32 [rows], the lowest index
        on a tie), chosen on the device right behind the head: the logits then never leave it
        (the reference keeps such a path for all-greedy batches,
        src/SharpInference.Engine/CudaForwardPass.cs:1574-1583)."""
        with section("embed", nbytes=ctx.n_tokens * self.hidden * 6):
            stream = ResidualStream(ops.embed_gather(ctx.token_ids, self.embed, scale=self.embedding_scale))
        for r in self.schedule:
            c = caches[r.cache]
            if not r.write:
                c = LayerCache(c.group, c.k, c.v, c.state, write=False)
            self.blocks[r.layer].forward(stream, ctx, c)
        if logit_rows is None or logit_rows.numel() == 0:
            return None
        n = self.final_norm.forward(stream, ctx.act_dtype, rows=logit_rows)
        m = n.shape[0]
        with section("head", nbytes=2 * self.vocab_size * self.hidden + 4 * m * self.vocab_size, flops=2.0 * m * self.vocab_size * self.hidden):
            logits = ops.linear(n, self.head, torch.float32)
            if self.logit_scale != 1.0 or self.logit_softcap:
                ops.scale_softcap(logits, self.logit_scale, self.logit_softcap)
        if select is None:
            return logits
        if select == "argmax":
            with section("select", nbytes=4 * m * self.vocab_size):
                return ops.argmax_rows(logits)
        raise ValueError(f"select {select!r} is not known (None for logits, 'argmax')")
