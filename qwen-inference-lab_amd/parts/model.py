"""A causal language model as data: parts, a run order and a tensor-name map."""
from dataclasses import dataclass

import torch

from .base import KVNeed, PagedNeed, StateNeed
from .. import ops


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a block in a step.

    block     index into ``CausalLM.blocks``; an index may appear more than once
    cache_of  None: the entry owns a cache of its mixer's need; an earlier entry's
              position in the schedule: the entry reads that entry's cache and
              writes nothing
    """
    block: int
    cache_of: int | None = None


class CausalLM:
    """embedding -> blocks in schedule order -> final norm -> head.

    names: checkpoint tensor name -> (part, local name).  Every declared tensor of
    every part must be reachable through it, or loading fails.
    tied:  checkpoint names that are accepted as a second name of a tensor, name
    -> canonical name (a tied head: 'lm_head.weight' -> 'model.embed_tokens.weight').
    """

    def __init__(self, *, config, embedding, blocks, schedule, final_norm, head, names, tied=None,
                 dtype=torch.bfloat16, device='cuda'):
        self.config, self.embedding, self.blocks, self.schedule = config, embedding, list(blocks), list(schedule)
        self.final_norm, self.head, self.names, self.tied = final_norm, head, dict(names), dict(tied or {})
        self.dtype, self.device = dtype, torch.device(device)
        for position, entry in enumerate(self.schedule):
            if not 0 <= entry.block < len(self.blocks):
                raise ValueError(f'schedule entry {position} names block {entry.block}, which does not exist')
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < position or self.schedule[entry.cache_of].cache_of is not None:
                    raise ValueError(f'schedule entry {position}: cache_of must name an earlier owning entry')
                if self._need(entry) != self._need(self.schedule[entry.cache_of]):
                    raise ValueError(f'schedule entry {position}: shared cache has another geometry')
        declared = {(id(part), local) for part in self.all_parts() for local in part.param_specs()}
        mapped = {(id(part), local) for part, local in self.names.values()}
        if declared != mapped:
            raise ValueError('tensor-name map does not cover the parts exactly '
                             f'({len(declared - mapped)} unnamed, {len(mapped - declared)} undeclared)')
        self.loaded = False

    def _need(self, entry):
        mixer = self.blocks[entry.block].mixer
        return mixer.cache_need() if mixer is not None else None

    def all_parts(self):
        seen, out = set(), []
        def visit(part):
            if id(part) not in seen:
                seen.add(id(part))
                out.append(part)
        visit(self.embedding)
        for block in self.blocks:
            visit(block)
            for part in block.parts().values():
                visit(part)
        visit(self.final_norm)
        visit(self.head)
        return out

    def cache_needs(self):
        """Per schedule entry: KVNeed | PagedNeed | StateNeed | None, or ('shared', owner position)."""
        needs = []
        for entry in self.schedule:
            need = self._need(entry)
            if need is not None and not isinstance(need, (KVNeed, PagedNeed, StateNeed)):
                raise TypeError(f'unknown cache need {need!r}')
            needs.append(need if entry.cache_of is None or need is None else ('shared', entry.cache_of))
        return needs

    def finalize(self):
        for part in self.all_parts():
            part.finalize()
        self.loaded = True

    def parameter_bytes(self):
        return sum(part.parameter_bytes() for part in self.all_parts())

    @property
    def vocab(self):
        return self.head.vocab

    def forward(self, ctx, caches):
        """Run the step's tokens; float32 logits [len(ctx.logit_rows), vocab] or None.

        Rows are selected before the final norm; with no wanted row neither the
        norm nor the head runs (qil/model.py:130-134).
        """
        stream = self.embedding.forward_step(ctx)
        pending = None
        for entry, cache in zip(self.schedule, caches):
            pending = self.blocks[entry.block].forward(stream, pending, ctx, cache)
        if ctx.n_logit_rows == 0:
            return None
        if isinstance(pending, ops.Added):                      # the last block's output is in the stream already
            pending = None
        rows = self.final_norm.forward_rows(stream, pending, ctx.logit_rows, self.dtype)
        return self.head.forward(rows)
