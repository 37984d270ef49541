"""A decoder model as data: an embedding, a list of layers, the order in which
they run, a final norm and an output head.

`schedule` is a list of ScheduleEntry.  An entry names the layer to run; the
same layer may be named twice (its weights are shared, every run has a cache
of its own), and an entry may say `reads` = index of an earlier entry, in which
case it keeps no cache and attends to what that entry wrote.  Cache *sites* are
schedule indices.  The reference's model is the fixed loop of
runtime/model.py:106-120; here the loop is over the schedule.
"""
from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class ScheduleEntry:
    layer: int
    reads: Optional[int] = None  # schedule index whose cache this run reads instead of keeping its own


class Model:
    def __init__(self, config, embedding, layers, final_norm, head, schedule=None, max_positions=None, vocab_size=None):
        """`max_positions` (the context limit) and `vocab_size`: given by the builder, or read from the
        configuration's fields `max_position_embeddings` and `vocab_size` if it has them under these names."""
        self.config = config
        self._max_positions = max_positions if max_positions is not None else getattr(config, "max_position_embeddings", None)
        self._vocab_size = vocab_size if vocab_size is not None else getattr(config, "vocab_size", None)
        if self._max_positions is None or self._vocab_size is None:
            raise ValueError("a model needs max_positions and vocab_size (arguments, or fields of its configuration)")
        self.embedding, self.layers, self.final_norm, self.head = embedding, list(layers), final_norm, head
        self.schedule = list(schedule) if schedule is not None else [ScheduleEntry(i) for i in range(len(self.layers))]
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {index} names layer {entry.layer}, which does not exist")
            if entry.reads is not None:
                if not 0 <= entry.reads < index or self.schedule[entry.reads].reads is not None:
                    raise ValueError(f"schedule entry {index} must read an earlier entry that keeps a cache")
                if self.layers[entry.layer].cache_need() is not None:
                    raise ValueError(f"schedule entry {index} reads another cache but its mixer keeps one")
                kept = self.layers[self.schedule[entry.reads].layer].cache_need()
                reader = self.layers[entry.layer]
                wanted = reader.cache_read() if hasattr(reader, "cache_read") else None
                if kept is None:
                    raise ValueError(f"schedule entry {index} reads entry {entry.reads}, which keeps no cache")
                if wanted is not None:
                    if (wanted.kv_heads, wanted.head_dim) != (kept.kv_heads, kept.head_dim):
                        raise ValueError(f"schedule entry {index} expects keys of {wanted.kv_heads} heads x {wanted.head_dim}, "
                                         f"entry {entry.reads} keeps {kept.kv_heads} x {kept.head_dim}")
                    if kept.window is not None and (wanted.window is None or wanted.window > kept.window):
                        raise ValueError(f"schedule entry {index} looks back over {wanted.window or 'all'} keys, "
                                         f"entry {entry.reads} keeps the last {kept.window}")
        self.dtype = None
        self.device = None

    # -- weights ------------------------------------------------------------
    def parts(self):
        return [self.embedding, *self.layers, self.final_norm, self.head]

    def tensor_specs(self):
        specs, seen = [], set()
        for part in self.parts():
            for spec in part.tensor_specs():
                if spec.name in seen:
                    raise ValueError(f"tensor {spec.name} is declared twice")
                seen.add(spec.name)
                specs.append(spec)
        return specs

    def ignored_tensors(self):
        """Names a checkpoint may hold that the model does not read: the copy of a tied head
        (the reference overwrites it with the embedding, runtime/checkpoint.py:38-39)."""
        tied = getattr(self.head, "tied_to", None)
        return (self.head.name + ".weight",) if tied is not None else ()

    def bind(self, tensors, dtype, device):
        self.dtype, self.device = dtype, device
        for part in self.parts():
            part.bind(tensors, dtype)
            part.prepare(device, dtype)

    # -- what the cache manager must provide ------------------------------------
    def site_of(self, index):
        entry = self.schedule[index]
        return index if entry.reads is None else entry.reads

    def cache_needs(self):
        needs = {}
        for index, entry in enumerate(self.schedule):
            need = self.layers[entry.layer].cache_need()
            if need is not None and entry.reads is None:
                needs[index] = need
        return needs

    def state_needs(self):
        needs = {}
        for index, entry in enumerate(self.schedule):
            need = self.layers[entry.layer].state_need()
            if need is not None:
                needs[index] = need
        return needs

    def kernel_units(self):
        """Shared objects beside the core that the model's parts need for its compute dtype."""
        return [u for part in self.parts() if hasattr(part, "kernel_units") for u in part.kernel_units(self.dtype)]

    def step_arrays(self):
        """Step arrays that the parts want every step's metadata to carry from the start."""
        return [a for part in self.parts() if hasattr(part, "step_arrays") for a in part.step_arrays()]

    @property
    def max_positions(self):
        return self._max_positions

    @property
    def vocab_size(self):
        return self._vocab_size

    # -- the forward pass over one step's rows ------------------------------------
    def forward(self, ctx):
        """Logits [R, vocab] (float) at ctx.logit_rows; None if no row is wanted
        (the layers still run: they fill the cache)."""
        x = self.embedding.forward(ctx)
        last = len(self.schedule) - 1
        for index, entry in enumerate(self.schedule):
            # a block may leave its last product to the norm that reads the residual stream next, if that block names one
            following = self.layers[self.schedule[index + 1].layer] if index < last else None
            ctx.next_norm = following.first_norm() if hasattr(following, "first_norm") else None
            x = self.layers[entry.layer].forward(x, ctx, self.site_of(index))
            ctx.next_norm = None
            if following is None or not hasattr(following, "first_norm"):
                ctx.settle(x)
        if ctx.logit_rows.shape[0] == 0:
            return None
        if self.head.fuses_norm(self.final_norm, x, ctx.logit_rows):
            return self.head.forward(None, ctx, norm=self.final_norm, residual=x)
        h = self.final_norm.forward(x, ctx, rows=ctx.logit_rows, tag="final_norm")
        return self.head.forward(h, ctx)
