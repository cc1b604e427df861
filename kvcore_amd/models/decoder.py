"""The generic decoder: builds the parts a ``ModelSpec`` names, owns their parameters,
runs the schedule.

Reference: kvcore/model/models/llama3.py:145-247 (embedding, layer loop, final norm,
head).  Which architecture this is, is decided wholly by the spec.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from kvcore_amd.engine.context import LayerCall, StepContext
from kvcore_amd.ops import library as ops
from kvcore_amd.parts import base as parts
from kvcore_amd.parts.base import CacheNeed, ParamSpec, Part, Runtime, StateNeed

from .spec import ModelSpec


@dataclass(frozen=True)
class CacheGroupSpec:
    """Entries of the schedule whose mixers need the same kind of paged memory share a
    group: one page pool, one block table per request, ``num_planes`` cache planes."""

    need: CacheNeed
    num_planes: int


@dataclass(frozen=True)
class StateArraySpec:
    need: StateNeed


@dataclass
class BoundParam:
    name: str  # full parameter name
    prefix: str  # checkpoint prefix of the owning part
    spec: ParamSpec
    tensor: torch.Tensor


@dataclass
class BuiltParts:
    positions: list
    embed: parts.Embedding
    head: parts.Head
    final_norm: parts.Norm
    blocks: list
    owned: list  # (checkpoint prefix, part), in the order parameters are declared


def build_parts(spec: ModelSpec) -> BuiltParts:
    """Every part that ``spec`` names, from the registries, with its checkpoint prefix.
    Nothing is allocated: the loader uses this to learn a model's checkpoint layout."""
    positions = [parts.POSITION_ENCODINGS.build(p) for p in spec.positions]
    embed = parts.EMBEDDINGS.build(spec.resolved_embedding())
    head = parts.HEADS.build(spec.resolved_head())
    final_norm = parts.NORMS.build(spec.final_norm)
    blocks: list[parts.Block] = []
    for layer in spec.layers:
        position = None if layer.position is None else positions[layer.position]
        mixer = parts.MIXERS.build(layer.mixer, position=position)
        ffn = parts.FEED_FORWARDS.build(layer.ffn)
        norms = {name: parts.NORMS.build(ns) for name, ns in layer.norms.items()}
        blocks.append(parts.BLOCKS.build(layer.block, mixer=mixer, ffn=ffn, norms=norms))
    owned: list[tuple[str, Part]] = [(spec.embed_prefix, embed), (spec.final_norm_prefix, final_norm),
                                     (spec.head_prefix, head)]
    if spec.position_prefixes and len(spec.position_prefixes) != len(positions):
        raise ValueError("position_prefixes must name every position encoding")
    for i, pe in enumerate(positions):
        prefix = spec.position_prefixes[i] if spec.position_prefixes else f"model.positions.{i}"
        owned.append((prefix, pe))
    for layer, block in zip(spec.layers, blocks):
        for sub, part in block.children().items():
            owned.append((f"{layer.prefix}.{sub}", part))
    return BuiltParts(positions, embed, head, final_norm, blocks, owned)


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device: torch.device | str) -> None:
        self.spec = spec
        self.runtime = Runtime(dtype=dtype, device=torch.device(device))
        self.dtype = dtype
        self.device = self.runtime.device

        built = build_parts(spec)
        self.positions = built.positions
        self.embed = built.embed
        self.head = built.head
        self.final_norm = built.final_norm
        self.blocks = built.blocks
        self._owned = built.owned
        for _, part in self._owned:
            part.setup(self.runtime)

        self._plan_caches()
        self.params: dict[str, BoundParam] = {}
        self._allocate_params()

    # ---------------------------------------------------------------- cache planning
    def _plan_caches(self) -> None:
        schedule = self.spec.resolved_schedule()
        group_of: dict[CacheNeed, int] = {}
        planes: list[int] = []
        needs: list[CacheNeed] = []
        states: list[StateArraySpec] = []
        calls: list[LayerCall] = []
        for e, entry in enumerate(schedule):
            if not 0 <= entry.layer < len(self.blocks):
                raise ValueError(f"schedule entry {e} names layer {entry.layer}, which does not exist")
            mixer = self.blocks[entry.layer].mixer
            need = mixer.cache_need()
            g = plane = None
            write = True
            if need is not None:
                if entry.cache_from is not None:
                    if not 0 <= entry.cache_from < e:
                        raise ValueError(f"schedule entry {e}: cache_from must name an earlier entry")
                    src = calls[entry.cache_from]
                    if src.group_index is None or needs[src.group_index] != need:
                        raise ValueError(f"schedule entry {e}: entry {entry.cache_from} has no cache "
                                         "of the shape this layer reads")
                    g, plane, write = src.group_index, src.cache_index, False
                else:
                    if need not in group_of:
                        group_of[need] = len(needs)
                        needs.append(need)
                        planes.append(0)
                    g = group_of[need]
                    plane = planes[g]
                    planes[g] += 1
            state_need = mixer.state_need()
            state_index = None
            if state_need is not None:
                state_index = len(states)
                states.append(StateArraySpec(state_need))
            calls.append(LayerCall(e, entry.layer, g, plane, write, state_index))
        self.calls = calls
        self.cache_groups = [CacheGroupSpec(n, c) for n, c in zip(needs, planes)]
        self.state_arrays = states

    # -------------------------------------------------------------------- parameters
    def _allocate_params(self) -> None:
        kinds = {"matrix": self.dtype, "vector": torch.float32, "table": torch.int32}
        for prefix, part in self._owned:
            local: dict[str, torch.Tensor] = {}
            for ps in part.param_specs():
                t = torch.empty(ps.shape, dtype=kinds[ps.kind], device=self.device)
                full = f"{prefix}.{ps.name}"
                if full in self.params:
                    raise ValueError(f"parameter {full} is declared twice")
                self.params[full] = BoundParam(full, prefix, ps, t)
                local[ps.name] = t
            part.bind(local)
        if self.head.tied:
            if "weight" not in self.embed.params:
                raise ValueError("a tied head needs an embedding with a parameter named 'weight'")
            self.head.bind({**self.head.params, "weight": self.embed.params["weight"]})

    def checkpoint_map(self) -> dict[str, tuple[BoundParam, int, int]]:
        """Checkpoint tensor name -> (parameter, first row, rows)."""
        out: dict[str, tuple[BoundParam, int, int]] = {}
        for bp in self.params.values():
            for src in bp.spec.resolved_sources():
                out[f"{bp.prefix}.{src.name}"] = (bp, src.row, src.rows)
        return out

    def optional_checkpoint_names(self) -> set[str]:
        """Names a file may hold that are not read: a tied head's own matrix
        (reference: kvcore/model/model_utils.py:51-53)."""
        if self.head.tied:
            return {f"{self.spec.head_prefix}.weight"}
        return set()

    def graph_safe(self) -> bool:
        """True iff every part says its forward may be captured into a HIP graph (it reads
        nothing from the device and decides nothing on the host per step)."""
        owned = [part for _, part in self._owned] + list(self.blocks)
        return all(getattr(part, "graph_safe", True) for part in owned)

    def num_param_bytes(self) -> int:
        return sum(bp.tensor.numel() * bp.tensor.element_size() for bp in self.params.values())

    # ------------------------------------------------------------------ packed copies
    def product_weights(self) -> list[torch.Tensor]:
        """The matrices that the parts stream in decode steps and that can be packed, each once
        (a tied head names the embedding's)."""
        seen: dict[int, torch.Tensor] = {}
        for _, part in self._owned:
            for name in part.product_weights():
                t = part.params.get(name)
                if t is not None and ops.can_pack_weight(t):
                    seen.setdefault(id(t), t)
        return list(seen.values())

    def pack_product_weights(self, enable: bool | None = None, budget: int | None = None) -> int:
        """Give the matrices that decode steps stream their packed twins (``ops.pack_weight``);
        returns the bytes taken.  ``enable`` None decides by room.  All of them, if the copies
        fit in a quarter of the device's memory and leave half of what is free now.  Else only
        the matrices that gain most from it, within an eighth of the device's memory and a
        quarter of what is free (``budget`` overrides that): those whose rows lie a multiple of
        16 KB apart, which a row-major walk reads through the same few memory channels
        (measured at 8 rows: 10240 x 8192 row-major 42.7 us, packed 36.0; 8192 x 8192 28.8 and
        26.3; 8192 x 28672, whose rows lie 56 KB apart, 80.4 and 78.7), all matrices of a shape
        or none, the small shapes first.
        A model that fills the device this way keeps the rest as they are.  The products give the
        same bits from a matrix and from its packed copy.  Call again after the weights changed."""
        if self.device.type != "cuda" or self.dtype != torch.bfloat16:
            return 0
        weights = self.product_weights()
        need = sum(w.numel() * w.element_size() for w in weights)
        chosen = weights
        if enable is None:
            free, total = torch.cuda.mem_get_info(self.device)
            already = sum(w.kvc_packed.numel() * 2 for w in weights if getattr(w, "kvc_packed", None) is not None)
            free += already
            if budget is None and need <= total // 4 and need <= free // 2:
                enable = True
            else:
                room = min(total // 8, free // 4) if budget is None else budget
                chosen = []
                shapes: dict[tuple[int, ...], list[torch.Tensor]] = {}
                for w in weights:  # all matrices of a shape or none: every layer runs alike
                    if (w.shape[1] * w.element_size()) % 16384 == 0:
                        shapes.setdefault(tuple(w.shape), []).append(w)
                for shape, group in sorted(shapes.items(), key=lambda kv: kv[0][0] * kv[0][1]):
                    size = sum(w.numel() * w.element_size() for w in group)
                    if size <= room:
                        chosen.extend(group)
                        room -= size
                enable = bool(chosen)
        keep = {id(w) for w in chosen} if enable else set()
        for w in weights:
            if id(w) not in keep and hasattr(w, "kvc_packed"):
                del w.kvc_packed
        taken = 0
        for w in weights:
            if id(w) in keep:
                if getattr(w, "kvc_packed", None) is None:
                    ops.pack_weight(w)
                taken += w.numel() * w.element_size()
        return taken

    # ----------------------------------------------------------------------- forward
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """Normalised hidden rows ``[T, H]`` in the model dtype for the batch in ``ctx``."""
        H = self.spec.hidden_size
        residual = ctx.buf("residual", H, torch.float32)
        self.embed.forward(residual, ctx.token_ids[: ctx.num_tokens])
        for pe in self.positions:
            pe.prepare(ctx)
            pe.embed(residual, ctx)
        delta = None
        for i, call in enumerate(self.calls):
            nxt = self.blocks[self.calls[i + 1].layer_index] if i + 1 < len(self.calls) else None
            delta = self.blocks[call.layer_index].forward(delta, residual, ctx, call, next_block=nxt)
        hidden = ctx.buf("final_hidden", H)
        self.final_norm.forward_fused(hidden, residual, delta)
        return hidden

    def compute_logits(self, ctx: StepContext, hidden: torch.Tensor, rows: torch.Tensor,
                       num_rows: int, every_row: bool = False) -> torch.Tensor:
        """float32 ``[S, V]`` at the flattened token indices ``rows[:S]``; ``every_row`` says
        that these are simply all ``S`` rows of ``hidden`` in order, which saves the copy."""
        H, V = self.spec.hidden_size, self.spec.vocab_size
        # a row per request that samples, as a rule: room for all of them at once, so that a
        # batch that fills up step by step does not make these grow (and drop the graphs)
        room = ctx.buffers.seq_capacity
        if every_row and hidden.shape == (num_rows, H) and hidden.dtype == self.dtype and hidden.is_contiguous():
            picked = hidden
        else:
            picked = ctx.buffers.get("head_rows", num_rows, H, self.dtype, reserve=room)
            ops.gather_rows(picked, hidden, rows[:num_rows])
        logits = ctx.buffers.get("logits", num_rows, V, torch.float32, reserve=room)
        self.head.forward(logits, picked, ctx)
        return logits
