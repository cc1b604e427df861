"""What one step hands to the parts: the flattened batch, the caches and tables, the
per-request state slots and a pool of step buffers.

The reference reaches the same record through a context variable
(kvcore/model/forward_context.py:12-40, kvcore/model/kv_runtime.py:10-26); here it is
an argument, so a part's inputs are visible in its signature.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass(frozen=True)
class LayerCall:
    """One entry of the model's schedule: which layer runs, which cache it uses.

    ``cache_index`` addresses the cache planes of this entry's group (None: the layer's
    mixer keeps no paged cache); ``write_cache`` is False when the entry reads the cache
    another entry wrote.  ``state_index`` addresses the layer's fixed-size state array.
    """

    exec_index: int
    layer_index: int
    group_index: int | None = None
    cache_index: int | None = None
    write_cache: bool = True
    state_index: int | None = None


@dataclass
class CacheGroupView:
    """Device side of one cache group.  ``storage[p]`` holds plane ``p`` of the group's need
    for every schedule entry of the group: ``[entries, pages, page_size * elements a token]``,
    a page being one contiguous row.  ``table`` is ``[max_seqs, max_pages_per_seq]`` int32,
    row = request slot, entry = page id (0 is the null page)."""

    storage: list[torch.Tensor]
    table: torch.Tensor
    page_size: int
    window: int = 0

    @property
    def num_pages(self) -> int:
        return self.storage[0].shape[1]

    def plane(self, cache_index: int, plane: int, *page_shape: int) -> torch.Tensor:
        """The pages of one plane of one schedule entry: ``[pages, *page_shape]`` (a view;
        ``page_shape`` must hold ``page_size`` tokens' worth of the plane, and defaults to one
        flat row a page).  Attention views its keys as ``(kv_heads, page_size, head_dim)`` and
        its values as ``(kv_heads, head_dim, page_size)``: a V page keeps the keys contiguous."""
        views = self.__dict__.setdefault("_plane_views", {})
        key = (cache_index, plane, page_shape)
        got = views.get(key)
        if got is None:
            flat = self.storage[plane][cache_index]
            got = flat.view(flat.shape[0], *page_shape) if page_shape else flat
            views[key] = got
        return got


class StepBuffers:
    """Named device buffers that live across steps, so a step allocates nothing once
    the largest batch has been seen.  ``get`` returns a view of the first ``rows`` rows.

    Buffers indexed by token are allocated for ``token_capacity`` rows at once, buffers with
    a row per request that samples for ``seq_capacity`` rows (``reserve`` of ``get``).  A
    buffer that still has to grow is replaced by a new tensor; ``on_grow`` is then called
    first, because a captured graph holds the old address."""

    def __init__(self, device: torch.device, token_capacity: int = 0, on_grow=None,
                 seq_capacity: int = 0) -> None:
        self.device = device
        self.token_capacity = token_capacity
        self.seq_capacity = seq_capacity
        self.on_grow = on_grow
        self._store: dict[str, torch.Tensor] = {}
        self.frozen = False

    def get(self, name: str, rows: int, cols: int, dtype: torch.dtype, reserve: int = 0) -> torch.Tensor:
        buf = self._store.get(name)
        if buf is None or buf.dtype != dtype or buf.shape[1] != cols or buf.shape[0] < rows:
            if self.frozen:
                raise RuntimeError(
                    f"step buffer {name!r} would have to grow to {rows}x{cols} while a graph is "
                    "being captured")
            if buf is not None and self.on_grow is not None:
                self.on_grow()
            buf = torch.empty((max(rows, reserve, 1), cols), dtype=dtype, device=self.device)
            self._store[name] = buf
        return buf[:rows]


@dataclass
class StepContext:
    """One step's batch, flattened.  All index tensors are int32 on the device.

    ``token_req[t]`` is the index of token ``t``'s request within this step (−1 marks a
    padding token); ``slots[r]`` is request ``r``'s slot: its row in every block table
    and state array (``token_rows[t]``, if given, is ``slots[token_req[t]]``, −1 for
    padding).  ``seq_lens[r]`` counts the request's tokens after this step,
    ``q_start[r] .. q_start[r+1]`` are its tokens in the flattened batch.
    """

    num_tokens: int
    num_reqs: int
    token_ids: torch.Tensor
    positions: torch.Tensor
    token_req: torch.Tensor
    q_start: torch.Tensor
    seq_lens: torch.Tensor
    slots: torch.Tensor
    groups: list[CacheGroupView]
    states: list[torch.Tensor]
    buffers: StepBuffers
    dtype: torch.dtype
    device: torch.device
    # host-side copies for parts that choose a kernel by the batch's shape
    host_query_lens: list[int] = field(default_factory=list)
    host_seq_lens: list[int] = field(default_factory=list)
    max_query_len: int = 0
    max_seq_len: int = 0
    scratch: dict = field(default_factory=dict)  # per-step values parts share (rotary tables)
    token_rows: torch.Tensor | None = None

    def buf(self, name: str, cols: int, dtype: torch.dtype | None = None, rows: int | None = None) -> torch.Tensor:
        return self.buffers.get(name, self.num_tokens if rows is None else rows, cols,
                                self.dtype if dtype is None else dtype,
                                reserve=self.buffers.token_capacity if rows is None else 0)
