"""Grouped-query attention over the paged cache.

Reference: kvcore/model/models/llama3.py:48-104 (stacked qkv projection with rows in
the order q, k, v; rotation of q and k; attention; output projection) and
kvcore/model/attn_backend/torch_paged.py:70-117 (keys and values are written to their
page slots first, then every query reads keys ``0..position`` back from the cache).
"""

from __future__ import annotations

import torch

from kvcore_amd.ops import library as ops

from .base import CacheNeed, Mixer, ParamSource, ParamSpec, PositionEncoding, register_mixer


DECODE_MAX_SPLITS = 32


def decode_target_blocks() -> int:
    """Blocks a launch of the decode kernel wants: one for each compute unit."""
    return ops.compute_units()


def prefill_target_blocks() -> int:
    """Blocks a launch of the kernel for portions wants: a compute unit holds two."""
    return 2 * ops.compute_units()


def prefill_split_rows(nkv: int, g: int) -> int:
    """An upper bound on tokens x splits when ``prefill_splits`` gives more than one split."""
    rows_tokens = max(128 // g, 1)
    return 4 * prefill_target_blocks() * rows_tokens // nkv + 2 * rows_tokens


def prefill_few_tiles() -> int:
    """Up to so many small tiles (half the compute units), splits go with small tiles."""
    return ops.compute_units() // 2


PREFILL_MIN_KEYS = 256      # for steps of few tokens, whose partial results are small
PREFILL_MIN_KEYS_MOST = 1024
PREFILL_MAX_SPLITS = 32


def prefill_splits(T: int, nkv: int, g: int, max_query_len: int, max_seq_len: int, window: int,
                   num_reqs: int = 1) -> int:
    """How many blocks share the keys of one tile of query rows in the kernel for portions
    of prompts.  A compute unit holds two of its blocks, so a launch wants some 512.  The
    kernel has tiles of 64 rows (one or two a block) and of 128 (two a block, cheaper per
    key); with splits it takes the small tiles one a block for very few rows and the large
    ones otherwise (`launch_prefill` in csrc/attention_prefill.hip, which must agree with
    this on where "very few" ends).  Measured on the 8B shape: splits pay when the rows are
    few and every block still has a few hundred keys to walk, a thousand for steps of a
    thousand tokens (a row sees ``max_seq_len`` keys at most and, under the causal mask,
    about half a portion fewer on average).  Every request but one may add a ragged tile."""
    small_tokens = max(64 // g, 1)
    small_tiles = (-(-T // small_tokens) + num_reqs - 1) * nkv  # blocks of one small tile each
    keys = max_seq_len - min(T, max_query_len) // 2
    if window > 0:
        keys = min(keys, window + 2 * small_tokens)
    target = prefill_target_blocks()
    if small_tiles <= prefill_few_tiles():
        return max(1, min(-(-target // small_tiles), keys // PREFILL_MIN_KEYS, PREFILL_MAX_SPLITS))
    if small_tiles <= target:
        if small_tiles == target:
            return 1  # one small tile a block fills the chip as it is
        min_keys = min(max(T, PREFILL_MIN_KEYS), PREFILL_MIN_KEYS_MOST)
    else:
        min_keys = min(max(T // 2, PREFILL_MIN_KEYS), PREFILL_MIN_KEYS_MOST)
    rows_tokens = max(128 // g, 1)
    blocks = ((-(-T // rows_tokens)) + num_reqs) // 2 * nkv
    if blocks >= target:
        return 1
    return max(1, min(-(-target // blocks), keys // min_keys, PREFILL_MAX_SPLITS))


def decode_splits(num_tokens: int, num_kv_heads: int, max_seq_len: int, waves: int,
                  window: int = 0) -> int:
    """Into how many parts each request's key range is cut for the decode kernel, beyond the
    ``waves`` waves of a block that share a part.  One compute unit draws keys and values
    from memory far slower than the chip can deliver them, so the parts are made many
    enough to occupy every unit, as long as each wave still has a block of 16 keys."""
    keys = max_seq_len if window <= 0 else min(max_seq_len, window + 16)
    blocks = -(-keys // 16)
    by_room = -(-decode_target_blocks() // max(num_tokens * num_kv_heads, 1))
    by_length = max(1, blocks // waves)
    return max(1, min(by_room, by_length, DECODE_MAX_SPLITS))


class PagedAttention(Mixer):
    """``scale`` is a parameter (the reference fixes ``head_dim ** -0.5`` at
    llama3.py:60); ``window`` 0 attends to every earlier token; ``page_size`` asks for cache
    pages of that many tokens for this layer's group (None: the engine's block size)."""

    @property
    def takes_scaled_rows(self) -> bool:  # x only goes into the qkv product
        return self.hidden_size % 8 == 0

    @property
    def takes_sink(self) -> bool:  # the output product's rows are whole heads
        return self.q_size % 8 == 0

    def __init__(self, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, bias: bool = False, window: int = 0, page_size: int | None = None,
                 position: PositionEncoding | None = None) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(f"head size {head_dim} is not supported (multiples of 16 up to 256)")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.scale = scale
        self.bias = bias
        self.window = window
        self.page_size = page_size  # None: the engine's block size
        self.position = position
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim

    def param_specs(self) -> list[ParamSpec]:
        total = self.q_size + 2 * self.kv_size

        def stacked(suffix: str) -> tuple[ParamSource, ...]:
            return (
                ParamSource(f"q_proj.{suffix}", 0, self.q_size),
                ParamSource(f"k_proj.{suffix}", self.q_size, self.kv_size),
                ParamSource(f"v_proj.{suffix}", self.q_size + self.kv_size, self.kv_size),
            )

        specs = [
            ParamSpec("qkv_proj.weight", (total, self.hidden_size), sources=stacked("weight")),
            ParamSpec("o_proj.weight", (self.hidden_size, self.q_size)),
        ]
        if self.bias:
            specs.append(ParamSpec("qkv_proj.bias", (total,), init="zeros", sources=stacked("bias")))
            specs.append(ParamSpec("o_proj.bias", (self.hidden_size,), init="zeros"))
        return specs

    def cache_need(self) -> CacheNeed:
        return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, self.window, self.page_size)

    def check_limits(self, limits) -> None:
        """The decode kernel keeps the page ids of a split's key range in LDS; a block table
        too wide for that is refused here, when the engine is built, not in a decode step.
        So is a cache in another dtype than the model's, which the attention kernels do not
        read (a subclass that names one in its ``cache_need`` must bring kernels that do)."""
        need = self.cache_need()
        if need.dtype is not None and need.dtype != self.runtime.dtype:
            raise ValueError(
                f"{type(self).__name__} keeps its cache in {need.dtype} beside a model in "
                f"{self.runtime.dtype}: the attention kernels read keys and values in the model's dtype")
        if self.runtime.dtype != torch.bfloat16 or not ops.decode_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, limits.page_size, self.runtime.dtype):
            return
        widest = ops.decode_attention_max_table(self.num_heads, self.num_kv_heads, self.head_dim)
        if limits.max_pages_per_seq > widest:
            raise ValueError(
                f"max_model_len={limits.max_model_len} with cache pages of {limits.page_size} tokens gives a "
                f"block table of {limits.max_pages_per_seq} entries per request; the decode attention kernel "
                f"serves at most {widest} for {self.num_heads} heads of {self.head_dim} over "
                f"{self.num_kv_heads} kv heads: use a larger block_size or a smaller max_model_len")

    def product_weights(self) -> tuple[str, ...]:
        return ("qkv_proj.weight", "o_proj.weight")

    def forward(self, x, ctx, call, sink=None):
        p = self.params
        qkv = ctx.buf("attn_qkv", self.q_size + 2 * self.kv_size)
        ops.linear(qkv, x, p["qkv_proj.weight"], p.get("qkv_proj.bias"))

        group = ctx.groups[call.group_index]
        # K pages [kv_heads, page, d]; V pages [kv_heads, d, page]: the keys of a page lie
        # side by side, which is how the matrix cores want the values
        k_cache = group.plane(call.cache_index, 0, self.num_kv_heads, group.page_size, self.head_dim)
        v_cache = group.plane(call.cache_index, 1, self.num_kv_heads, self.head_dim, group.page_size)
        rot = self.position.rotary(ctx) if self.position is not None else None
        if rot is None:
            cos = sin = ctx.buffers.get("rope_none", ctx.num_tokens, 0, torch.float32)
            rot_dim, interleaved = 0, False
        else:
            cos, sin, rot_dim, interleaved = rot.cos, rot.sin, rot.rot_dim, rot.interleaved
        attn = ctx.buf("attn_out", self.q_size)
        common = dict(table=group.table, positions=ctx.positions, token_req=ctx.token_req,
                      slots=ctx.slots, nh=self.num_heads, nkv=self.num_kv_heads, d=self.head_dim,
                      scale=self.scale, window=self.window)
        if ctx.max_query_len == 1 and ops.decode_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, group.page_size, x.dtype):
            # single tokens: rotation, cache write and attention in one kernel on the matrix
            # cores, a block per (token, kv head, split)
            T = ctx.num_tokens
            waves = ops.decode_attention_waves(self.num_heads, self.num_kv_heads, self.head_dim)
            nsplit = decode_splits(T, self.num_kv_heads, ctx.max_seq_len, waves, self.window)
            part_o = part_ml = None
            if nsplit > 1:
                # tokens x splits is at most the blocks wanted per kv head plus the tokens: room
                # for the largest at once, since a buffer that grows drops the graphs
                most = (decode_target_blocks() // self.num_kv_heads + 1 + max(T, ctx.buffers.seq_capacity)) \
                    * self.num_heads
                part_o = ctx.buffers.get("attn_part_o", T * self.num_heads * nsplit, self.head_dim,
                                         torch.float32, reserve=most)
                part_ml = ctx.buffers.get("attn_part_ml", T * self.num_heads * nsplit, 2, torch.float32,
                                          reserve=most)
            ops.decode_attention(attn, qkv, k_cache, v_cache, nsplit=nsplit, part_o=part_o,
                                 part_ml=part_ml, cos=cos, sin=sin, rot_dim=rot_dim,
                                 interleaved=interleaved, write_kv=call.write_cache,
                                 token_rows=ctx.token_rows, **common)
        else:
            # where each token's key and value go: once per step and cache group
            slot_key = ("kv_slot", call.group_index)
            kv_slot = ctx.scratch.get(slot_key)
            if kv_slot is None:
                kv_slot = ctx.buf(f"kv_slot_{call.group_index}", 1, torch.int32).view(-1)
                ops.kv_slots(kv_slot, positions=ctx.positions, token_req=ctx.token_req,
                             slots=ctx.slots, table=group.table, page_size=group.page_size,
                             num_pages=k_cache.shape[0])
                ctx.scratch[slot_key] = kv_slot
            on_matrix_cores = ctx.max_query_len > 1 and self.scale > 0 and ops.prefill_attention_supported(
                self.num_heads, self.num_kv_heads, self.head_dim, group.page_size, x.dtype)
            # the kernel for portions rotates the queries on their way in where it can, which
            # saves writing them and reading them again
            rotates = on_matrix_cores and ops.prefill_attention_rotates(rot_dim, interleaved)
            ops.rope_kv_write(qkv, k_cache, v_cache, cos, sin, rot_dim=rot_dim,
                              interleaved=interleaved, kv_slot=kv_slot, nh=self.num_heads,
                              nkv=self.num_kv_heads, d=self.head_dim, write_kv=call.write_cache,
                              rotate_q=not rotates)
            if on_matrix_cores:
                # portions of prompts (single tokens may ride along): tiles of query rows per
                # block, and several blocks per tile where few rows meet many keys
                T = ctx.num_tokens
                nsplit = prefill_splits(T, self.num_kv_heads, self.num_heads // self.num_kv_heads,
                                        ctx.max_query_len, ctx.max_seq_len, self.window, ctx.num_reqs)
                part_o = part_ml = None
                if nsplit > 1:
                    # asked for at their largest at once: a buffer that grows drops the graphs
                    most = prefill_split_rows(self.num_kv_heads, self.num_heads // self.num_kv_heads) * self.num_heads
                    part_o = ctx.buffers.get("attn_prefill_part_o", T * self.num_heads * nsplit,
                                             self.head_dim, torch.float32, reserve=most)
                    part_ml = ctx.buffers.get("attn_prefill_part_ml", T * self.num_heads * nsplit, 2,
                                              torch.float32, reserve=most)
                ops.prefill_attention(attn, qkv, k_cache, v_cache, table=group.table,
                                      positions=ctx.positions, q_start=ctx.q_start, slots=ctx.slots,
                                      num_reqs=ctx.num_reqs, nh=self.num_heads, nkv=self.num_kv_heads,
                                      d=self.head_dim, scale=self.scale, window=self.window,
                                      nsplit=nsplit, part_o=part_o, part_ml=part_ml,
                                      **(dict(cos=cos, sin=sin, rot_dim=rot_dim, interleaved=interleaved)
                                         if rotates else {}))
            else:
                ops.paged_attention(attn, qkv, k_cache, v_cache, **common)
        if sink is not None:
            return ops.linear(sink, attn, p["o_proj.weight"], p.get("o_proj.bias"))
        out = ctx.buf("mixer_out", self.hidden_size)
        ops.linear(out, attn, p["o_proj.weight"], p.get("o_proj.bias"))
        return out


register_mixer("paged_attention", PagedAttention)
