"""Causal grouped-query attention over the paged key/value cache.

x -> fused q/k/v projection -> (optional) per-head RMSNorm of q and k -> rotary
encoding -> keys and values stored in the cache -> attention over the cache ->
output projection.  The order follows the reference's decoder,
runtime/include/execution/decoder.hpp:121-158.  Three separate checkpoint matrices
become one [Q + 2 KV, H] matrix when the part is built: each output element is
still the same dot product.  Each projection may have a bias
(runtime/include/models/qwen3_model.hpp:386-395: taken if the checkpoint holds it).

Options of the spec beyond that decoder (the matrix-core kernels have an extended form for
chunks, slopes and the sink; values of another width than the keys go down the generic
float32-arithmetic kernels): values narrower or wider than keys (`value_dim`), one RMS norm
over the whole q and the whole k projection instead of one per head (`qk_norm_scope =
"projection"`), visibility in blocks of `chunk` positions counted from the sequence's start,
a distance term slope_h (i - j) taken off the score with slope_h = 2^(-r (h + 1) / heads)
(`distance_slope_range` = r), a learned `sink` per head in the softmax's denominator or a
plain 1 there (`unit_sink`), and `talking_heads`: a learned matrix T [heads, heads] mixes the
scaled scores of every (query, key) pair over the heads before the softmax.  A mix of scores is
the score of mixed queries: with the heads g of kv head c sharing the key k_c,
sum_g T[h, g] (q_g . k_c(g)) = sum_c (sum_{g in c} T[h, g] q_g) . k_c, so the queries are mixed
once a row (`lib.mix_heads`: a row of n_kv_heads * head_dim a head) and the generic kernel
meets them with the keys of all kv heads laid end to end (`key_heads`).

A rotation whose angles the store kernel works out itself (position kind "rope_half":
frequencies that may be rescaled, any rotated width, values of their own width),
`value_mix` (what a layer caches is (1 - lambda) v + lambda v_source, v_source the values that
the step's source layer computed for the same token, kept in float32 for the step) and
`output_gate` (the concatenated heads times sigmoid(W_g x), the gate's rows fused into the
q/k/v product) go through `lib.head_store`, the store kernel for rows that go on after v.
So do a rotation of neighbouring pairs (position kind "rope_pairs": a query and a key give
the same score when both are permuted alike, so the rows of the q and k projections are
reordered when the part is built, evens then odds within a head's rotated part, and the
rotation of halves does the rest), `query_temperature` (queries grow with the position),
`output_gate = "head"` (one gate a head, applied by the attention kernel), `shared_kv` (a part
without key and value projections, whose runs read what another run cached) and `pool`
(besides its window a query sees one key and value, the means, for every block of `pool`
positions that lies wholly before the window: the part keeps them in a second paged cache of
its own, one entry a block, which `lib.pool_store` fills from the cached tokens as blocks
become complete, and the generic kernel walks after the window).
"""
from __future__ import annotations

import dataclasses
import functools
import os

import numpy as np
import torch

from ..csrc import lib
from ..csrc.lib import PAGE_TOKENS
from ..weights.loader import ParamSpec
from .base import KVRequest
from .linear import Linear

# EDGE_INFER_FUSED_DECODE=0: decode steps launch the norm-rotate-store kernel of their own
# instead of letting the matrix-core decode kernel do that work
FUSED_DECODE = os.environ.get("EDGE_INFER_FUSED_DECODE", "1") != "0"
# EDGE_INFER_MATRIX_CORE_ATTENTION=0: bfloat16 attention runs on the generic kernel (float32
# arithmetic on the cached bfloat16 keys and values) whatever the head size
MATRIX_CORE_ATTENTION = os.environ.get("EDGE_INFER_MATRIX_CORE_ATTENTION", "1") != "0"


# What the matrix-core decode kernel costs, measured on an MI355X: a wave walks a tile of 16
# keys of head size 128 in 1.9 us (other head sizes in proportion: a tile's bytes are what it
# waits for); merging slices costs 4.5 us and 0.1 us a slice.
TILE_US_128, MERGE_US, MERGE_SLICE_US = 1.9, 4.5, 0.1
WAVES_A_UNIT = 16       # waves of this kernel that a compute unit holds at once
MAX_SLICES = 32
MAX_LAUNCH_PLANS = 512  # decode launch shapes a part remembers
VALUE_SOURCE = "attn.v_source"   # ctx.notes / buffer: the source layer's values of this step


@functools.lru_cache(maxsize=512)
def _decode_items(n_seqs: int, live: int):
    """One work item a sequence, [3, n_seqs]: sequence (-1: padding), its row, one position."""
    seq = np.full(n_seqs, -1, dtype=np.int32)
    seq[:live] = np.arange(live)
    npos = np.zeros(n_seqs, dtype=np.int32)
    npos[:live] = 1
    items = np.stack([seq, np.arange(n_seqs, dtype=np.int32), npos])
    items.setflags(write=False)
    return items


class Attention:
    @property
    def capture_safe(self):
        """Launches only this library's kernels and allocates nothing per step, as long as
        its products do."""
        return self.qkv.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.qkv.capture_rows, self.o.capture_rows)

    @classmethod
    def parameters(cls, spec, hidden):
        # (in this order: a model of random weights draws them in the order of this table)
        params = {"q_proj.weight": ParamSpec((spec.q_width, hidden))}
        if not spec.shared_kv:
            params["k_proj.weight"] = ParamSpec((spec.kv_width, hidden))
            params["v_proj.weight"] = ParamSpec((spec.v_width, hidden))
        params["o_proj.weight"] = ParamSpec((hidden, spec.out_width))
        if spec.o_bias is not False:
            params["o_proj.bias"] = ParamSpec((hidden,), optional=spec.o_bias is not True)
        if spec.talking_heads:
            params["talk"] = ParamSpec((spec.n_heads, spec.n_heads), init="near_identity",
                                       scale=0.2)
        if spec.qkv_bias is not False and not spec.shared_kv:
            required = spec.qkv_bias is True
            params["q_proj.bias"] = ParamSpec((spec.q_width,), optional=not required)
            params["k_proj.bias"] = ParamSpec((spec.kv_width,), optional=not required)
            params["v_proj.bias"] = ParamSpec((spec.v_width,), optional=not required)
        if spec.qk_norm:
            whole = spec.qk_norm_scope == "projection"
            params["q_norm.weight"] = ParamSpec((spec.q_width if whole else spec.head_dim,),
                                                init="norm")
            params["k_norm.weight"] = ParamSpec((spec.kv_width if whole else spec.head_dim,),
                                                init="norm")
        if spec.sink:
            params["sink"] = ParamSpec((spec.n_heads,), init="uniform", low=-1.0, high=1.0)
        if spec.value_mix is not None:
            # one number; the source layer and a layer that mixes nothing may hold it unused
            params["value_mix"] = ParamSpec((), init="uniform", low=0.1, high=0.6,
                                            optional=spec.value_mix != "mix")
        if spec.output_gate:
            rows = spec.n_heads if spec.output_gate == "head" else spec.out_width
            params["gate_proj.weight"] = ParamSpec((rows, hidden))
        return params

    @classmethod
    def cache_request(cls, spec):
        # positions the cache keeps behind the newest one: the window's, and the block's that
        # the newest position may complete; more where other runs read with a wider mask
        keep = spec.window
        if keep is not None and spec.pool is not None:
            keep = max(keep, spec.pool)
        if spec.cache_span is not None:
            keep = None if spec.cache_span == 0 or keep is None else max(keep, spec.cache_span)
        return KVRequest(n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim, window=keep,
                         value_dim=None if spec.v_dim == spec.head_dim else spec.v_dim,
                         chunk=spec.chunk)

    POOL = "pool"      # the name of the pooled cache under the run's own cache id

    @classmethod
    def own_cache_request(cls, spec):
        """What a run keeps for itself even when it reads another run's keys and values: the
        pooled blocks, which depend on its own block size."""
        if spec.pool is None:
            return None
        return {cls.POOL: KVRequest(n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim,
                                    value_dim=None if spec.v_dim == spec.head_dim else spec.v_dim,
                                    stride=spec.pool)}

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        """What this part will run, so that a model can have it compiled ahead of its first
        step."""
        group = spec.n_heads // max(1, spec.n_kv_heads)
        fast = (dtype == torch.bfloat16 and spec.v_dim == spec.head_dim and MATRIX_CORE_ATTENTION
                and not spec.talking_heads
                and lib.attention_decode_mfma_supported(spec.head_dim, group))
        kernels = "attention_mfma" if fast else "attention_generic"
        if cls.wide_keys(spec, dtype):
            kernels = "attention_wide"
        # (the pooled blocks are stored, and beside the matrix-core kernels also gathered, by
        # kernels of the generic library)
        return ("rope_store", kernels, *(("attention_generic",) if spec.pool is not None else ()),
                *(("head_ops",) if spec.talking_heads else ()), *Linear.kernel_libraries(dtype))

    @classmethod
    def wide_keys(cls, spec, dtype) -> bool:
        """Whether this part runs the matrix-core kernel for wide keys: scores mixed over heads
        (queries as wide as the keys of all kv heads together), bfloat16, sizes it takes."""
        return (spec.talking_heads and MATRIX_CORE_ATTENTION and spec.chunk is None
                and lib.attention_wide_supported(dtype, spec.n_kv_heads * spec.head_dim,
                                                 spec.head_dim, spec.v_dim))

    @classmethod
    def general_store(cls, spec) -> bool:
        """Whether the part norms, rotates and stores through `lib.head_store`."""
        return (spec.position.kind in ("rope_half", "rope_pairs")
                or spec.value_mix in ("source", "mix") or bool(spec.output_gate)
                or spec.query_temperature is not None or spec.shared_kv or spec.pool is not None)

    @classmethod
    def check(cls, spec):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("attention: n_heads must be a multiple of n_kv_heads")
        if spec.qk_norm_scope not in ("head", "projection"):
            raise ValueError(f"attention: unknown qk_norm_scope '{spec.qk_norm_scope}'")
        whole = spec.qk_norm_scope == "projection" or not spec.qk_norm
        if spec.value_mix not in (None, "off", "source", "mix"):
            raise ValueError(f"attention: unknown value_mix '{spec.value_mix}'")
        if cls.general_store(spec):
            if spec.position.kind not in ("rope_half", "rope_pairs", "none"):
                raise ValueError("attention: value mixing and the output gate are implemented "
                                 "with position kinds 'rope_half', 'rope_pairs' and 'none'")
            if spec.qk_norm and spec.qk_norm_scope != "head":
                raise ValueError("attention: this store norms per head only")
            if spec.talking_heads or spec.qkv_bias:
                raise ValueError("attention: this store takes no biases and no mixed scores")
            if not (1 <= spec.head_dim <= 256 and 1 <= spec.v_dim <= 256):
                raise ValueError("attention: key and value head sizes must lie in 1..256, got "
                                 f"{spec.head_dim} and {spec.v_dim}")
        elif whole and spec.position.kind == "none":
            # the store kernel without a rotation takes any sizes the attention kernel takes
            if not (1 <= spec.head_dim <= 256 and 1 <= spec.v_dim <= 256):
                raise ValueError("attention: key and value head sizes must lie in 1..256, got "
                                 f"{spec.head_dim} and {spec.v_dim}")
        else:
            if spec.qk_norm_scope == "projection" and spec.qk_norm:
                raise ValueError("attention: a norm over the whole projection is implemented "
                                 "only without a rotation")
            if spec.v_dim != spec.head_dim:
                raise ValueError("attention: values of another width than the keys are "
                                 "implemented only without a rotation and per-head norms")
            if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
                raise ValueError("attention: head_dim must be a multiple of 16 between 16 and "
                                 f"256, got {spec.head_dim}")
        if spec.sink and spec.unit_sink:
            raise ValueError("attention: a learned sink and a sink of 1 exclude each other")
        if spec.talking_heads and spec.n_kv_heads * spec.head_dim > 1024:
            raise ValueError("attention: with talking heads the keys of all kv heads of a "
                             "position may hold 1024 elements at most, got "
                             f"{spec.n_kv_heads * spec.head_dim}")
        if spec.talking_heads and spec.distance_slope_range is not None:
            raise ValueError("attention: talking heads with a distance term are not implemented")
        if spec.window is not None and spec.window < 1:
            raise ValueError("attention: a window must be at least 1")
        if spec.output_gate not in (False, True, "head"):
            raise ValueError(f"attention: unknown output_gate {spec.output_gate!r}")
        if spec.pool is not None:
            if spec.pool < 1 or spec.window is None:
                raise ValueError("attention: pooled blocks hold at least one position and need "
                                 "a window")
            if spec.chunk is not None or spec.talking_heads or spec.distance_slope_range is not None:
                raise ValueError("attention: pooled blocks with chunks, mixed scores or a "
                                 "distance term are not implemented")
        if spec.query_temperature is not None and spec.query_temperature[1] < 1:
            raise ValueError("attention: the query temperature's step must be at least 1")
        if spec.shared_kv and spec.value_mix in ("source", "mix"):
            raise ValueError("attention: a part without values of its own mixes none")
        if spec.chunk is not None and spec.chunk < 1:
            raise ValueError("attention: a chunk must hold at least one position")

    def __init__(self, spec, hidden, params, dtype, device, positions):
        self.check(spec)
        self.spec = spec
        self.hidden = hidden
        self.dtype = dtype
        q_weight = params["q_proj.weight"]
        k_weight = None if spec.shared_kv else params["k_proj.weight"]
        position_spec = spec.position
        if spec.position.kind == "rope_pairs":
            # neighbouring pairs (2i, 2i + 1) become the pairs (i, i + R/2) of permuted rows
            order = self._pairs_to_halves(spec.head_dim, spec.position.dim)
            q_weight = self._permute_heads(q_weight, spec.n_heads, order)
            if k_weight is not None:
                k_weight = self._permute_heads(k_weight, spec.n_kv_heads, order)
            position_spec = dataclasses.replace(spec.position, kind="rope_half", scaling=None)
        fused = torch.cat([q_weight]
                          + ([] if spec.shared_kv else [k_weight, params["v_proj.weight"]])
                          + ([params["gate_proj.weight"]] if spec.output_gate else []), dim=0)
        names = ("q_proj",) if spec.shared_kv else ("q_proj", "k_proj", "v_proj")
        fused_bias = None
        if any(f"{name}.bias" in params for name in names):   # absent ones count as zero
            fused_bias = torch.cat([
                params[f"{name}.bias"] if f"{name}.bias" in params
                else params[f"{name}.weight"].new_zeros(params[f"{name}.weight"].shape[0])
                for name in names])
        self.qkv = Linear(fused, dtype, device, bias=fused_bias)
        self.o = Linear(params["o_proj.weight"], dtype, device, bias=params.get("o_proj.bias"))
        self.q_norm = self.k_norm = None
        if spec.qk_norm:
            self.q_norm = params["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.k_norm = params["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        self.position = positions(position_spec)   # shared table object
        self.group = spec.n_heads // spec.n_kv_heads
        self.scale = spec.scale if spec.scale is not None else spec.head_dim ** -0.5
        # without a rotation and without per-head norms, one kernel norms (or not) and stores
        self.general = self.general_store(spec)
        self.whole_store = (not self.general and spec.position.kind == "none"
                            and (spec.qk_norm_scope == "projection" or not spec.qk_norm))
        self.value_lambda = None
        if spec.value_mix == "mix":
            self.value_lambda = params["value_mix"].to(device=device, dtype=torch.float32).reshape(1).contiguous()
        # kv heads whose keys and values the rows of this part's projection hold
        self.own_kv_heads = 0 if spec.shared_kv else spec.n_kv_heads
        # where the gate's columns begin
        self.gate_column = spec.q_width + (0 if spec.shared_kv else spec.kv_width + spec.v_width)
        self.head_gate = spec.output_gate == "head"
        self.slopes = self.sinks = None
        if spec.distance_slope_range is not None:
            exponent = -float(spec.distance_slope_range) * torch.arange(
                1, spec.n_heads + 1, dtype=torch.float64) / spec.n_heads
            self.slopes = torch.pow(2.0, exponent).to(device=device, dtype=torch.float32).contiguous()
        if spec.sink:
            self.sinks = params["sink"].to(device=device, dtype=torch.float32).contiguous()
        elif spec.unit_sink:      # a sink of score 0: e^0 = 1 joins the denominator
            self.sinks = torch.zeros(spec.n_heads, dtype=torch.float32, device=device)
        self.talk = None
        if spec.talking_heads:
            self.talk = params["talk"].to(device=device, dtype=torch.float32).contiguous()
        # the matrix-core kernels take bfloat16 with head sizes 64 and 128 and values as wide
        # as the keys; every other case runs the generic kernel
        self.matrix_cores = (dtype == torch.bfloat16 and spec.v_dim == spec.head_dim and
                            MATRIX_CORE_ATTENTION and self.talk is None and
                            lib.attention_decode_mfma_supported(spec.head_dim, self.group))
        # beside the matrix-core kernels the pooled blocks are gathered by the generic kernel
        # (they are few: one for `pool` tokens) and taken in as one more slice of the softmax
        self.pooled_aside = self.matrix_cores and spec.pool is not None
        # chunk, slopes, sink: what the kernels take beyond a window
        self.wide = self.wide_keys(spec, dtype)
        self.extras = dict(chunk=spec.chunk, slopes=self.slopes, sinks=self.sinks)
        self.has_extras = spec.chunk is not None or self.slopes is not None or self.sinks is not None
        self.compute_units = lib.compute_units(device)     # the chip's size, for launch plans
        self._decode_launches = {}     # (sequences, pages of context) -> decode_launch's answer

    @staticmethod
    def _pairs_to_halves(head_dim: int, rotated: int):
        """Order of a head's rows after which the rotation of the pairs (i, i + R/2) turns what
        the rotation of the neighbours (2i, 2i + 1) turned: the even rows of the rotated part,
        then its odd rows, then the rest."""
        return list(range(0, rotated, 2)) + list(range(1, rotated, 2)) + list(range(rotated, head_dim))

    @staticmethod
    def _permute_heads(weight, heads: int, order):
        head_dim = len(order)
        index = torch.tensor([head * head_dim + row for head in range(heads) for row in order],
                             dtype=torch.long, device=weight.device)
        return weight.index_select(0, index)

    # the number of positions of one sequence that a prefill work item covers
    def positions_per_item(self, key_ways: int = 1):
        if self.wide:
            return lib.attention_wide_positions(self.group) if key_ways == 1 else 0
        if self.matrix_cores:          # the matrix-core prefill kernel takes the same cases
            return lib.attention_prefill_mfma_positions(self.group, key_ways)
        return lib.attention_positions_per_item(self.group) if key_ways == 1 else 0

    def prefill_key_ways(self, counts) -> int:
        """1 or 2: how many waves share the keys of a page for the same rows in the prompt
        step whose sequences bring `counts` tokens.  A step that gives every compute unit
        about one block (one prompt of 2,048 tokens of the 8B shape: 256, whose walks are 1 to
        32 pages long) takes items half as long, and with them twice the blocks, which the
        kernel then pairs, a long one with a short one; with more blocks than that the
        hardware balances them, and a wave that takes every key of a page for its rows does
        less beside its products (measured, one prompt of the 8B shape: 2,048 tokens 60
        against 71 us, 3,072 tokens 147 against 105)."""
        if not self.matrix_cores or self.positions_per_item(2) == 0:
            return 1
        size = self.positions_per_item(1)
        heads = lib.attention_prefill_mfma_heads(self.group)
        items = sum((count + size - 1) // size for count in counts)
        blocks = items * (self.group // heads) * self.spec.n_kv_heads
        return 2 if 4 * blocks <= 5 * self.compute_units else 1

    @property
    def plan_key(self):
        """Attention parts with equal keys plan the same sections."""
        return ("attention", self.positions_per_item(), self.group, self.spec.n_kv_heads, self.wide,
                self.pooled_aside, self.spec.pool)

    def _items_section(self, key_ways: int = 1):
        return f"attention.items{self.positions_per_item(key_ways)}"

    def _aside_size(self) -> int:
        """Positions of an item of the generic kernel, which gathers the pooled blocks beside
        the matrix-core kernels."""
        return lib.attention_positions_per_item(self.group)

    @staticmethod
    def _prompt_items(plan, size: int):
        """Every sequence's rows cut into items of `size`, the ones with the longest key range
        first, as [3, items]: sequence, first row, positions."""
        items = []
        for index, seq in enumerate(plan.seqs):
            for p0 in range(0, seq.count, size):
                npos = min(size, seq.count - p0)
                items.append((-(seq.start + p0 + npos), index, seq.row0 + p0, npos))
        items.sort()
        return np.asarray([item[1:] for item in items], dtype=np.int32).T.copy()

    def plan_step(self, plan):
        """The work items of this step's attention kernels, as one int32 section [3, items]:
        sequence (-1: padding), first row, positions.  A prompt step cuts every sequence's
        rows into items of `positions_per_item`, the ones with the longest key range first
        (they take longest, so they start first); a decode step has one item a sequence."""
        if plan.decode:
            return {"attention.decode_items": _decode_items(plan.n_seqs, plan.n_live_seqs)}
        key_ways = self.prefill_key_ways([seq.count for seq in plan.seqs])
        sections = {self._items_section(key_ways):
                    self._prompt_items(plan, self.positions_per_item(key_ways))}
        if self.pooled_aside:
            name = f"attention.items{self._aside_size()}"
            if name not in sections:
                sections[name] = self._prompt_items(plan, self._aside_size())
        if self.spec.pool is not None:
            # the rows of this step that end a block of `pool` positions (-1: there is none)
            pool = self.spec.pool
            rows = [seq.row0 + k for seq in plan.seqs
                    for k in range((-(seq.start + 1)) % pool, seq.count, pool)]
            sections[f"attention.pool_rows{pool}"] = np.asarray(rows or [-1], dtype=np.int32)
        return sections

    @staticmethod
    def _items(ctx, name):
        section = ctx.meta.section(name)
        count = section.numel() // 3
        return section[:count], section[count:2 * count], section[2 * count:], count

    def decode_launch(self, n_seqs: int, context: int):
        """(slices of the key range, waves a block, query heads of a group a block takes) of
        a decode step over `n_seqs` sequences of up to `context` tokens.  A slice is the same
        number of pages for every sequence.  A layer with a window reads at most the window's
        keys (and the rest of the page they begin in), so its slices are sized for those.

        Matrix-core kernel, up to as many (sequence, kv head) pairs as the chip has compute
        units: blocks of 16 waves, a tile of 16 keys per wave at a time, and as many slices as
        shorten a wave's walk by more than the merge kernel costs, while all blocks still fit
        the chip at once; if they then leave compute units empty, a block takes fewer heads (2
        or 1 instead of 4), as long as every block still has a unit of its own: the keys are
        fetched once more per block, from the L2, and each block has less to do per tile.  Up
        to twice as many pairs: blocks of 8 waves, no slices.  More pairs, and the generic
        kernel: blocks of 4 waves and enough slices to put about two blocks on each compute
        unit, never more than there are pages."""
        if self.spec.window is not None:
            context = min(context, self.spec.window + PAGE_TOKENS - 1)
        if self.spec.chunk is not None:
            context = min(context, self.spec.chunk + PAGE_TOKENS - 1)
        pages = max(1, (context + PAGE_TOKENS - 1) // PAGE_TOKENS)
        n_kv_heads = self.spec.n_kv_heads
        units = self.compute_units
        if self.matrix_cores:
            # a block of 16 waves takes at most 4 query heads of a group: larger groups have
            # several blocks per pair
            pairs = n_seqs * n_kv_heads * ((self.group + 3) // 4)
            if pairs <= units:
                tile_us = TILE_US_128 * self.spec.head_dim / 128
                tiles = (context + 15) // 16
                best, best_cost = 1, tile_us * ((tiles + 15) // 16)
                slices = 2
                while (slices <= min(pages, MAX_SLICES)
                       and pairs * 16 * slices <= units * WAVES_A_UNIT):
                    cost = (tile_us * ((tiles + 16 * slices - 1) // (16 * slices)) + MERGE_US
                            + MERGE_SLICE_US * slices)
                    if cost < best_cost:
                        best, best_cost = slices, cost
                    slices *= 2
                heads = min(4, 1 << (self.group.bit_length() - 1))
                while heads > 1:
                    blocks = n_seqs * n_kv_heads * best * -(-self.group // (heads // 2))
                    if blocks > units:
                        break
                    heads //= 2
                return best, 16, heads
            # up to twice as many pairs of at most 8 heads: blocks of 8 waves fill the chip's
            # wave slots once without slices (measured 1 to 3 % ahead of 4 waves at 32 to 64
            # sequences)
            pairs = n_seqs * n_kv_heads * ((self.group + 7) // 8)
            if pairs <= 2 * units:
                return 1, 8, 0
        blocks = n_seqs * n_kv_heads
        wanted = (2 * units + blocks - 1) // blocks
        return max(1, min(wanted, pages, MAX_SLICES)), 4, 0

    def _decode_launch_for(self, n_seqs: int, context: int):
        """`decode_launch`, remembered per (sequences, pages of context): a step that is not
        replayed from a graph asks in every layer and for every length, and the answer changes
        with the pages at most."""
        pages = (context + PAGE_TOKENS - 1) // PAGE_TOKENS
        launch = self._decode_launches.get((n_seqs, pages))
        if launch is None:
            if len(self._decode_launches) >= MAX_LAUNCH_PLANS:
                self._decode_launches.clear()
            launch = self._decode_launches[(n_seqs, pages)] = \
                self.decode_launch(n_seqs, pages * PAGE_TOKENS)
        return launch

    bias_later = True      # forward(..., bias_later=True) hands the last product's bias on

    def forward(self, ctx, x, entry, bias_later=False):
        """The mixer's rows; with `bias_later`, (rows, float32 bias of the output projection
        that is still to be added, or None), for a caller whose next kernel adds it."""
        spec = self.spec
        n = x.shape[0]
        meta = ctx.meta
        group_index, k_pages, v_pages = ctx.cache.kv(entry.cache)
        page_table = meta.page_table(group_index)
        # (the kernel that norms and stores the whole projection adds its bias as well)
        qkv, bias = (self.qkv.forward(ctx, x, "attn.qkv", bias_later=True) if self.whole_store
                     else (self.qkv.forward(ctx, x, "attn.qkv"), None))
        gate, pooled, aside = None, {}, {}
        if self.general:
            q = ctx.buffer("attn.q", (n, spec.q_width))
            v_first, v_mode = None, 0
            if spec.value_mix == "source":
                # this layer's values, kept in float32 for the layers of the step that mix them in
                v_first = ctx.buffer(VALUE_SOURCE, (n, spec.v_width), torch.float32)
                ctx.notes[VALUE_SOURCE] = v_first
                v_mode = 1
            elif spec.value_mix == "mix":
                v_first = ctx.notes.get(VALUE_SOURCE)
                if v_first is None or tuple(v_first.shape) != (n, spec.v_width):
                    raise ValueError("attention: a layer mixes values in, but no earlier layer of "
                                     "the step has kept values of that width")
                v_mode = 2
            if self.head_gate:
                gate = ctx.buffer("attn.gate", (n, spec.n_heads), torch.float32)
            if entry.writes_cache and spec.shared_kv:
                raise ValueError("attention: a part without key and value projections cannot "
                                 "write a cache entry")
            lib.head_store(qkv, self.q_norm, self.k_norm, spec.qk_norm_eps,
                           getattr(self.position, "frequencies", None), meta.row_pos,
                           meta.row_seq, page_table, q, k_pages, v_pages, spec.n_heads,
                           self.own_kv_heads, spec.head_dim, spec.v_dim,
                           write_cache=entry.writes_cache, v_first=v_first, v_mode=v_mode,
                           v_lambda=self.value_lambda, query_temperature=spec.query_temperature,
                           gate_out=gate, gate_column=self.gate_column)
            if spec.pool is not None:
                # the blocks that this step's rows complete, from the keys as the cache holds them
                pool_group, pool_k, pool_v = ctx.cache.kv((entry.own_id, self.POOL))
                pool_table = meta.page_table(pool_group)
                lib.pool_store(k_pages, v_pages, meta.row_pos, meta.row_seq, page_table,
                               pool_table, pool_k, pool_v, n, spec.pool,
                               row_list=None if ctx.decode else
                               meta.section(f"attention.pool_rows{spec.pool}"))
                pooled = dict(pool=spec.pool, pool_k=pool_k, pool_v=pool_v, pool_table=pool_table)
                if self.pooled_aside:
                    # every row's sums over the pooled blocks it sees, for the matrix-core
                    # kernels to take in as one more slice
                    pool_o = ctx.buffer("attn.pool_o", (n * spec.n_heads * spec.v_dim,), torch.float32)
                    pool_ml = ctx.buffer("attn.pool_ml", (n * spec.n_heads * 2,), torch.float32)
                    items = self._items(ctx, "attention.decode_items" if ctx.decode
                                        else f"attention.items{self._aside_size()}")
                    # (in this mode the kernel writes the sums only; `q` stands where the
                    # output's shape is asked for)
                    lib.attention(q, k_pages, v_pages, items[0], items[1], items[2], items[3],
                                  meta.row_pos, meta.row_seq, page_table, q, spec.n_heads,
                                  spec.n_kv_heads, spec.head_dim, window=spec.window,
                                  scale=self.scale, part_o=pool_o, part_ml=pool_ml,
                                  value_dim=spec.v_dim, pool_only=True, **pooled)
                    aside = dict(pool_o=pool_o, pool_ml=pool_ml)
        elif (ctx.decode and self.matrix_cores and FUSED_DECODE and qkv.dim() == 3
                and qkv.dtype == torch.float32 and not self.whole_store and not self.has_extras):
            # the decode kernel norms, rotates and stores for its rows itself: one launch less
            q = lib.DecodeProjection(qkv, self.q_norm, self.k_norm, spec.qk_norm_eps,
                                     self.position.table, entry.writes_cache)
        elif self.whole_store:
            q = ctx.buffer("attn.q", (n, spec.q_width))
            lib.projection_norm_store(
                qkv, self.q_norm, self.k_norm, spec.qk_norm_eps, meta.row_pos, meta.row_seq,
                page_table, q, k_pages, v_pages, spec.n_heads, spec.n_kv_heads, spec.head_dim,
                spec.v_dim, write_cache=entry.writes_cache, bias=bias)
        else:
            q = ctx.buffer("attn.q", (n, spec.q_width))
            lib.qk_norm_rope_store(
                qkv, self.q_norm, self.k_norm, spec.qk_norm_eps, self.position.table,
                meta.row_pos, meta.row_seq, page_table, q, k_pages, v_pages, spec.n_heads,
                spec.n_kv_heads, spec.head_dim, write_cache=entry.writes_cache)
        if self.talk is not None:
            # the queries mixed over heads, one part for every kv head's keys
            mixed = ctx.buffer("attn.q_mixed", (n, spec.q_width * spec.n_kv_heads))
            lib.mix_heads(q, self.talk, mixed, spec.n_heads, spec.n_kv_heads, spec.head_dim)
            ctx.release(q)
            q = mixed
        out = ctx.buffer("attn.out", (n, spec.out_width))
        more = dict(value_dim=spec.v_dim, key_heads=1 if self.talk is None else spec.n_kv_heads,
                    gate=gate, **pooled, **self.extras)
        part_o = part_ml = None
        if ctx.decode:
            splits, waves, heads = self._decode_launch_for(ctx.n_seqs, ctx.context_bound)
            if self.matrix_cores and (aside or gate is not None):
                splits = max(2, splits)      # the merge of slices takes the other source and the gate in
            if splits > 1:
                part_o = ctx.buffer("attn.part_o", (n * spec.n_heads * splits * spec.v_dim,),
                                    torch.float32)
                part_ml = ctx.buffer("attn.part_ml", (n * spec.n_heads * splits * 2,),
                                     torch.float32)
            if self.matrix_cores:
                lib.attention_decode_mfma(q, k_pages, v_pages, meta.row_pos, meta.row_seq,
                                          page_table, out, spec.n_heads, spec.n_kv_heads,
                                          spec.head_dim, window=spec.window, scale=self.scale,
                                          n_splits=splits, part_o=part_o, part_ml=part_ml,
                                          waves=waves, longest=meta.longest, heads=heads,
                                          gate=gate, **aside, **self.extras)
            else:
                item_seq, item_row0, item_npos, n_items = self._items(ctx, "attention.decode_items")
                if self.wide:
                    lib.attention_wide(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                                       meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                                       spec.n_kv_heads, spec.head_dim, window=spec.window,
                                       scale=self.scale, n_splits=splits, part_o=part_o,
                                       part_ml=part_ml, value_dim=spec.v_dim, sinks=self.sinks,
                                       key_heads=spec.n_kv_heads)
                else:
                    lib.attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                                  meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                                  spec.n_kv_heads, spec.head_dim, window=spec.window,
                                  scale=self.scale, n_splits=splits, part_o=part_o,
                                  part_ml=part_ml, **more)
        else:
            key_ways = self.prefill_key_ways([seq.count for seq in ctx.sequences])
            section = self._items_section(key_ways)
            item_seq, item_row0, item_npos, n_items = self._items(ctx, section)
            if self.matrix_cores:
                # the largest item of the list as the host planned it: the kernel's blocks
                # hold a fixed number of rows and are told how many that must cover
                largest = ctx.notes.get(section)
                if largest is None:
                    largest = ctx.notes[section] = int(ctx.meta.host_section(section)[2 * n_items:].max())
                lib.attention_prefill_mfma(q, k_pages, v_pages, item_seq, item_row0, item_npos,
                                           n_items, meta.row_pos, page_table, out, spec.n_heads,
                                           spec.n_kv_heads, spec.head_dim, window=spec.window,
                                           scale=self.scale, key_ways=key_ways,
                                           pair_items=len({(seq.start, seq.count) for seq in ctx.sequences}) == 1,
                                           largest_item=largest, gate=gate, **aside, **self.extras)
            elif self.wide:
                lib.attention_wide(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                                   meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                                   spec.n_kv_heads, spec.head_dim, window=spec.window,
                                   scale=self.scale, value_dim=spec.v_dim, sinks=self.sinks,
                                   key_heads=spec.n_kv_heads)
            else:
                lib.attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                              meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                              spec.n_kv_heads, spec.head_dim, window=spec.window,
                              scale=self.scale, **more)
        if spec.output_gate and not self.head_gate:
            lib.gate_rows(qkv, self.gate_column, out)
        ctx.release(qkv, None if isinstance(q, lib.DecodeProjection) else q, part_o, part_ml, gate,
                    aside.get("pool_o"), aside.get("pool_ml"))
        delta = self.o.forward(ctx, out, "attn.o", bias_later=bias_later)
        ctx.release(out)
        return delta
