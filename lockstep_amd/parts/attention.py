"""Grouped-query attention over the paged cache.

Order of operations, as in the reference (engine/model/qwen3.py:327-363):
projections of the normalised hidden rows (no bias), optional RMSNorm per head
on q and k with one ``[d]`` weight for all heads, position encoding on q and
k, keys and values written to the request's pages, causal attention of the
step's queries over everything the request has cached (its own keys of this
step included), output projection added to the residual stream.

The three projections are one matrix product over the concatenation
``[Wq; Wk; Wv]`` (each output column keeps its own sum over the hidden size,
so this changes nothing in the result).  Norm, rotation and cache write are
one kernel; attention is one launch for all requests of the step.
"""

from __future__ import annotations

import os
from dataclasses import dataclass

import numpy as np
import torch

from ..config.base import PartSpec
from ..ops import ADD_F32, STORE_F32, pack_attention_items, pack_combine_items
from .base import Mixer, PagedKVSpec, PendingAdd, WeightSpec, build_part, deferred_rows, register_part

# Steps of single decoded tokens run norm, rotation and cache write inside the
# attention kernel (one launch less per layer); "0" keeps the separate kernel.
FUSE_DECODE = os.environ.get("LOCKSTEP_FUSE_DECODE", "1") not in ("", "0")
# A bound on the (request, kv head) pairs of a step that is fused, for measurements: with the prologue as it
# is now (operands requested ahead of the tile, norm and rotation by row rotations) one launch less pays at every
# batch measured (batch 64: 2.36 -> 2.32 ms a step at 0.6B sizes, 3.35 -> 3.32 at 8B, 3.43 -> 3.41 at 32B; batch
# 128: 3.30 -> 3.25); with the earlier prologue it cost 2 % from 512 pairs on.
FUSE_DECODE_BELOW = int(os.environ.get("LOCKSTEP_FUSE_DECODE_BELOW", str(1 << 30)))
# The most splits one cooperative workgroup walks when a request is cut over several.
MAX_SPAN = int(os.environ.get("LOCKSTEP_MAX_SPAN", "8"))   # splits of a work item where requests of a ragged batch are cut
# Work items (times kv heads) a CU that a decode step of few long requests is cut for.  Measured at 0.6B sizes
# (ms a step, whole requests / this rule / every split an item): 8 requests of 2,048 tokens 2.23 / 1.50 / 1.50,
# 8 of 4,096 - / 1.94 / 1.94 (2.12 with two items a CU), 24 of 512 - / 1.56 / 1.56 (1.65), 16 of 8,192 5.82 / - / 4.34;
# from a workgroup for every CU on, whole requests win (32 of 2,048: 2.70 against 2.87; 32 of 8,192: 6.29 against 7.46;
# 64 of 512 cut in items of three and two splits 2.46 to 2.57 against 2.32, 64 of 4,096 in four to six items 7.5 against 6.9).
WORKGROUPS_A_CU = int(os.environ.get("LOCKSTEP_WORKGROUPS_A_CU", "8"))
RAGGED_RATIO = 2.0         # a batch is ragged when its longest request has more than this many times the mean splits
PART_ROWS_STEP = 4096      # rows of partial results are taken in steps of this many (sizes of replayed steps)
# A step of few decoded tokens whose requests have few splits each leaves the fold of the splits to the output
# product (``gemm_slices_folded``: one launch and one round trip less a layer); every request is then laid out
# with the same number of splits.  Each column block of the product repeats the fold, so this is for few rows
# times splits only.  "0" switches it off.
FOLD_IN_PRODUCT = os.environ.get("LOCKSTEP_FOLD_IN_PRODUCT", "1") not in ("", "0")
# Items of one key tile of a fused decode step bring the tile's page ids along, so that the kernel's tile loads
# need no look-up in the block table first; "0" switches it off.
EMBED_PAGES = os.environ.get("LOCKSTEP_EMBED_PAGES", "1") not in ("", "0")
FOLD_MAX_SPLITS = int(os.environ.get("LOCKSTEP_FOLD_MAX_SPLITS", "8"))
FOLD_MAX_ROW_SPLITS = int(os.environ.get("LOCKSTEP_FOLD_MAX_ROW_SPLITS", "128"))   # requests times splits
# ... and for output products of at most this many columns: every block of 64 columns repeats the fold (measured at
# 4,096 columns, Qwen3-8B sizes: 1 % slower at 8 requests and 8 % at 16 than the combine launch; at 1,024 columns
# the fold is ahead at every batch it takes)
FOLD_MAX_COLUMNS = int(os.environ.get("LOCKSTEP_FOLD_MAX_COLUMNS", "2048"))


# ---------------------------------------------------------------------------
# The step's attention work, laid out on the host.  The lists go into the step's
# upload as one declared block per set of attention constants (layers with the
# same constants share it); the kernels read them from there.
# ---------------------------------------------------------------------------

@dataclass
class AttentionPlan:
    """Where the lists of one set of attention constants lie inside their block, and what the
    launches need to know about them."""

    n_items: int              # staged / direct items (32 ints each), first in the block
    n_combine: int            # combine items (8 ints each)
    n_coop: int               # cooperative items (decoded tokens)
    coop_max_rows: int
    n_wide: int               # wide items (long prompt portions)
    part_rows: int            # rows of partial results the split items leave
    decode_fused: bool        # every request brings one token and the fused decode kernel can take the step
    wide_variant: int = 4     # 4: row blocks of 128 rows, 5: of 64
    spans: bool = False       # cooperative items that leave partial results hold several splits each
    #: > 0: single decoded tokens only, every request laid out with this many splits, partial row of
    #: (request i, head h, split s) = (i * heads + h) * fold_splits + s: the output product may fold them itself
    fold_splits: int = 0
    single_tile: bool = False  # every cooperative item holds one key tile (one tile buffer a workgroup is enough)

    ITEM, COMBINE = 32, 8

    def offsets(self):
        items = 0
        combine = items + self.ITEM * self.n_items
        coop = combine + self.COMBINE * self.n_combine
        wide = coop + self.ITEM * self.n_coop
        return items, combine, coop, wide, wide + self.ITEM * self.n_wide

    def signature(self):
        return (self.n_items, self.n_combine, self.n_coop, self.n_wide, self.part_rows, self.decode_fused,
                self.wide_variant, self.spans, self.fold_splits, self.single_tile)


def _round_up(n: int, buckets=(1, 2, 4, 8, 12, 16, 24, 32, 40, 48, 56, 64), step: int = 16) -> int:
    """``n`` rounded up to one of a few sizes (then to a multiple of ``step``): list sizes of
    graph-replayed steps, so that one graph serves many steps."""
    for b in buckets:
        if n <= b:
            return b
    return -(-n // step) * step


def plan_attention(ctx, group_size: int, nkv: int, head_dim: int, window: int, out_columns: int = 0):
    """Work items of one set of attention constants for this step: (plan, ints of the block).

    Requests are cut at the kernels' own, position-anchored splits; which kernel takes a request
    and whether a workgroup walks a request's splits itself or leaves a partial result per split
    to the fold is chosen here freely, because every choice gives the same bits.

    Decoded tokens (at most 16 rows a kv head) go to the cooperative kernel.  While the step's
    splits would not fill the GPU twice over, every split is a work item of its own.  Beyond
    that a workgroup walks a whole request and writes the output -- unless there are too few
    requests for that to give every CU two workgroups (a CU alone streams slowly: eight
    requests of 4,096 tokens walked whole keep a quarter of the GPU busy), then requests are cut
    into the longest items that still do; and unless the requests are of very different
    lengths: a workgroup takes a few microseconds a tile whatever else runs, so the longest
    request would decide when the launch ends; requests are then cut into items of at most
    MAX_SPAN splits.  With ``ctx.fixed_shape`` (a step whose launches are captured and replayed)
    the lists are laid out for the lengths the requests will have ``ctx.horizon`` tokens on,
    and their sizes are rounded up with null items, so that one graph serves the steps to come."""
    kernels, dtype, page_size = ctx.rt.kernels, ctx.rt.dtype, ctx.cache.page_size
    tile, split = kernels.attention_geometry(head_dim)
    coop_ok = kernels.coop_supported(head_dim, dtype, page_size)
    wide_ok = kernels.wide_supported(head_dim, dtype, page_size)
    wide_variant, wide_rows = 4, kernels.attention_block_rows(head_dim, 4)
    if wide_ok:
        # so few rows that the large row blocks would leave half of the CUs without a workgroup: smaller blocks
        blocks = sum(-(-(int(q) * group_size) // wide_rows) for q in ctx.q_len if int(q) * group_size > 64)
        if 0 < blocks * nkv <= kernels.compute_units() // 2:
            wide_variant, wide_rows = 5, kernels.attention_block_rows(head_dim, 5)

    # splits every request has (when the step's last token of the horizon is in): first, count
    first_query = ctx.q_start
    lo = (np.maximum(0, first_query - window + 1) // split) if window > 0 else np.zeros(ctx.n_seqs, dtype=np.int64)
    counts = (ctx.kv_len + ctx.horizon - 1) // split + 1 - lo
    rows_of = ctx.q_len * group_size
    to_coop = (rows_of <= 16) & coop_ok
    span = 1
    if to_coop.any():
        mine = counts[to_coop]
        cus = kernels.compute_units()
        if len(mine) * nkv >= cus:
            span = int(mine.max())                              # a workgroup for every CU: requests are walked whole
        else:
            # fewer: items of one split (one tile, the kernel's shortest chain) while their number stays moderate,
            # else the longest items that still give every CU WORKGROUPS_A_CU of them
            enough = WORKGROUPS_A_CU * cus
            if int(mine.sum()) * nkv >= enough:
                low, high = 1, int(mine.max())
                while low < high:
                    middle = (low + high + 1) // 2
                    if int((-(-mine // middle)).sum()) * nkv >= enough:
                        low = middle
                    else:
                        high = middle - 1
                span = low
        if span > 1 and int(mine.max()) > RAGGED_RATIO * float(mine.mean()):
            span = min(span, MAX_SPAN)

    fold_splits = 0
    if (FOLD_IN_PRODUCT and 0 < out_columns <= FOLD_MAX_COLUMNS and span == 1 and window == 0 and ctx.n_seqs <= 16
            and bool(to_coop.all())
            and bool((ctx.q_len == 1).all())):
        most = int(counts.max())
        # (with one split everywhere nothing is folded anyway: the workgroups write the output themselves)
        if 2 <= most <= FOLD_MAX_SPLITS and most * ctx.n_seqs <= FOLD_MAX_ROW_SPLITS:
            fold_splits = most

    items, coop, wide, combine = [], [], [], []
    coop_max_rows = part_rows = 0
    for i in range(ctx.n_seqs):
        if fold_splits:
            # the same number of splits for every request (those beyond a request's end leave empty sums), the
            # partial rows of a request one after the other in the order of its heads
            base = i * nkv * group_size * fold_splits
            coop_max_rows = max(coop_max_rows, group_size)
            coop += [(i, 0, int(lo[i]) + s, int(lo[i]) + s + 1, base, fold_splits, int(lo[i]), 0) for s in range(fold_splits)]
            combine.append((i, 0, base, fold_splits))
            part_rows = base + nkv * group_size * fold_splits
            continue
        q_len, q_start = int(ctx.q_len[i]), int(ctx.q_start[i])
        rows = int(rows_of[i])
        split_lo, n_splits = int(lo[i]), int(counts[i])
        if to_coop[i]:
            coop_max_rows = max(coop_max_rows, rows)
            if n_splits <= span:
                coop.append((i, 0, split_lo, split_lo + n_splits, -1, 0, 0, 0))       # writes the output itself
            else:
                base = part_rows
                part_rows += nkv * rows * n_splits
                pieces = -(-n_splits // span)
                even = -(-n_splits // pieces)               # items of even length: the longest decides
                for first in range(split_lo, split_lo + n_splits, even):
                    coop.append((i, 0, first, min(first + even, split_lo + n_splits), base, n_splits, split_lo, 0))
                combine.append((i, 0, base, n_splits))
        elif rows <= 64 and (n_splits > 1 or ctx.fixed_shape):
            base = part_rows
            part_rows += nkv * rows * n_splits
            for first in range(split_lo, split_lo + n_splits):
                items.append((i, 0, first, first + 1, base, n_splits, split_lo, 0))
            combine.append((i, 0, base, n_splits))
        else:
            # long portions go to the wide kernel, in larger row blocks
            target, block_rows = (wide, wide_rows) if (wide_ok and rows > 64) else (items, 64)
            for block in range(-(-rows // block_rows)):
                first_pos = q_start + (block * block_rows) // group_size
                last_pos = q_start + min((block + 1) * block_rows - 1, rows - 1) // group_size
                begin = (max(0, first_pos - window + 1) // split) if window > 0 else 0
                target.append((i, block, begin, last_pos // split + 1, -1, 0, 0, 0))
    if ctx.fixed_shape:
        # null work (request -1 here, an item of zeros on the device) up to a size that many steps share
        null_item, null_fold = (-1, 0, 0, 0, -1, 0, 0, 0), (-1, 0, 0, 0)
        for work, null in ((items, null_item), (coop, null_item), (combine, null_fold)):
            if work:
                work += [null] * (_round_up(len(work)) - len(work))
        part_rows = _round_up(part_rows, buckets=(), step=PART_ROWS_STEP) if part_rows else 0
    decode_fused = (coop_ok and not items and not wide and bool((ctx.q_len == 1).all())
                    and kernels.decode_fused_supported(head_dim, dtype, page_size))
    # the longest row blocks first: they decide when the launch ends
    wide.sort(key=lambda it: it[2] - it[3])
    spans = any(it[4] >= 0 and it[3] - it[2] > 1 for it in coop)
    single_tile = bool(coop) and all((it[3] - it[2]) * split <= tile for it in coop)
    plan = AttentionPlan(len(items), len(combine), len(coop), coop_max_rows, len(wide), part_rows, decode_fused,
                         wide_variant, spans, fold_splits, single_tile)
    coop_pages = None
    if EMBED_PAGES and decode_fused and single_tile and split == tile and tile // page_size <= 16:
        coop_pages = tile_page_ids(ctx, coop, nkv, head_dim, window, tile)
    return plan, np.concatenate([pack_attention_items(items, ctx.seq_rows), pack_combine_items(combine, ctx.seq_rows),
                                 pack_attention_items(coop, ctx.seq_rows, coop_pages),
                                 pack_attention_items(wide, ctx.seq_rows)])


def tile_page_ids(ctx, coop, nkv: int, head_dim: int, window: int, tile: int):
    """The block-table entries of the one key tile of every cooperative item (``[items, 16]``, -1 where the
    request holds no page), read from the host's copy of the table of the cache group with these constants;
    None if no group has them."""
    cache, page_size = ctx.cache, ctx.cache.page_size
    group = next((g for g in cache.groups if (g.spec.num_kv_heads, g.spec.head_dim, g.spec.window or 0)
                  == (nkv, head_dim, window)), None)
    if group is None:
        return None
    per_tile = tile // page_size
    work = np.asarray(coop, dtype=np.int64).reshape(-1, 8)
    live = work[:, 0] >= 0
    slots = ctx.slots[np.maximum(work[:, 0], 0)]
    first = work[:, 2] * per_tile                                        # first logical page of the item's tile
    columns = first[:, None] + np.arange(per_tile)[None, :]
    inside = columns < group.table_host.shape[1]
    ids = np.where(inside, group.table_host[slots[:, None], np.minimum(columns, group.table_host.shape[1] - 1)], -1)
    out = np.full((len(work), 16), -1, dtype=np.int64)
    out[:, :per_tile] = np.where(live[:, None], ids, -1)
    return out


def advancing_fields(plan: AttentionPlan):
    """The copies of a request's first position and length inside the attention items: they move
    on with every token decoded without the host."""
    items, _, coop, wide, _ = plan.offsets()
    runs = []
    for first, count in ((items, plan.n_items), (coop, plan.n_coop), (wide, plan.n_wide)):
        runs += [(first + 10, AttentionPlan.ITEM, count), (first + 11, AttentionPlan.ITEM, count)]
    return [r for r in runs if r[2]]


@register_part("attention")
class Attention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``,
    ``head_dim``, ``qk_norm`` (a norm ``PartSpec`` or None), ``position`` (a
    position-encoding ``PartSpec``), ``window`` (keys visible to a query,
    None for all), ``bias`` (biases of the q, k and v projections), ``out_bias`` (optional, a
    bias of the output projection), ``scale`` (score multiplier)."""

    graph_safe = True
    repeatable = True

    def parts(self):
        return (self.position,)

    def __init__(self, spec: PartSpec, prefix: str = ""):
        super().__init__(spec, prefix)
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nq = int(p["num_heads"])
        self.nkv = int(p["num_kv_heads"])
        self.d = int(p["head_dim"])
        self.window = p.get("window")
        self.scale = float(p["scale"])
        self.bias = bool(p.get("bias"))              # q_proj.bias, k_proj.bias, v_proj.bias
        self.out_bias = bool(p.get("out_bias"))      # o_proj.bias
        if self.nq % self.nkv:
            raise ValueError(f"{self.nq} query heads are not a multiple of {self.nkv} kv heads")
        if self.d % 16 or not 16 <= self.d <= 256:
            raise ValueError(f"head size {self.d} is not supported: the attention kernels take "
                             "multiples of 16 from 16 to 256")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"window {self.window} must be positive")
        self.qk_norm_spec = p.get("qk_norm")
        self.position = build_part(p["position"], prefix)
        if self.position.rotary_dim > self.d:
            raise ValueError(f"rotary_dim {self.position.rotary_dim} exceeds head size {self.d}")
        self.w_qkv = self.w_q = self.w_o = self.q_norm = self.k_norm = None
        self.b_qkv = self.b_q = self.b_o = None
        self.norm_eps = float(self.qk_norm_spec["eps"]) if self.qk_norm_spec else 0.0
        if self.qk_norm_spec is not None:
            if self.qk_norm_spec.kind != "rmsnorm" or int(self.qk_norm_spec["size"]) != self.d:
                raise ValueError("the per-head norm must be an rmsnorm over the head size")

    @classmethod
    def weight_specs(cls, spec: PartSpec, prefix: str) -> list[WeightSpec]:
        p = spec.params
        h, nq, nkv, d = int(p["hidden_size"]), int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        out = [
            WeightSpec(f"{prefix}.q_proj.weight", (nq * d, h)),
            WeightSpec(f"{prefix}.k_proj.weight", (nkv * d, h)),
            WeightSpec(f"{prefix}.v_proj.weight", (nkv * d, h)),
            WeightSpec(f"{prefix}.o_proj.weight", (h, nq * d)),
        ]
        if p.get("qk_norm") is not None:
            out += [WeightSpec(f"{prefix}.q_norm.weight", (d,), kind="vector", init="norm"),
                    WeightSpec(f"{prefix}.k_norm.weight", (d,), kind="vector", init="norm")]
        if p.get("bias"):
            out += [WeightSpec(f"{prefix}.q_proj.bias", (nq * d,), kind="vector"),
                    WeightSpec(f"{prefix}.k_proj.bias", (nkv * d,), kind="vector"),
                    WeightSpec(f"{prefix}.v_proj.bias", (nkv * d,), kind="vector")]
        if p.get("out_bias"):
            out.append(WeightSpec(f"{prefix}.o_proj.bias", (h,), kind="vector"))
        return out

    def cache_spec(self):
        return PagedKVSpec(self.nkv, self.d, int(self.window) if self.window is not None else None)

    def load(self, weights, rt) -> None:
        q = weights.get(f"{self.prefix}.q_proj.weight")
        k = weights.get(f"{self.prefix}.k_proj.weight")
        v = weights.get(f"{self.prefix}.v_proj.weight")
        order = self.position.dim_order(self.d) if hasattr(self.position, "dim_order") else None
        if order is not None:
            order = torch.as_tensor(list(order), dtype=torch.long)
            if sorted(order.tolist()) != list(range(self.d)):
                raise ValueError(f"the position encoding's dim_order is no permutation of range({self.d})")
            q = q.view(self.nq, self.d, -1)[:, order].reshape(q.shape)       # every head's dimensions alike
            k = k.view(self.nkv, self.d, -1)[:, order].reshape(k.shape)
        self.w_qkv = rt.matrix(torch.cat([q.to(torch.float32), k.to(torch.float32), v.to(torch.float32)], dim=0)
                               if len({q.dtype, k.dtype, v.dtype}) > 1 else torch.cat([q, k, v], dim=0))
        self.w_q = self.w_qkv[: self.nq * self.d]
        self.w_o = rt.matrix(weights.get(f"{self.prefix}.o_proj.weight"))
        if self.bias:
            bq, bk, bv = (weights.get(f"{self.prefix}.{n}_proj.bias").to(torch.float32) for n in "qkv")
            if order is not None:
                bq = bq.view(self.nq, self.d)[:, order].reshape(-1)
                bk = bk.view(self.nkv, self.d)[:, order].reshape(-1)
            self.b_qkv = rt.vector(torch.cat([bq, bk, bv]))
            self.b_q = self.b_qkv[: self.nq * self.d]
        if self.out_bias:
            self.b_o = rt.vector(weights.get(f"{self.prefix}.o_proj.bias"))
        if self.qk_norm_spec is not None:
            q_norm, k_norm = weights.get(f"{self.prefix}.q_norm.weight"), weights.get(f"{self.prefix}.k_norm.weight")
            if order is not None:
                q_norm, k_norm = q_norm[order], k_norm[order]
            self.q_norm = rt.vector(q_norm)
            self.k_norm = rt.vector(k_norm)
        rt.kernels.attention_lib(self.d)
        if hasattr(self.position, "bind"):
            self.position.bind(rt)      # layers with equal constants share their tables

    def mixing_flops(self, tokens: int, start: int) -> float:
        """Scores and value products over the (query, key) pairs a query sees."""
        window = int(self.window) if self.window is not None else None
        pairs = sum(min(start + i + 1, window or start + i + 1) for i in range(tokens))
        return 4.0 * self.d * self.nq * pairs

    def split_keys(self, rt) -> int:
        """Keys of one split of the attention kernels for this head size."""
        return int(rt.kernels.attention_geometry(self.d)[1])

    def prepare_group(self):
        share = getattr(self.position, "share_key", None)
        if share is None:
            return None
        return ("attention", self.nq, self.nkv, self.d, self.window, share())

    def _block_key(self):
        window = int(self.window) if self.window is not None else 0
        # (the width of the output product is part of the plan: the fold of the splits may be left to it)
        return ("attention", self.nq // self.nkv, self.nkv, self.d, window, self.hidden)

    def prepare(self, ctx) -> None:
        self.position.ensure(ctx.max_position + 1, ctx.rt)
        key = self._block_key()
        if ctx.declared(key):
            return
        plan, ints = plan_attention(ctx, *key[1:])
        ctx.declare(key, ints, advance=advancing_fields(plan), signature=plan.signature())
        ctx.notes[key] = plan                         # for forward, which runs after the upload

    def forward(self, ctx, run, x, out, accumulate: bool, norm=None, defer: bool = False):
        """``norm``: when given, ``x`` is the float32 residual stream and ``norm``
        (an RMSNorm part) is applied inside the projection.  ``defer``: the addition
        of the output projection to ``out`` may be left to the caller (a ``PendingAdd``
        is returned)."""
        rt = ctx.rt
        k = rt.kernels
        t = ctx.n_tokens
        nq, nkv, d = self.nq, self.nkv, self.d
        group, key_pages, value_pages = ctx.cache.unit_pages(run.cache)
        width = (nq + 2 * nkv) * d
        qkv = ctx.buf("attention.qkv", (t, width), rt.dtype)
        fused = {} if norm is None else {"norm_weight": norm.weight, "eps": norm.eps}
        if self.b_qkv is not None:
            # biases: the product in float32, then a pass that adds them and rounds to the compute dtype
            raw = ctx.buf("attention.qkv_f32", (t, width), torch.float32)
            if run.writes_cache:
                k.gemm(x, self.w_qkv, raw, STORE_F32, **fused)
                k.bias_act(raw, self.b_qkv, qkv)
            else:
                k.gemm(x, self.w_q, raw[:, : nq * d], STORE_F32, **fused)
                k.bias_act(raw[:, : nq * d], self.b_q, qkv[:, : nq * d])
        elif run.writes_cache:
            k.gemm(x, self.w_qkv, qkv, **fused)
        else:
            k.gemm(x, self.w_q, qkv[:, : nq * d], **fused)
        attn = ctx.buf("attention.out", (t, nq * d), rt.dtype)
        window = int(self.window) if self.window is not None else 0
        key = self._block_key()
        plan = ctx.notes[key]
        block = ctx.block(key)
        at_items, at_combine, at_coop, at_wide, end = plan.offsets()
        items, combine_items = block[at_items:at_combine], block[at_combine:at_coop]
        coop_items, wide_items = block[at_coop:at_wide], block[at_wide:end]
        part_acc = part_ml = None
        if plan.part_rows:
            part_acc = ctx.buf(f"attention.part_acc.{d}", (plan.part_rows, d), torch.float32)
            part_ml = ctx.buf("attention.part_ml", (plan.part_rows, 2), torch.float32)
        if plan.decode_fused and FUSE_DECODE and ctx.n_seqs * nkv < FUSE_DECODE_BELOW:
            # single decoded tokens: norm, rotation and cache write happen inside the attention kernel
            k.attention_decode(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                               coop_items, plan.n_coop, attn, part_acc, part_ml, self.scale, window,
                               self.q_norm, self.k_norm, self.norm_eps, self.position.cos, self.position.sin,
                               self.position.rotary_dim, ctx.max_position, run.writes_cache, plan.spans,
                               plan.single_tile)
            folded = self._folded_operand(ctx, plan, part_acc, part_ml, out, accumulate, defer)
            if plan.n_combine and folded is None:
                k.attention_combine(d, ctx.seqs, combine_items, plan.n_combine, nq, nkv, part_acc, part_ml, attn,
                                    max_rows=plan.coop_max_rows if not plan.n_items else 0)
            return self._project_out(ctx, attn, out, accumulate, defer, folded)
        k.qk_rope_kv(qkv, t, nq, nkv, d, self.q_norm, self.k_norm, self.norm_eps, self.position.cos,
                     self.position.sin, self.position.rotary_dim, ctx.tok_seq, ctx.tok_pos, ctx.seqs,
                     ctx.max_position, group.table, key_pages, value_pages, group.page_size, run.writes_cache)
        if plan.n_items:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        items, plan.n_items, attn, part_acc, part_ml, self.scale, window)
        if plan.n_coop:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        coop_items, plan.n_coop, attn, part_acc, part_ml, self.scale, window,
                        variant=3, max_rows=plan.coop_max_rows, spans=plan.spans, single_tile=plan.single_tile)
        if plan.n_wide:
            k.attention(qkv, nq, nkv, d, key_pages, value_pages, group.page_size, group.table, ctx.seqs,
                        wide_items, plan.n_wide, attn, part_acc, part_ml, self.scale, window,
                        variant=plan.wide_variant)
        folded = self._folded_operand(ctx, plan, part_acc, part_ml, out, accumulate, defer)
        if plan.n_combine and folded is None:
            k.attention_combine(d, ctx.seqs, combine_items, plan.n_combine, nq, nkv, part_acc, part_ml, attn,
                                    max_rows=plan.coop_max_rows if not plan.n_items else 0)
        return self._project_out(ctx, attn, out, accumulate, defer, folded)

    def _folded_operand(self, ctx, plan, part_acc, part_ml, out, accumulate: bool, defer: bool):
        """(part_acc, part_ml, splits) if the output product of this step can fold the splits' partial
        results itself (the plan laid them out for it, the product is left as slice sums, and the kernel
        takes these sizes), else None: the combine launch folds them into the attention output."""
        if not plan.fold_splits or not (defer and accumulate) or self.b_o is not None:
            return None
        if not 0 < ctx.n_tokens <= deferred_rows(ctx, self.nq * self.d, out.shape[1]):
            return None
        if not ctx.rt.kernels.gemm_slices_folded_ok(ctx.rt.dtype, ctx.n_tokens, out.shape[1], self.nq * self.d, self.d,
                                                    plan.fold_splits):
            return None
        return part_acc, part_ml, plan.fold_splits

    def _project_out(self, ctx, attn, out, accumulate: bool, defer: bool, folded=None):
        k = ctx.rt.kernels
        if folded is not None:
            slices = k.gemm_slices_count(self.nq * self.d)
            partials = ctx.buf("attention.out_slices", (slices * ctx.n_tokens, out.shape[1]), torch.float32)
            partials = partials.view(slices, ctx.n_tokens, out.shape[1])
            k.gemm_slices_folded(folded[0], folded[1], folded[2], self.d, self.w_o, partials)
            return PendingAdd(partials)
        if self.b_o is not None:
            # (stream + product) + bias, at once: the order of the additions must not depend on the batch
            k.gemm(attn, self.w_o, out, ADD_F32 if accumulate else STORE_F32)
            k.bias_act(out, self.b_o, out)
            return None
        if defer and accumulate and 0 < ctx.n_tokens <= deferred_rows(ctx, self.nq * self.d, out.shape[1]):
            slices = k.gemm_slices_count(self.nq * self.d)
            partials = ctx.buf("attention.out_slices", (slices * ctx.n_tokens, out.shape[1]), torch.float32)
            partials = partials.view(slices, ctx.n_tokens, out.shape[1])
            k.gemm_slices(attn, self.w_o, partials)
            return PendingAdd(partials)
        k.gemm(attn, self.w_o, out, ADD_F32 if accumulate else STORE_F32)
        return None
