"""One step's batch: packed tokens, per-request metadata and the attention
work lists, built on the host and uploaded in one copy.

A step holds, for each request in it, one run of consecutive tokens that
starts at the request's current length: a whole prompt, a portion of one, or
a single decoded token.  All runs are packed into one ``[T, ...]`` batch.
Device-side layout of the metadata (int32):

    token ids [T] | request index of each token [T] | position of each token [T]
    | per request 8 ints: first row, rows, first position, length after the
      step, block-table row (the request's slot), 0, 0, 0
    | rows whose logits are wanted [W]
    | attention items (8 ints each) and combine items (4 ints each) per plan
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Hashable, Sequence

import numpy as np
import torch

from ..ops.kernels import pack_attention_items, pack_combine_items


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class AttentionPlan:
    items: torch.Tensor
    n_items: int
    coop_items: torch.Tensor | None
    n_coop: int
    coop_max_rows: int
    decode_fused: bool        # every request brings one token and the fused decode kernel can take the step
    wide_items: torch.Tensor | None
    n_wide: int
    combine_items: torch.Tensor | None
    n_combine: int
    part_acc: torch.Tensor | None
    part_ml: torch.Tensor | None
    wide_variant: int = 4     # 4: row blocks of 128 rows, 5: of 64


class Workspace:
    """Named device buffers that grow on demand and persist between steps.
    ``version`` counts reallocations: a captured graph that points into these
    buffers is stale once it changes."""

    def __init__(self, device):
        self.device = device
        self._buffers: dict[tuple, torch.Tensor] = {}
        self._views: dict[tuple, torch.Tensor] = {}     # (name, shape, dtype) -> the view of its buffer
        self.version = 0
        self.plan_templates: dict[tuple, tuple] = {}   # work lists of decode steps by shape
        self._stage = None                             # pinned host buffer of the metadata upload
        self._stage_np = None
        self._stage_done = None

    def staging(self, n: int):
        """A pinned int32 host buffer of at least ``n`` elements as a numpy view, free to be
        overwritten (its last copy to the device has finished)."""
        if self._stage is None or self._stage.shape[0] < n:
            if self._stage_done is not None:
                self._stage_done.synchronize()
            self._stage = torch.empty(max(2 * n, 4096), dtype=torch.int32, pin_memory=True)
            self._stage_np = self._stage.numpy()
            self._stage_done = torch.cuda.Event()
        elif self._stage_done is not None:
            self._stage_done.synchronize()
        return self._stage, self._stage_np, self._stage_done

    def get(self, name: str, shape, dtype) -> torch.Tensor:
        # the views handed out are kept: a step asks for some two hundred buffers, mostly with the
        # shapes of the step before, and making a view costs more than finding one
        asked = (name, shape if type(shape) is tuple else tuple(shape), dtype)
        view = self._views.get(asked)
        if view is not None:
            return view
        shape = tuple(int(s) for s in shape)
        rows, inner = shape[0], shape[1:]
        key = (name, inner, dtype)
        have = self._buffers.get(key)
        if have is None or have.shape[0] < rows:
            grow = max(rows, 2 * have.shape[0] if have is not None else rows)
            have = torch.empty((grow, *inner), dtype=dtype, device=self.device)
            self._buffers[key] = have
            self.version += 1
            self._views = {k: v for k, v in self._views.items() if (k[0], k[1][1:], k[2]) != key}
        if len(self._views) > 4096:      # many step shapes have gone by: start again
            self._views.clear()
        view = have[:rows]
        self._views[asked] = view
        return view


class StepContext:
    """Everything a part may read about the step (see module docstring)."""

    def __init__(self, rt, cache, workspace: Workspace, entries: Sequence[StepEntry], fixed_shape: bool = False,
                 horizon: int = 0):
        """``fixed_shape`` lays the attention work out so that its size depends
        only on the number of requests and on a bucket of the longest context:
        every request gets one work item per split up to the bucket (items past a
        request's own length produce empty partial results, which the combine
        step skips, so the bits do not change).  A captured graph of the step
        then stays valid from one decode step to the next.  ``horizon``: the
        layout (and the position tables) must also hold when every request has grown
        by this many more tokens (decode steps that run without the host)."""
        self.fixed_shape = fixed_shape
        self.horizon = int(horizon)
        self.rt = rt
        self.cache = cache
        self.workspace = workspace
        self.entries = list(entries)
        lengths = [len(e.tokens) for e in self.entries]
        self.n_seqs = len(self.entries)
        self.n_tokens = int(sum(lengths))
        self._single_tokens = self.n_tokens == self.n_seqs
        # host-side views, also for parts written in plain torch (tests)
        starts = [cache.length(e.request) for e in self.entries]
        offsets = [0] * self.n_seqs
        for i in range(1, self.n_seqs):
            offsets[i] = offsets[i - 1] + lengths[i - 1]
        seqs = np.zeros((self.n_seqs, 8), dtype=np.int64)
        seqs[:, 0], seqs[:, 1], seqs[:, 2] = offsets, lengths, starts
        seqs[:, 3] = seqs[:, 1] + seqs[:, 2]
        seqs[:, 4] = [cache.slot(e.request) for e in self.entries]
        self.q_off, self.q_len, self.q_start, self.kv_len, self.slots = (seqs[:, c] for c in range(5))
        self.max_position = int(self.kv_len.max()) - 1 + self.horizon

        if self._single_tokens:
            tokens = np.asarray([e.tokens[0] for e in self.entries], dtype=np.int64)
            tok_seq = np.arange(self.n_seqs)
            tok_pos = self.q_start
            want = [i for i, e in enumerate(self.entries) for w in e.want]
        else:
            tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in self.entries])
            tok_seq = np.repeat(np.arange(self.n_seqs), self.q_len)
            tok_pos = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, lengths)])
            want = [offsets[i] + int(w) for i, e in enumerate(self.entries) for w in e.want]
        self.n_want = len(want)
        self._seq_rows = seqs
        self._host_parts: list[np.ndarray] = [tokens, tok_seq, tok_pos, seqs.reshape(-1),
                                              np.asarray(want, dtype=np.int64)]
        self._plans: dict[tuple, tuple] = {}
        self._plan_specs: list[tuple] = []
        self._wide_variants: dict[tuple, int] = {}
        self._uploaded = False
        self._meta = None
        self._views = None
        self.host_tokens = tokens

    # -- attention work lists -----------------------------------------------------
    def plan_attention(self, group_size: int, nkv: int, head_dim: int, window: int) -> None:
        """Declare that a mixer with these constants runs in this step (before upload)."""
        key = (group_size, nkv, head_dim, window)
        if key in self._plans:
            return
        tile, split = self.rt.kernels.attention_geometry(head_dim)
        kernels = self.rt.kernels
        coop_ok = kernels.coop_supported(head_dim, self.rt.dtype, self.cache.page_size)
        # with a workgroup per CU anyway, one workgroup walks all splits of a request itself
        whole_requests = self.n_seqs * nkv >= 256
        wide_ok = self.rt.kernels.wide_supported(head_dim, self.rt.dtype, self.cache.page_size)
        wide_variant, wide_rows = 4, self.rt.kernels.attention_block_rows(head_dim, 4)
        if wide_ok:
            # so few rows that the large row blocks would leave half of the CUs without a workgroup: smaller blocks
            blocks = sum(-(-(int(q) * group_size) // wide_rows) for q in self.q_len if int(q) * group_size > 64)
            if 0 < blocks * nkv <= kernels.compute_units() // 2:
                wide_variant, wide_rows = 5, self.rt.kernels.attention_block_rows(head_dim, 5)
        items, coop, wide, combine = [], [], [], []
        coop_max_rows = 0
        part_rows = 0
        bucket = 0
        if self.fixed_shape:
            longest = (int(self.kv_len.max()) + self.horizon - 1) // split + 1
            bucket = 1
            while bucket < longest:
                bucket = bucket * 2 if bucket < 8 else bucket + 8
            if coop_ok and group_size <= 16 and self._single_tokens:
                # a decode step: the lists depend on its shape only, the requests' rows are appended
                shape = (self.n_seqs, group_size, nkv, bucket, whole_requests)
                made = self.workspace.plan_templates.get(shape)
                if made is None:
                    for i in range(self.n_seqs):
                        if whole_requests:
                            coop.append((i, 0, 0, bucket, -1, 0, 0, 0))
                        else:
                            base = part_rows
                            part_rows += nkv * group_size * bucket
                            coop += [(i, 0, s, s + 1, base, bucket, 0, 0) for s in range(bucket)]
                            combine.append((i, 0, base, bucket))
                    made = (np.asarray(coop, dtype=np.int64).reshape(-1, 8),
                            np.asarray(combine, dtype=np.int64).reshape(-1, 4), part_rows)
                    self.workspace.plan_templates[shape] = made
                coop_t, combine_t, part_rows = made
                empty = np.zeros(0, dtype=np.int64)
                decode_fused = kernels.decode_fused_supported(head_dim, self.rt.dtype, self.cache.page_size)
                self._plans[key] = (empty, pack_combine_items(combine_t, self._seq_rows), 0, len(combine_t), part_rows,
                                    pack_attention_items(coop_t, self._seq_rows), len(coop_t), group_size,
                                    empty, 0, decode_fused)
                self._plan_specs.append(key)
                return
        for i in range(self.n_seqs):
            q_len, q_start, kv_len = int(self.q_len[i]), int(self.q_start[i]), int(self.kv_len[i])
            rows = q_len * group_size
            lo_valid = max(0, q_start - window + 1) if window > 0 else 0
            split_lo = lo_valid // split
            n_splits = (kv_len - 1) // split + 1 - split_lo
            if self.fixed_shape:
                split_lo, n_splits = 0, bucket
            # items of at most 16 rows (decoded tokens) go to the cooperative kernel
            target = coop if (coop_ok and rows <= 16) else items
            if target is coop:
                coop_max_rows = max(coop_max_rows, rows)
            if rows <= 64 and (n_splits > 1 or self.fixed_shape) and not (target is coop and whole_requests):
                base = part_rows
                part_rows += nkv * rows * n_splits
                for s in range(split_lo, split_lo + n_splits):
                    target.append((i, 0, s, s + 1, base, n_splits, split_lo, 0))
                combine.append((i, 0, base, n_splits))
            else:
                # long portions go to the wide kernel, in larger row blocks
                if wide_ok and rows > 64:
                    target, block_rows = wide, wide_rows
                else:
                    block_rows = 64
                for block in range(-(-rows // block_rows)):
                    first_pos = q_start + (block * block_rows) // group_size
                    last_pos = q_start + min((block + 1) * block_rows - 1, rows - 1) // group_size
                    begin = (max(0, first_pos - window + 1) // split) if window > 0 else 0
                    target.append((i, block, begin, last_pos // split + 1, -1, 0, 0, 0))
        decode_fused = (coop_ok and not items and not wide and bool((self.q_len == 1).all())
                        and kernels.decode_fused_supported(head_dim, self.rt.dtype, self.cache.page_size))
        # the longest row blocks first: they decide when the launch ends
        wide.sort(key=lambda it: it[2] - it[3])
        self._plans[key] = (pack_attention_items(items, self._seq_rows),
                            pack_combine_items(combine, self._seq_rows), len(items), len(combine), part_rows,
                            pack_attention_items(coop, self._seq_rows), len(coop), coop_max_rows,
                            pack_attention_items(wide, self._seq_rows), len(wide), decode_fused)
        self._wide_variants[key] = wide_variant
        self._plan_specs.append(key)

    def upload(self) -> None:
        """Copy all metadata to the device in one transfer (from a pinned buffer, asynchronously)."""
        parts = list(self._host_parts)
        for key in self._plan_specs:
            items, combine, _, _, _, coop, _, _, wide, _, _ = self._plans[key]
            parts += [items, combine, coop, wide]
        total = sum(p.shape[0] for p in parts)
        stage, view, done = self.workspace.staging(total)
        at = 0
        for p in parts:
            n = p.shape[0]
            if n:
                view[at:at + n] = p
                at += n
        dev = self.workspace.get("step.meta", (total,), torch.int32)
        dev.copy_(stage[:total], non_blocking=True)
        done.record()
        self._meta = dev
        self._views = None
        self._uploaded = True

    def meta_layout(self) -> dict:
        """Where things lie inside the uploaded metadata (offsets in ints): ``tokens``, ``positions``,
        ``seqs`` and ``item_lists``, the (offset, count) of every list of attention work items."""
        t, s = self.n_tokens, self.n_seqs
        at = 3 * t + 8 * s + self.n_want
        lists = []
        for key in self._plan_specs:
            items, combine, n_items, _, _, coop, n_coop, _, wide, n_wide, _ = self._plans[key]
            if n_items:
                lists.append((at, n_items))
            at += items.shape[0] + combine.shape[0]
            if n_coop:
                lists.append((at, n_coop))
            at += coop.shape[0]
            if n_wide:
                lists.append((at, n_wide))
            at += wide.shape[0]
        return {"tokens": 0, "positions": 2 * t, "seqs": 3 * t, "item_lists": lists, "meta": self._meta}

    def _materialize(self) -> dict:
        """Device views of the uploaded metadata (made when a part first asks: a replayed graph never does)."""
        if self._views is not None:
            return self._views
        dev = self._meta
        offset = 0

        def take(n):
            nonlocal offset
            out = dev[offset:offset + n]
            offset += n
            return out

        t, s = self.n_tokens, self.n_seqs
        views = {"token_ids": take(t), "tok_seq": take(t), "tok_pos": take(t), "seqs": take(8 * s),
                 "want_rows": take(self.n_want), "plans": {}}
        for key in self._plan_specs:
            (items, combine, n_items, n_combine, part_rows, coop, n_coop, coop_max_rows, wide, n_wide,
             decode_fused) = self._plans[key]
            head_dim = key[2]
            d_items, d_combine, d_coop = take(items.shape[0]), take(combine.shape[0]), take(coop.shape[0])
            d_wide = take(wide.shape[0])
            part_acc = part_ml = None
            if part_rows:
                part_acc = self.workspace.get(f"attention.part_acc.{head_dim}", (part_rows, head_dim), torch.float32)
                part_ml = self.workspace.get("attention.part_ml", (part_rows, 2), torch.float32)
            views["plans"][key] = AttentionPlan(d_items, n_items, d_coop if n_coop else None, n_coop,
                                                coop_max_rows, decode_fused,
                                                d_wide if n_wide else None, n_wide,
                                                d_combine if n_combine else None,
                                                n_combine, part_acc, part_ml, self._wide_variants.get(key, 4))
        self._views = views
        return views

    token_ids = property(lambda self: self._materialize()["token_ids"])
    tok_seq = property(lambda self: self._materialize()["tok_seq"])
    tok_pos = property(lambda self: self._materialize()["tok_pos"])
    seqs = property(lambda self: self._materialize()["seqs"])
    want_rows = property(lambda self: self._materialize()["want_rows"])

    def plan_signature(self) -> tuple:
        """Sizes of the work lists: equal signatures mean an equal device layout."""
        return tuple((key, self._plans[key][2], self._plans[key][3], self._plans[key][4], self._plans[key][6],
                      self._plans[key][9])
                     for key in self._plan_specs) + (self.n_tokens, self.n_want)

    def attention_plan(self, group_size: int, nkv: int, head_dim: int, window: int) -> AttentionPlan:
        return self._materialize()["plans"][(group_size, nkv, head_dim, window)]

    def buf(self, name: str, shape, dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)
