"""One step's batch: packed tokens, per-request metadata and whatever the parts
add of their own (work lists, slots), built on the host and uploaded in one copy.

A step holds, for each request in it, one run of consecutive tokens that
starts at the request's current length: a whole prompt, a portion of one, or
a single decoded token.  All runs are packed into one ``[T, ...]`` batch.
Device-side layout of the metadata (int32):

    token ids [T] | request index of each token [T] | position of each token [T]
    | per request 8 ints: first row, rows, first position, length after the
      step, block-table row (the request's slot), 0, 0, 0
    | rows whose logits are wanted [W]
    | the blocks that parts declared (``StepContext.declare``), in the order of declaration:
      a mixer's work lists, a state mixer's slots -- whatever its kernels read of the step
    | for steps that go on without the host: the table of (first, stride, count) runs of
      values that move on by one with every decoded token
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Hashable, Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class Workspace:
    """Named device buffers that grow on demand and persist between steps.
    ``version`` counts reallocations: a captured graph that points into these
    buffers is stale once it changes."""

    def __init__(self, device):
        self.device = device
        self._buffers: dict[tuple, torch.Tensor] = {}
        self._views: dict[tuple, torch.Tensor] = {}     # (name, shape, dtype) -> the view of its buffer
        self.version = 0
        self.memo: dict = {}                           # host-side memory of the parts (work-list templates by shape)
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
    """Everything a part may read about the step (see module docstring), and the place where a
    part leaves device-side metadata of its own."""

    def __init__(self, rt, cache, workspace: Workspace, entries: Sequence[StepEntry], fixed_shape: bool = False,
                 horizon: int = 0):
        """``fixed_shape``: the step is one of single decoded tokens whose launches are captured
        in a graph and replayed for later steps of the same shape; a part must then lay its work
        out so that its size depends on the number of requests and on a bucket of the longest
        context only, and may read nothing of the step on the host while it runs.  ``horizon``:
        the layout (and tables indexed by position) must also hold when every request has grown
        by this many more tokens (decode steps that run without the host in between)."""
        self.fixed_shape = fixed_shape
        self.horizon = int(horizon)
        self.rt = rt
        self.cache = cache
        self.workspace = workspace
        self.memo = workspace.memo          # host-side memory of the parts, kept from step to step
        self.notes: dict = {}               # what a part's ``prepare`` leaves for its ``forward`` of this step
        self.entries = list(entries)
        lengths = [len(e.tokens) for e in self.entries]
        self.n_seqs = len(self.entries)
        self.n_tokens = int(sum(lengths))
        self.single_tokens = self.n_tokens == self.n_seqs
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

        if self.single_tokens:
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
        self.seq_rows = seqs                       # [requests, 8] as the device gets them
        self._host_parts: list[np.ndarray] = [tokens, tok_seq, tok_pos, seqs.reshape(-1),
                                              np.asarray(want, dtype=np.int64)]
        self._declared: dict = {}                  # key -> [ints, advance runs, signature, offset]
        self._uploaded = False
        self._meta = None
        self._views = None
        self._runs_at = (0, 0)
        self.host_tokens = tokens

    # -- metadata that parts own -------------------------------------------------------
    def declare(self, key, ints, advance=(), signature=None) -> None:
        """Add a block of int32 values to the step's upload (before ``upload``); ``block(key)``
        is its device view afterwards.  ``advance``: runs ``(first, stride, count)`` inside the
        block whose values move on by one with every token decoded without the host (positions,
        lengths and copies of them).  ``signature``: anything hashable that, beside the block's
        size, must be equal for a captured graph of this step's launches to serve another step."""
        if self._uploaded:
            raise RuntimeError("blocks are declared before the step's metadata is uploaded (in prepare)")
        if key in self._declared:
            raise KeyError(f"block {key!r} was declared twice")
        ints = np.asarray(ints, dtype=np.int64).reshape(-1)
        for first, stride, count in advance:
            if count and not (0 <= first and stride > 0 and first + stride * (count - 1) < ints.shape[0]):
                raise ValueError(f"block {key!r}: the run ({first}, {stride}, {count}) leaves its {ints.shape[0]} ints")
        self._declared[key] = [ints, tuple(tuple(int(v) for v in run) for run in advance), signature, None]

    def declared(self, key) -> bool:
        return key in self._declared

    def block(self, key) -> torch.Tensor:
        ints, _, _, offset = self._declared[key]
        return self._meta[offset:offset + ints.shape[0]]

    def upload(self) -> None:
        """Copy all metadata to the device in one transfer (from a pinned buffer, asynchronously)."""
        t, s = self.n_tokens, self.n_seqs
        parts = list(self._host_parts)
        at = 3 * t + 8 * s + self.n_want
        runs = [(2 * t, 1, t if self.single_tokens else 0),              # positions of the tokens
                (3 * t + 2, 8, s), (3 * t + 3, 8, s)]                     # first position and length of every request
        for entry in self._declared.values():
            entry[3] = at
            parts.append(entry[0])
            runs += [(at + first, stride, count) for first, stride, count in entry[1]]
            at += entry[0].shape[0]
        if self.horizon:
            table = np.asarray([r for r in runs if r[2]], dtype=np.int64).reshape(-1, 3)
            touched = np.concatenate([first + stride * np.arange(count) for first, stride, count in table])
            if np.unique(touched).shape[0] != touched.shape[0]:
                raise ValueError("two runs of values that advance with every decoded token overlap")
            self._runs_at = (at, table.shape[0])
            parts.append(table.reshape(-1))
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
        """Where things lie inside the uploaded metadata (offsets in ints): ``tokens``, and
        ``runs``, the (offset, count) of the table of (first, stride, count) runs that advance
        with every decoded token (present when the step was laid out with a horizon)."""
        return {"tokens": 0, "runs": self._runs_at, "meta": self._meta}

    def _materialize(self) -> dict:
        """Device views of the uploaded metadata (made when a part first asks: a replayed graph never does)."""
        if self._views is not None:
            return self._views
        dev = self._meta
        t, s = self.n_tokens, self.n_seqs
        self._views = {"token_ids": dev[:t], "tok_seq": dev[t:2 * t], "tok_pos": dev[2 * t:3 * t],
                       "seqs": dev[3 * t:3 * t + 8 * s], "want_rows": dev[3 * t + 8 * s:3 * t + 8 * s + self.n_want]}
        return self._views

    token_ids = property(lambda self: self._materialize()["token_ids"])
    tok_seq = property(lambda self: self._materialize()["tok_seq"])
    tok_pos = property(lambda self: self._materialize()["tok_pos"])
    seqs = property(lambda self: self._materialize()["seqs"])
    want_rows = property(lambda self: self._materialize()["want_rows"])

    def plan_signature(self) -> tuple:
        """Sizes of everything uploaded: equal signatures mean an equal device layout."""
        return tuple((key, entry[0].shape[0], entry[2]) for key, entry in self._declared.items()) + (
            self.n_tokens, self.n_want, bool(self.horizon))

    def buf(self, name: str, shape, dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)
