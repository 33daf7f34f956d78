"""The model: parts assembled from a ``ModelSpec``, and the step function.

``Model.step`` is the one way tokens go through the network: a batch of
(request, its next tokens), prompt portions beside single decoded tokens, cut
anywhere.  It runs only the tokens it is given, as one packed batch, on top
of what earlier steps left in the cache, and returns float32 logits at the
wanted places (reference engine/model/qwen3.py:294-378, which computes every
row; here the final norm and the head run on the wanted rows only).
"""

from __future__ import annotations

import itertools
import os
import weakref
from typing import Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..config import ModelConfig, ModelSpec, config_from_dir
from ..parts import WeightSpec, build_part, part_class
from ..parts.base import device_epoch, graph_safe_tree, takes
from ..weights.store import load_weights, weights_from_dict
from .batch import StepContext, StepEntry, Workspace
from .runtime import Runtime
from .tape import LayerTape, RunKinds, TapeMismatch, TapeRefused


def collect_weight_specs(spec: ModelSpec) -> list[WeightSpec]:
    """Every tensor the model expects, in checkpoint order."""
    out = list(part_class(spec.embedding.kind).weight_specs(spec.embedding, ""))
    for layer in spec.layers:
        out += part_class(layer.arrangement.kind).weight_specs(layer)
    out += part_class(spec.final_norm.kind).weight_specs(spec.final_norm, "")
    out += part_class(spec.head.kind).weight_specs(spec.head, "")
    seen, unique = set(), []
    for w in out:
        if w.name not in seen:
            seen.add(w.name)
            unique.append(w)
    return unique


def collect_ties(spec: ModelSpec) -> dict[str, str]:
    head = part_class(spec.head.kind)
    return dict(head.ties(spec.head)) if hasattr(head, "ties") else {}


_MODEL_SERIAL = itertools.count()


class Model:
    def __init__(self, config: ModelConfig, rt: Runtime):
        self.serial = next(_MODEL_SERIAL)
        self.config = config
        self.rt = rt
        self.spec = config.model_spec()
        self.embedding = build_part(self.spec.embedding)
        self.layers = [part_class(layer.arrangement.kind)(layer) for layer in self.spec.layers]
        self.final_norm = build_part(self.spec.final_norm, "")
        self.head = build_part(self.spec.head)
        self.schedule = self.spec.schedule
        for run in self.schedule:
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"the schedule names layer {run.layer}, the model has {len(self.layers)}")
        self.workspace = Workspace(rt.device)
        self.use_graphs = os.environ.get("LOCKSTEP_NO_GRAPHS", "") in ("", "0")
        # debugging aid: every replayed decode step is also run eagerly and the logits compared bit for bit
        self.verify_graphs = os.environ.get("LOCKSTEP_VERIFY_GRAPHS", "") not in ("", "0")
        self._graph_safe = all(graph_safe_tree(part)
                               for part in (self.embedding, *self.layers, self.final_norm, self.head))
        # which arrangements, and the final norm, take over an addition the previous layer left open
        self._layer_takes_pending = [takes(layer.forward, "pending") for layer in self.layers]
        self._final_takes_pending = takes(self.final_norm.forward, "pending")
        # one mixer of each group of equal ones is asked to prepare a step
        seen, self._preparers = set(), []
        for layer in self.layers:
            if layer.mixer is None:                    # a layer without a mixer keeps and prepares nothing
                continue
            group = layer.mixer.prepare_group()
            if group is None or group not in seen:
                self._preparers.append(layer.mixer)
                if group is not None:
                    seen.add(group)
        self.graph_replays = 0
        # layers alike repeat the launches of the second of them (engine/tape.py)
        self.use_tapes = os.environ.get("LOCKSTEP_NO_TAPES", "") in ("", "0")
        self.verify_tapes = os.environ.get("LOCKSTEP_VERIFY_TAPE", "") not in ("", "0")
        # the launches of repeated layers handed to the library as one list ("0": one call a launch, from Python)
        self.list_launches = os.environ.get("LOCKSTEP_LIST_LAUNCHES", "1") not in ("", "0")
        self._run_kinds = weakref.WeakKeyDictionary()      # cache manager -> (device epoch, RunKinds)
        self.layers_repeated = 0
        self.tapes_refused = 0

    @property
    def split_keys(self):
        """Keys of one attention split: the unit in which the mixers' kernels cut a request's keys
        (the smallest, if mixers differ; None if no mixer cuts)."""
        sizes = [layer.mixer.split_keys(self.rt) for layer in self.layers if hasattr(layer.mixer, "split_keys")]
        # (a layer without a mixer has ``mixer`` None, which has no such method)
        return min(sizes) if sizes else None

    def _kinds_for(self, cache) -> RunKinds:
        held = self._run_kinds.get(cache)
        if held is None or held[0] != device_epoch():
            held = self._run_kinds[cache] = (device_epoch(), RunKinds(self, cache))
        return held[1]

    # -- weights --------------------------------------------------------------
    def load(self, weights) -> "Model":
        self.embedding.load(weights, self.rt)
        for layer in self.layers:
            layer.load(weights, self.rt)
        self.final_norm.load(weights, self.rt)
        self.head.load(weights, self.rt)
        return self

    def weight_cast_report(self) -> dict:
        """What casting the checkpoint's tensors to the dtypes they are used in cost: elements
        cast, how many changed value, largest absolute and relative change (all zero for a
        bfloat16 checkpoint on either path)."""
        return dict(self.rt.cast_report)

    # -- cache ------------------------------------------------------------------
    def cache_unit_specs(self) -> list:
        units = [None] * self.spec.cache_units()
        for run in self.schedule:
            mixer = self.layers[run.layer].mixer
            if run.writes_cache and mixer is not None:
                units[run.cache] = mixer.cache_spec()
        return units

    def make_cache(self, num_pages: int, page_size: int = 16, max_requests: int = 64,
                   max_tokens_per_request: int | None = None, poison_on_free: bool = False) -> CacheManager:
        if max_tokens_per_request is None:
            max_tokens_per_request = num_pages * page_size
        return CacheManager(self.cache_unit_specs(), page_size, num_pages, max_requests, max_tokens_per_request,
                            torch_dtype=self.rt.dtype, device=self.rt.device, poison_on_free=poison_on_free)

    # -- the step ------------------------------------------------------------------
    def step(self, cache: CacheManager, entries: Sequence[StepEntry]):
        """Run one batch.  Returns float32 logits ``[wanted, vocab]`` on the
        device in the order of the entries and of their ``want``, or None."""
        entries = [e for e in entries if len(e.tokens)]
        if not entries:
            return None
        vocab = self.spec.vocab_size
        seen = set()
        for e in entries:
            if e.request in seen:
                raise ValueError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) == 1:
                inside = 0 <= int(e.tokens[0]) < vocab
            else:
                ids = np.asarray(e.tokens)
                inside = ids.min() >= 0 and ids.max() < vocab
            if not inside:
                raise ValueError(f"request {e.request!r} brings a token id outside [0, {vocab})")
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise ValueError(f"request {e.request!r} wants logits at {w}, it brings {len(e.tokens)} tokens")
        limit = self.spec.max_positions
        for e in entries:                               # every request's bound before anything is taken for any
            start = cache.length(e.request)
            if limit is not None and start + len(e.tokens) > limit:
                raise ValueError(f"request {e.request!r} would reach {start + len(e.tokens)} tokens; the model's "
                                 f"positions end at {limit}")
        for e in entries:
            start = cache.length(e.request)
            cache.reserve(e.request, start + len(e.tokens))
            if cache.ever_shared:
                for gi in range(len(cache.groups)):
                    for logical in range(start // cache.page_size, -(-(start + len(e.tokens)) // cache.page_size)):
                        cache.assert_exclusive(e.request, gi, logical)
        cache.sync_tables()

        # A step of single decoded tokens has a shape that repeats from step to
        # step: run it from a captured HIP graph.
        graphed = (self.use_graphs and self._graph_safe
                   and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries))
        ctx = StepContext(self.rt, cache, self.workspace, entries, fixed_shape=graphed)
        for mixer in self._preparers:
            mixer.prepare(ctx)
        ctx.upload()
        logits = self._forward_graphed(ctx, cache) if graphed else self._forward(ctx)
        for e, end in zip(entries, ctx.kv_len):
            cache.commit(e.request, int(end))
        return logits

    def _forward(self, ctx: StepContext, logits=None):
        """Launch the step's kernels on the current stream."""
        h = ctx.buf("residual", (ctx.n_tokens, self.spec.hidden_size), torch.float32)
        self.embedding.forward(ctx, ctx.token_ids, h)
        pending = None          # an addition to h that a layer left to the next reader of h
        kernels = self.rt.kernels
        kinds = self._kinds_for(ctx.cache) if self.use_tapes else None
        met: dict = {}          # kind of run -> None after its first run, then (tape, situation, what it left)
        index = -1
        while index + 1 < len(self.schedule):
            index += 1
            run = self.schedule[index]
            kind = kinds.kind[index] if kinds is not None else None
            situation = None
            if kind is not None:
                situation = (self.workspace.version,
                             None if pending is None else (pending.partials.data_ptr(), tuple(pending.partials.shape)))
                held = met.get(kind)
                if held is not None and held[1] == situation and kind in kinds.verified and not self.verify_tapes:
                    if held[0].words is not None:
                        # this layer and the ones like it that follow at once (a repeated layer leaves the
                        # situation it found): their launches go to the library as one list
                        left = held[2]
                        follows = held[1] == (self.workspace.version, None if left is None else (
                            left.partials.data_ptr(), tuple(left.partials.shape)))
                        last = index
                        while follows and last + 1 < len(self.schedule) and kinds.kind[last + 1] == kind:
                            last += 1
                        held[0].repeat_many(kernels, [kinds.addresses[i] for i in range(index, last + 1)])
                        self.layers_repeated += last + 1 - index
                        index = last
                    else:
                        held[0].repeat(kinds.addresses[index])
                        self.layers_repeated += 1
                    pending = held[2]
                    continue
            noting = kind is not None and kind in met
            if noting:
                outer, kernels.tape = kernels.tape, []
            try:
                layer = self.layers[run.layer]
                if self._layer_takes_pending[run.layer]:
                    pending = layer.forward(ctx, run, h, pending=pending)
                else:
                    if pending is not None:
                        pending.flush(ctx, h)
                    pending = None
                    layer.forward(ctx, run, h)
            finally:
                if noting:
                    launches, kernels.tape = kernels.tape, outer
                    if outer is not None:
                        outer.extend(launches)
            if kind is None:
                continue
            if not noting:
                met[kind] = None
                continue
            held = met[kind]
            if held is not None and held[1] == situation:
                # The first layer of a kind that a tape could have stood for (once per model and cache; every
                # one with verify_tapes) ran in Python as well: its launches must be what the tape would launch.
                try:
                    held[0].compare(launches, kinds.addresses[index], f"layer run {index}")
                    kinds.verified.add(kind)
                except TapeMismatch:
                    if self.verify_tapes:
                        raise
                    kinds.refuse(kind)                             # these layers run in Python from now on
                    self.tapes_refused += 1
                    continue
            if situation[0] == self.workspace.version:             # the run did not move the workspace
                try:
                    tape = LayerTape(launches, kinds.addresses[index], kinds.foreign[index])
                    if self.list_launches:
                        tape.as_words(kernels)
                    met[kind] = (tape, situation, pending)
                except TapeRefused:
                    kinds.refuse(kind)
                    self.tapes_refused += 1
        if ctx.n_want:
            x = ctx.buf("final.normed", (ctx.n_want, self.spec.hidden_size), self.rt.dtype)
            if pending is not None and self._final_takes_pending:
                self.final_norm.forward(ctx, h, x, rows=ctx.want_rows, pending=pending)
            else:
                if pending is not None:
                    pending.flush(ctx, h)
                self.final_norm.forward(ctx, h, x, rows=ctx.want_rows)
            if logits is None:
                logits = torch.empty((ctx.n_want, self.spec.vocab_size), dtype=torch.float32, device=self.rt.device)
            self.head.forward(ctx, x, logits)
        return logits

    def _graph_key(self, ctx: StepContext) -> tuple:
        return (self.serial, ctx.n_seqs, ctx.plan_signature(), self.workspace.version, device_epoch())

    def _forward_graphed(self, ctx: StepContext, cache):
        """Replay the captured graph of this step shape, capturing it first if
        needed.  The graph reads the step's metadata, the block tables and the
        cache through fixed addresses; only their contents change between
        replays.  The first step of a shape runs eagerly (that also sizes the
        workspace), then the same launches are recorded for the steps to come.
        Graphs are kept on the cache manager they point into and die with it."""
        graphs = cache.step_graphs
        key = self._graph_key(ctx)
        held = graphs.get(key)
        if held is not None:
            graph, logits = held
            # (the check runs the step twice: per-request state that the step moves on is put back in between)
            before = {unit: t.clone() for unit, t in cache.state.items()} if self.verify_graphs else None
            graph.replay()
            self.graph_replays += 1
            if self.verify_graphs:
                replayed = logits.clone()
                after = {unit: t.clone() for unit, t in cache.state.items()}
                for unit, t in cache.state.items():
                    t.copy_(before[unit])
                eager = self._forward(ctx)
                same_state = all(torch.equal(after[unit].view(torch.uint8), t.view(torch.uint8))
                                 for unit, t in cache.state.items())
                if not (torch.equal(replayed, eager) and same_state):
                    raise RuntimeError("a replayed step graph and the same step run eagerly disagree: a device "
                                       "buffer the graph points at was replaced without the graph key changing")
            return logits.clone()
        logits = torch.empty((ctx.n_want, self.spec.vocab_size), dtype=torch.float32, device=self.rt.device)
        self._forward(ctx, logits)
        key = self._graph_key(ctx)                 # the eager run may have grown the workspace
        graphs.make_room()
        result = logits.clone()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self._forward(ctx, logits)
        graphs[key] = (graph, logits)
        return result


    # -- decode steps without the host ---------------------------------------------------
    LOOP_CAPACITY = 256           # steps one call of the device loop may run

    def decode_greedy(self, cache: CacheManager, requests: Sequence, tokens: Sequence[int], n_steps: int):
        """``n_steps`` decode steps of ``requests`` (ids of open requests whose next input tokens are
        ``tokens``) with the greedy pick of each step fed back on the device: the host launches the
        captured step ``n_steps`` times and reads the picked tokens once at the end.  Returns them as
        an int array ``[n_steps, len(requests)]``.  Logits are those of ``step`` (same kernels, same
        bits), so the tokens equal those of step-by-step greedy decoding."""
        n = len(requests)
        if n == 0 or n_steps <= 0:
            return np.zeros((0, n), dtype=np.int64)
        if len(set(requests)) != n:
            raise ValueError("a request appears twice")
        vocab = self.spec.vocab_size
        if any(not 0 <= int(t) < vocab for t in tokens):
            raise ValueError(f"a token id lies outside [0, {vocab})")
        if not (self.use_graphs and self._graph_safe):
            return self._decode_greedy_stepwise(cache, requests, tokens, n_steps)
        out = []
        tokens = [int(t) for t in tokens]
        while n_steps > 0:
            chunk = min(n_steps, self.LOOP_CAPACITY)
            picked = self._decode_loop(cache, requests, tokens, chunk)
            if picked is None:
                return np.concatenate(out + [self._decode_greedy_stepwise(cache, requests, tokens, n_steps)])
            out.append(picked)
            tokens = picked[-1].tolist()
            n_steps -= chunk
        return np.concatenate(out)

    def decode_sampled(self, cache: CacheManager, requests: Sequence, tokens: Sequence[int], n_steps: int,
                       sampling: Sequence):
        """``decode_greedy`` where some requests draw their tokens: ``sampling[i]`` is None (greedy) or
        ``(temperature > 0, top_p, seed XOR k(uid))``; the draw of a step is keyed on the position of the
        step's input token, as the host sampler keys it.  The sampling kernels run inside the captured
        step and the positions in their records move on with every token, so the tokens equal those of
        step-by-step sampling.  Returns None where the steps cannot run from a captured graph (the caller
        then takes single steps)."""
        if not any(s is not None for s in sampling):
            return self.decode_greedy(cache, requests, tokens, n_steps)
        n = len(requests)
        if n == 0 or n_steps <= 0:
            return np.zeros((0, n), dtype=np.int64)
        if len(set(requests)) != n or len(sampling) != n:
            raise ValueError("a request appears twice, or the sampling list has another length")
        vocab = self.spec.vocab_size
        if any(not 0 <= int(t) < vocab for t in tokens):
            raise ValueError(f"a token id lies outside [0, {vocab})")
        if not (self.use_graphs and self._graph_safe):
            return None
        out = []
        tokens = [int(t) for t in tokens]
        while n_steps > 0:
            chunk = min(n_steps, self.LOOP_CAPACITY)
            picked = self._decode_loop(cache, requests, tokens, chunk, sampling)
            out.append(picked)
            tokens = picked[-1].tolist()
            n_steps -= chunk
        return np.concatenate(out)

    def _decode_greedy_stepwise(self, cache, requests, tokens, n_steps):
        picked = torch.empty(len(requests), dtype=torch.int32, device=self.rt.device)
        out = np.zeros((n_steps, len(requests)), dtype=np.int64)
        tokens = [int(t) for t in tokens]
        for i in range(n_steps):
            logits = self.step(cache, [StepEntry(r, [t], [0]) for r, t in zip(requests, tokens)])
            self.rt.kernels.argmax(logits, picked)
            tokens = picked.cpu().tolist()
            out[i] = tokens
        return out

    def _decode_loop(self, cache, requests, tokens, n_steps, sampling=None):
        n = len(requests)
        starts = [cache.length(r) for r in requests]
        limit = self.spec.max_positions
        for r, start in zip(requests, starts):         # every request's bound before anything is taken for any
            if limit is not None and start + n_steps > limit:
                raise ValueError(f"request {r!r} would reach {start + n_steps} tokens; the model's positions end "
                                 f"at {limit}")
        for r, start in zip(requests, starts):
            cache.reserve(r, start + n_steps)          # every page the loop will write, now
            if cache.ever_shared:
                for gi in range(len(cache.groups)):
                    for logical in range(start // cache.page_size, -(-(start + n_steps) // cache.page_size)):
                        cache.assert_exclusive(r, gi, logical)
        cache.sync_tables()
        entries = [StepEntry(r, [t], [0]) for r, t in zip(requests, tokens)]
        # (a loop of one step is laid out like longer ones, so that they share a graph)
        ctx = StepContext(self.rt, cache, self.workspace, entries, fixed_shape=True, horizon=max(n_steps - 1, 1))
        for mixer in self._preparers:
            mixer.prepare(ctx)
        kernels = self.rt.kernels
        drawn = [i for i in range(n) if sampling is not None and sampling[i] is not None]
        any_nucleus = any(sampling[i][1] < 1.0 for i in drawn)
        if drawn:
            # the sampling kernels' records travel with the step's metadata; the position a draw is keyed on
            # is that of the step's input token and moves on with it
            records = kernels.pack_sample_requests([(i, float(sampling[i][0]), float(sampling[i][1]), int(sampling[i][2]),
                                                     starts[i]) for i in drawn], n)
            ctx.declare(("loop", "sampling"), records,
                        advance=[(kernels.SAMPLE_POSITION_AT, kernels.SAMPLE_ROW_INTS, len(drawn))],
                        signature=("sampling", len(drawn), any_nucleus))
        ctx.upload()
        layout = ctx.meta_layout()
        ring = self.workspace.get("loop.ring", (self.LOOP_CAPACITY * max(n, 64),), torch.int32)
        counter = self.workspace.get("loop.counter", (1,), torch.int32)
        picked = self.workspace.get("loop.picked", (max(n, 64),), torch.int32)
        counter.zero_()

        def one_step(logits):
            self._forward(ctx, logits)
            kernels.argmax(logits, picked[:n])
            if drawn:                                     # the drawn rows' picks replace their arg-max
                kernels.sample_top_p(logits, None, picked, records=ctx.block(("loop", "sampling")),
                                     any_nucleus=any_nucleus, scatter=True)
            kernels.advance_decode(layout["meta"], n, layout["tokens"], picked, ring, counter, *layout["runs"])

        graphs = cache.step_graphs
        key = ("loop",) + self._graph_key(ctx)
        held = graphs.get(key)
        done = 0
        if held is None:
            logits = torch.empty((n, self.spec.vocab_size), dtype=torch.float32, device=self.rt.device)
            one_step(logits)                              # sizes the workspace; it is the loop's first step
            done = 1
            key = ("loop",) + self._graph_key(ctx)
            graphs.make_room()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                one_step(logits)
            graphs[key] = held = (graph, logits)
        graph = held[0]
        for _ in range(n_steps - done):
            graph.replay()
        self.graph_replays += n_steps - done
        out = ring[: n_steps * n].cpu().numpy().reshape(n_steps, n).astype(np.int64)
        for r, start in zip(requests, starts):
            cache.commit(r, start + n_steps)
        return out


def load_model(model_dir, dtype="bfloat16", device="cuda:0") -> Model:
    """Open a folder with config.json and model.safetensors; the class of the
    configuration, and with it the architecture, is chosen by config.json."""
    config = config_from_dir(model_dir)
    rt = Runtime(device, dtype)
    model = Model(config, rt)
    weights = load_weights(model_dir, collect_weight_specs(model.spec), collect_ties(model.spec))
    return model.load(weights)


def model_from_tensors(config: ModelConfig, tensors, dtype="bfloat16", device="cuda:0") -> Model:
    rt = Runtime(device, dtype)
    model = Model(config, rt)
    weights = weights_from_dict(tensors, collect_weight_specs(model.spec), collect_ties(model.spec))
    return model.load(weights)
