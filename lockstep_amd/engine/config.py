"""How an engine is run, as one typed value: what the command line, ``LLM``
and ``Scheduler.from_config`` share.  The reference passes these as loose
constructor arguments (engine/sched/scheduler.py:51-60: ``num_blocks``,
``block_size``, ``enable_prefix_cache``, ``audit``, ``eos_token_ids``,
``policy``); the scheduler here still takes them under those names."""

from __future__ import annotations

from dataclasses import dataclass, fields, replace

from ..cache.manager import SUPPORTED_PAGE_SIZES
from .policy import DefaultPolicy, FixedChunkPolicy, Policy


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"                     # "bfloat16" or "float32" (the true 32-bit path)
    page_size: int = 16                         # tokens a cache page holds
    num_pages: int = 512                        # pages in every cache group's pool
    max_running: int = 64                       # requests that run at a time (also the request slots)
    max_batched_tokens: int | None = None       # token budget of one step; None: no bound
    prefill_chunk: int | None = None            # prompts are cut into portions of this many tokens; None: whole
    enable_prefix_cache: bool = False           # finished requests leave their whole pages to later ones
    audit: bool = False                         # check the cache ledger and keep the step ledger every step
    reserve: str = "full"                       # "full": a request's pages at admission; "lazy": step by step
    decode_burst: int = 32                      # greedy decode steps per device-side loop call (1: single steps)
    eos_token_ids: tuple = ()                   # a request stops after emitting one of these
    max_tokens_per_request: int | None = None   # bound of the block table's width; None: the whole pool

    def __post_init__(self):
        object.__setattr__(self, "eos_token_ids", tuple(int(t) for t in (self.eos_token_ids or ())))
        self.validate()

    def validate(self) -> None:
        from .runtime import parse_dtype

        parse_dtype(self.dtype)
        if self.page_size not in SUPPORTED_PAGE_SIZES:
            raise ValueError(f"page_size {self.page_size} is not one of {SUPPORTED_PAGE_SIZES}")
        for name in ("num_pages", "max_running", "decode_burst"):
            if int(getattr(self, name)) < 1:
                raise ValueError(f"{name} must be at least 1, got {getattr(self, name)}")
        for name in ("max_batched_tokens", "prefill_chunk", "max_tokens_per_request"):
            value = getattr(self, name)
            if value is not None and int(value) < 1:
                raise ValueError(f"{name} must be at least 1 or None, got {value}")
        if self.reserve not in ("full", "lazy"):
            raise ValueError(f"reserve must be 'full' or 'lazy', got {self.reserve!r}")

    def policy(self) -> Policy:
        if self.prefill_chunk:
            return FixedChunkPolicy(self.prefill_chunk, max_running=self.max_running)
        return DefaultPolicy(max_running=self.max_running)

    def with_(self, **changes) -> "EngineConfig":
        return replace(self, **changes)

    def to_dict(self) -> dict:
        return {f.name: getattr(self, f.name) for f in fields(self)}
