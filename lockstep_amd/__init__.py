"""lockstep_amd: a small, whole, batch-invariant inference engine for one GPU
(AMD MI355X, gfx950), with hand-written HIP kernels.

Typical use::

    from lockstep_amd import load_model, Scheduler, Request
    model = load_model("path/to/model", dtype="bfloat16")
    s = Scheduler(model, num_blocks=512)
    s.submit(Request(uid="r0", prompt=[1, 2, 3], max_new_tokens=16))
    outputs = s.run()            # {"r0": [token ids]}
"""

__version__ = "0.1.0"

_LAZY = {
    "load_model": ("lockstep_amd.engine.model", "load_model"),
    "Model": ("lockstep_amd.engine.model", "Model"),
    "StepEntry": ("lockstep_amd.engine.batch", "StepEntry"),
    "Scheduler": ("lockstep_amd.engine.scheduler", "Scheduler"),
    "Request": ("lockstep_amd.engine.scheduler", "Request"),
    "OversizedRequest": ("lockstep_amd.engine.scheduler", "OversizedRequest"),
    "LLM": ("lockstep_amd.engine.llm", "LLM"),
    "EngineConfig": ("lockstep_amd.engine.config", "EngineConfig"),
    "generate_greedy": ("lockstep_amd.engine.llm", "generate_greedy"),
    "DefaultPolicy": ("lockstep_amd.engine.policy", "DefaultPolicy"),
    "FixedChunkPolicy": ("lockstep_amd.engine.policy", "FixedChunkPolicy"),
    "OutOfPages": ("lockstep_amd.cache", "OutOfPages"),
    "write_random_model": ("lockstep_amd.weights", "write_random_model"),
}


def __getattr__(name):
    if name in _LAZY:
        import importlib

        module, attr = _LAZY[name]
        return getattr(importlib.import_module(module), attr)
    raise AttributeError(f"module 'lockstep_amd' has no attribute {name!r}")
