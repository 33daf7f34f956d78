"""lockstep_amd: a small, whole, batch-invariant inference engine for one GPU
(AMD MI355X, gfx950), with hand-written HIP kernels."""

__version__ = "0.1.0"
