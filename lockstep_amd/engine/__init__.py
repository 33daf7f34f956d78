"""The engine: runtime, step function, scheduler and the user-facing entry points."""
