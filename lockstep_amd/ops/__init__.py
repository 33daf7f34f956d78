"""Hand-written gfx950 kernels and the code that builds and loads them."""

from .kernels import (ADD_F32, STORE, STORE_F32, SWIGLU, KernelError, Kernels, interleave_gate_up,
                      kernels, pack_attention_items, pack_combine_items)

__all__ = ["ADD_F32", "STORE", "STORE_F32", "SWIGLU", "KernelError", "Kernels", "interleave_gate_up", "kernels",
           "pack_attention_items", "pack_combine_items"]
