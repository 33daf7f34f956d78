"""The tape of one layer's launches (engine/tape.py) on the host: where a layer's addresses are
found among the arguments, what another layer's launches look like, and what the comparison of
verify mode reports."""

from __future__ import annotations

from ctypes import c_float, c_int, c_void_p

import pytest

from lockstep_amd.engine.tape import LayerTape
from lockstep_amd.ops.kernels import KernelError


class FakeLibrary:
    def __init__(self):
        self.calls = []
        self.fail = False

    def entry(self, *args):
        self.calls.append([getattr(a, "value", a) for a in args])
        return 1 if self.fail else 0

    def ls_last_error(self):
        return b"refused"


def launches_of(lib, weights, cache, workspace=0x9000):
    return [(lib, lib.entry, (c_int(3), c_void_p(workspace), c_void_p(weights), c_void_p(0), c_float(1e-6))),
            (lib, lib.entry, (c_void_p(weights + 64), c_void_p(cache), c_void_p(cache + 4096), c_int(7)))]


def addresses(weights, cache):
    return {"w_qkv": (weights, 4096), "w_q": (weights, 1024), "cache[0]": (cache, 1 << 20)}


def test_addresses_of_the_noted_layer_are_replaced_and_nothing_else():
    lib = FakeLibrary()
    tape = LayerTape(launches_of(lib, 0x100000, 0x800000), addresses(0x100000, 0x800000))
    tape.repeat(addresses(0x300000, 0xA00000))
    assert lib.calls == [[3, 0x9000, 0x300000, None, pytest.approx(1e-6)],
                         [0x300000 + 64, 0xA00000, 0xA00000 + 4096, 7]]
    # the tape itself is unchanged: a third layer starts from the noted one again
    lib.calls.clear()
    tape.repeat(addresses(0x500000, 0xC00000))
    assert lib.calls[1] == [0x500000 + 64, 0xC00000, 0xC00000 + 4096, 7]


def test_a_view_into_a_larger_tensor_keeps_its_offset():
    lib = FakeLibrary()
    where = {"w_qkv": (0x100000, 4096), "w_q": (0x100000, 1024)}
    tape = LayerTape([(lib, lib.entry, (c_void_p(0x100000 + 2048),))], where)     # beyond w_q, inside w_qkv
    tape.repeat({"w_qkv": (0x700000, 4096), "w_q": (0x700000, 1024)})
    assert lib.calls == [[0x700000 + 2048]]


def test_a_refused_launch_raises_the_library_error():
    lib = FakeLibrary()
    tape = LayerTape(launches_of(lib, 0x100000, 0x800000), addresses(0x100000, 0x800000))
    lib.fail = True
    with pytest.raises(KernelError, match="refused"):
        tape.repeat(addresses(0x300000, 0xA00000))


def test_compare_accepts_the_same_launches_and_names_the_first_other_one():
    lib = FakeLibrary()
    tape = LayerTape(launches_of(lib, 0x100000, 0x800000), addresses(0x100000, 0x800000))
    tape.compare(launches_of(lib, 0x300000, 0xA00000), addresses(0x300000, 0xA00000), "layer run 2")
    other = launches_of(lib, 0x300000, 0xA00000)
    other[1] = (lib, lib.entry, (c_void_p(0x300000 + 64), c_void_p(0xA00000), c_void_p(0xA00000 + 4096), c_int(8)))
    with pytest.raises(RuntimeError, match="layer run 2: launch 1 .* differs from the tape"):
        tape.compare(other, addresses(0x300000, 0xA00000), "layer run 2")
    with pytest.raises(RuntimeError, match="launched 1 kernels, the tape holds 2"):
        tape.compare(other[:1], addresses(0x300000, 0xA00000), "layer run 2")
    # an address that should have been this layer's own but was the noted layer's
    stale = launches_of(lib, 0x300000, 0xA00000)
    stale[0] = launches_of(lib, 0x100000, 0xA00000)[0]
    with pytest.raises(RuntimeError, match="launch 0"):
        tape.compare(stale, addresses(0x300000, 0xA00000), "layer run 2")


def test_an_address_inside_another_layers_tensor_refuses_the_tape():
    """A launch of the noted layer names a tensor that is listed for another layer only: the noted
    layer holds it somewhere the walk over its attributes does not reach."""
    from lockstep_amd.engine.tape import TapeRefused

    lib = FakeLibrary()
    foreign = sorted([(0x300000, 0x300000 + 4096), (0xA00000, 0xA00000 + (1 << 20))])
    LayerTape(launches_of(lib, 0x100000, 0x800000), addresses(0x100000, 0x800000), foreign)      # all its own: fine
    odd = launches_of(lib, 0x100000, 0x800000)
    odd[0] = (lib, lib.entry, (c_int(3), c_void_p(0x9000), c_void_p(0x300000 + 128), c_void_p(0), c_float(1e-6)))
    with pytest.raises(TapeRefused, match="argument 2 .* another layer"):
        LayerTape(odd, addresses(0x100000, 0x800000), foreign)
    LayerTape(odd, addresses(0x100000, 0x800000))                                                # not asked to look
