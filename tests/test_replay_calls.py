"""The packing of recorded launches into slots, on the CPU: integers, negative integers,
addresses and floats land in 64-bit slots as the slot forms of the entry points read them
(csrc/slots.h), and an entry point without a slot form is refused."""

import ctypes
import struct
from ctypes import c_float, c_int, c_long, c_void_p

from tokamak_amd.kernels import ops


class FakeFn:
    def __init__(self, argtypes, slots_address=1234):
        self.argtypes = argtypes
        self.slots_address = slots_address


def test_arguments_become_slots():
    fn = FakeFn([c_int, c_void_p, c_void_p, c_long, c_float, c_int, c_void_p])
    args = (7, c_void_p(0x7F0012345678), c_void_p(0), -3, 0.125, c_int(-1), 0x1000)
    slots = ops.slots_of(fn, args)
    assert slots[0] == 7 and slots[1] == 0x7F0012345678 and slots[2] == 0
    assert slots[3] == (1 << 64) - 3                       # two's complement: the low 8 bytes are a long -3
    assert slots[4] == struct.unpack("<I", struct.pack("<f", 0.125))[0]
    assert slots[5] & 0xFFFFFFFF == 0xFFFFFFFF             # the low 4 bytes are an int -1
    assert slots[6] == 0x1000
    # what the slot form does with them: the low bytes, reinterpreted
    low4 = struct.pack("<Q", slots[5])[:4]
    assert struct.unpack("<i", low4)[0] == -1
    assert struct.unpack("<f", struct.pack("<Q", slots[4])[:4])[0] == 0.125
    assert ctypes.c_long(slots[3]).value == -3


def test_an_entry_point_without_a_slot_form_is_not_packed():
    assert ops.slots_of(FakeFn([c_int], slots_address=None), (1,)) is None
    assert ops.slots_of(FakeFn([c_int, c_int]), (1,)) is None          # arguments and signature disagree


def test_a_recording_with_such_a_call_falls_back_to_call_by_call():
    from tokamak_amd.engine.layer_replay import PackedCalls

    good = FakeFn([c_int, c_void_p])
    bad = FakeFn([c_int], slots_address=None)
    packed = PackedCalls([(good, (1, c_void_p(64)), ((1, ("part", "mixer", "w"), 16),), 0), (good, (2, c_void_p(0)), (), 0)])
    assert packed.ok and packed.keys == [("part", "mixer", "w")]
    assert packed.first.tolist() == [0, 2] and packed.slots.tolist() == [1, 64, 2, 0]
    assert packed.patch_slot.tolist() == [1] and packed.patch_key.tolist() == [0] and packed.patch_offset.tolist() == [16]
    assert not PackedCalls([(good, (1, c_void_p(64)), (), 0), (bad, (1,), (), 0)]).ok
