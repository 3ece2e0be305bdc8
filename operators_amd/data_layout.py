"""ctypes image of the library's element-type descriptor.

`DataLayout` is a 4-byte bitfield passed by value to
`infiniopCreateTensorDescriptor` (C side: include/infiniop.h; reference:
include/data_type.h:4-46, Python mirror operatorspy/data_layout.py:5-26).
"""
import ctypes


class DataLayout(ctypes.LittleEndianStructure):
    _fields_ = [
        ("packed", ctypes.c_ushort, 8),
        ("sign", ctypes.c_ushort, 1),
        ("size", ctypes.c_ushort, 7),
        ("mantissa", ctypes.c_ushort, 8),
        ("exponent", ctypes.c_ushort, 8),
    ]

    def key(self):
        return (self.packed, self.sign, self.size, self.mantissa, self.exponent)

    def __eq__(self, other):
        return isinstance(other, DataLayout) and self.key() == other.key()

    def __hash__(self):
        return hash(self.key())

    def __repr__(self):
        return _NAMES.get(self.key(), f"DataLayout{self.key()}")


_TABLE = {
    "I8": (1, 1, 1, 7, 0),
    "I16": (1, 1, 2, 15, 0),
    "I32": (1, 1, 4, 31, 0),
    "I64": (1, 1, 8, 63, 0),
    "U8": (1, 0, 1, 8, 0),
    "U16": (1, 0, 2, 16, 0),
    "U32": (1, 0, 4, 32, 0),
    "U64": (1, 0, 8, 64, 0),
    "F16": (1, 1, 2, 10, 5),
    "BF16": (1, 1, 2, 7, 8),
    "F32": (1, 1, 4, 23, 8),
    "F64": (1, 1, 8, 52, 11),
}
_NAMES = {v: k for k, v in _TABLE.items()}

I8 = DataLayout(*_TABLE["I8"])
I16 = DataLayout(*_TABLE["I16"])
I32 = DataLayout(*_TABLE["I32"])
I64 = DataLayout(*_TABLE["I64"])
U8 = DataLayout(*_TABLE["U8"])
U16 = DataLayout(*_TABLE["U16"])
U32 = DataLayout(*_TABLE["U32"])
U64 = DataLayout(*_TABLE["U64"])
F16 = DataLayout(*_TABLE["F16"])
BF16 = DataLayout(*_TABLE["BF16"])
F32 = DataLayout(*_TABLE["F32"])
F64 = DataLayout(*_TABLE["F64"])

__all__ = ["DataLayout"] + list(_TABLE)
