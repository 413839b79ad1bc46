"""Enumerations shared with callers (csrc/include/aiter_enum.h:16-26 of the reference)."""

import enum


class QuantType(enum.IntEnum):
    No = 0
    per_Tensor = 1
    per_Token = 2
    per_1x32 = 3
    per_1x128 = 4
    per_128x128 = 5
    per_256x128 = 6
    per_1024x128 = 7
