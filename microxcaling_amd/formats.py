"""Element formats and rounding modes; same names and values as the reference's mx/formats.py."""
from enum import Enum, IntEnum

FP32_EXPONENT_BIAS = 127
FP32_MIN_NORMAL = 2 ** (-FP32_EXPONENT_BIAS + 1)


class RoundingMode(IntEnum):
    """The integer value is what crosses the native boundary (mx/formats.py:12-19)."""
    nearest = 0
    floor = 1
    even = 2

    @staticmethod
    def string_enums():
        return list(_ROUNDING_NAMES)


_ROUNDING_NAMES = tuple(m.name for m in RoundingMode)
ROUNDING_VALUES = {m.name: int(m) for m in RoundingMode}          # name -> what crosses the native boundary


class ElemFormat(Enum):
    """mx/formats.py:22-44; aliases share a value."""
    int8 = 1
    int4 = 2
    int2 = 3
    fp8_e5m2 = 4
    fp8_e4m3 = 5
    fp6_e3m2 = 6
    fp6_e2m3 = 7
    fp4 = 8
    fp4_e2m1 = 8
    float16 = 9
    fp16 = 9
    bfloat16 = 10
    bf16 = 10

    @staticmethod
    def from_str(s):
        assert s is not None, "String elem_format == None"
        s = s.lower()
        if hasattr(ElemFormat, s):
            return getattr(ElemFormat, s)
        raise Exception("Undefined elem format", s)


# (exponent bits, bits of sign + implicit one + fraction, IEEE-style top exponent reserved?)
_LAYOUT = {
    ElemFormat.int8: (0, 8, False), ElemFormat.int4: (0, 4, False), ElemFormat.int2: (0, 2, False),
    ElemFormat.fp8_e5m2: (5, 4, True), ElemFormat.fp8_e4m3: (4, 5, False),
    ElemFormat.fp6_e3m2: (3, 4, False), ElemFormat.fp6_e2m3: (2, 5, False),
    ElemFormat.fp4: (2, 3, False),
    ElemFormat.float16: (5, 12, True), ElemFormat.bfloat16: (8, 9, True),
}


def _get_min_norm(ebits):
    """Smallest normal of a float format with `ebits` exponent bits; 0 for integers."""
    return 0 if ebits == 0 else 2 ** (2 - (2 ** (ebits - 1)))


def _get_max_norm(ebits, mbits):
    """Largest normal when the top exponent encodes Inf/NaN (mx/formats.py:53-57)."""
    assert ebits >= 5, "invalid for floats that don't define NaN"
    emax = 2 ** (ebits - 1) - 1
    return 2 ** emax * float(2 ** (mbits - 1) - 1) / 2 ** (mbits - 2)


_FORMAT_CACHE = {}


def _get_format_params(fmt):
    """(ebits, mbits, emax, max_norm, min_norm), as mx/formats.py:61-125."""
    if type(fmt) is str:
        hit = _FORMAT_CACHE.get(fmt)              # layers pass the same few names over and over
        if hit is not None:
            return hit
        _FORMAT_CACHE[fmt] = _get_format_params(ElemFormat.from_str(fmt))
        return _FORMAT_CACHE[fmt]
    if fmt in _FORMAT_CACHE:
        return _FORMAT_CACHE[fmt]
    if fmt not in _LAYOUT:
        raise Exception("Unknown element format %s" % fmt)
    ebits, mbits, ieee_like = _LAYOUT[fmt]
    if ebits == 0:
        emax = 0
    elif ieee_like:
        emax = 2 ** (ebits - 1) - 1
    else:
        emax = 2 ** (ebits - 1)
    if fmt == ElemFormat.fp8_e4m3:
        max_norm = 2 ** emax * 1.75        # the all-ones code is NaN
    else:
        max_norm = 2 ** emax * float(2 ** (mbits - 1) - 1) / 2 ** (mbits - 2)
    _FORMAT_CACHE[fmt] = (ebits, mbits, emax, max_norm, _get_min_norm(ebits))
    return _FORMAT_CACHE[fmt]
