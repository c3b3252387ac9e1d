"""Integer helpers of the PSH layer (reference: flash3dxfmr/psh/arithmatic.py:12-29; the module keeps
the reference's spelling so imports read the same)."""


def round_next_two_power(v: int) -> int:
    """Smallest power of two >= v for v >= 1; 0 for v == 0 (the bit-smearing of the reference maps
    0 -> 0, which callers must treat as "cloud smaller than one bucket")."""
    if v <= 0:
        return 0
    return 1 << (int(v) - 1).bit_length()


def round_next_multiply(v, base):
    return type(v)(cdiv(v, base) * base)


def cdiv(a, b) -> int:
    a, b = int(a), int(b)
    return -(-a // b)
