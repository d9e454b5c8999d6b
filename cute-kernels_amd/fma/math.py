"""Integer helpers with the reference's names (fma/math.py:6-37)."""


def ceil_divide(x: int, y: int) -> int:
    return -(-x // y)


def divide_if_divisible(dividend: int, divisor: int, msg: str = "") -> int:
    assert dividend % divisor == 0, msg
    return dividend // divisor
