"""Small integer helpers (same names and contracts as cute_kernels/math.py:1-35)."""


def ceil_divide(x: int, y: int) -> int:
    return -(-x // y)


def check_power_of_2(n: int) -> bool:
    return n > 0 and (n & (n - 1)) == 0


def get_powers_of_2(start: int, end: int) -> list[int]:
    assert check_power_of_2(start), "start is not a power of 2"
    assert check_power_of_2(end), "end is not a power of 2"
    return [1 << s for s in range(start.bit_length() - 1, end.bit_length())]


def divide_if_divisible(dividend: int, divisor: int, msg: str = "") -> int:
    assert dividend % divisor == 0, msg
    return dividend // divisor


_MAX_POWER_OF_2 = 65536


def get_next_power_of_2(x: int) -> int:
    if x > _MAX_POWER_OF_2:
        raise ValueError(f"x ({x}) is bigger than the max allowable power of 2 ({_MAX_POWER_OF_2})")
    return 1 if x <= 1 else 1 << (x - 1).bit_length()
