import math


def nearest_power_of_two(x: int, round_up: bool = False) -> int:
    """Largest power of two <= x, or smallest >= x with round_up
    (reference: flash_stu/utils/numerics.py:3-6)."""
    e = math.log2(x)
    return 1 << (math.ceil(e) if round_up else math.floor(e))
