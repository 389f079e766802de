"""Constants and small helpers shared by the placement-evaluation path.

Mirrors the parts of the reference's ``alpa_serve/util.py`` that the simulator
and the placement search consume (constants :11-23, ``ServingCase`` :17-18,
partition helpers :74-161, ``write_tsv`` :55-71, ``to_str_round`` :88-106).
The Ray helpers of that file (:32-52) belong to the online serving runtime and
are not part of this package.
"""
from collections import namedtuple
from typing import Any, List, Sequence

import numpy as np

# Batch sizes the batching simulator may form (reference util.py:13).  It is a
# module-level list on purpose: experiments edit it in place.
batchsize_config = [1, 2, 4, 8, 16]

# (register_models, generate_workload, placement_policy) -- reference util.py:17-18.
ServingCase = namedtuple(
    "ServingCase", ("register_models", "generate_workload", "placement_policy"))

GB = 1 << 30
eps = 1e-6
inf = 1e100          # finite in fp64, +inf once stored as fp32 (util.py:23)

FIXED_OVERHEAD = 0.011   # simulator/controller.py:517,575,644
STAGE_PENALTY = 0.009    # per pipeline stage, simulator/controller.py:439,456,472


def get_factors(n: int) -> List[int]:
    """All positive divisors of ``n`` in ascending order (util.py:74-85)."""
    small, large = [], []
    d = 1
    while d * d <= n:
        if n % d == 0:
            small.append(d)
            if d != n // d:
                large.append(n // d)
        d += 1
    return small + large[::-1]


def is_valid_size(n: int, i: int) -> bool:
    """Admissible size ``i`` of the last part when splitting ``n`` devices
    into node-aligned pieces (util.py:109-113)."""
    return i <= n % 8 or (n - i) % 8 == 0 or n % 8 == 0


def get_partitions(n: int, k: int) -> List[List[int]]:
    """Ordered splits of ``n`` into ``k`` positive parts whose trailing parts
    satisfy :func:`is_valid_size` (util.py:117-126).  The enumeration order is
    part of the behaviour: the search breaks score ties by first occurrence."""
    if k == 1:
        return [[n]]
    out = []
    for last in range(1, n):
        if is_valid_size(n, last):
            out.extend(head + [last] for head in get_partitions(n - last, k - 1))
    return out


def get2tok(n: int) -> List[int]:
    """Powers of two not exceeding ``n`` (util.py:143-151)."""
    assert n > 0
    out = [1]
    while out[-1] * 2 <= n:
        out.append(out[-1] * 2)
    return out


def decompose2tok(n: int) -> List[int]:
    """Binary decomposition of ``n`` as ascending powers of two (util.py:154-162)."""
    return [1 << b for b in range(max(int(n), 0).bit_length()) if (n >> b) & 1]


def to_str_round(x: Any, decimal: int = 6) -> str:
    """Render nested containers with floats rounded (util.py:88-106)."""
    if x is None or isinstance(x, str):
        return str(x)
    if isinstance(x, dict):
        return str({k: to_str_round(v, decimal) for k, v in x.items()})
    if isinstance(x, (list, tuple, np.ndarray)):
        return "[" + ", ".join(to_str_round(y, decimal) for y in x) + "]"
    if isinstance(x, (bool, int, np.integer)):
        return str(x)
    if isinstance(x, (float, np.floating)):
        return f"{x:.{decimal}f}"
    raise ValueError("Invalid value: " + str(x))


def write_tsv(heads: Sequence[str], values: Sequence[Any], filename: str,
              print_line: bool = True) -> None:
    """Append one tab-separated row (util.py:55-71)."""
    assert len(heads) == len(values)
    cells = [str(v) for v in values]
    with open(filename, "a", encoding="utf-8") as fout:
        fout.write("\t".join(cells) + "\n")
    if print_line:
        print("".join(f"{h}: {c}  " for h, c in zip(heads, cells)))
