"""Small helpers shared by the schedule search (counterpart of reference python/ios/utils.py:4-24)."""
from typing import Iterator, List, Sequence


def seqeq(seq1: Sequence, seq2: Sequence) -> bool:
    """True when the two sequences agree on their common prefix (zip semantics)."""
    return all(a == b for a, b in zip(seq1, seq2))


def iter_subset(s: int, include_emtpy_set=False) -> Iterator[int]:
    """All non-empty sub-masks of the bit mask ``s`` in decreasing numeric order, optionally followed by 0."""
    sub = s
    while sub:
        yield sub
        sub = (sub - 1) & s
    if include_emtpy_set:
        yield 0


def bits_of(mask: int) -> List[int]:
    """Indices of the set bits of ``mask`` in increasing order."""
    out = []
    index = 0
    while mask:
        if mask & 1:
            out.append(index)
        mask >>= 1
        index += 1
    return out


def mask_of(indices) -> int:
    mask = 0
    for i in indices:
        mask |= 1 << i
    return mask
