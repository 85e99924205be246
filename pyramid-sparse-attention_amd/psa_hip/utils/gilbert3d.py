"""Generalised Hilbert ("gilbert") space-filling curve over an arbitrary W x H x D box.

Own iterative implementation of the published algorithm of Jakub Cerveny (github.com/jakubcerveny/gilbert,
BSD-2-Clause), which the reference vendors (reference: src/psa_triton/utils/gilbert3d.py:6-167).  The box is
described by three axis vectors a, b, c; a box is either emitted as a straight line or split into two to
five sub-boxes whose axes are permuted / reversed so that consecutive sub-boxes touch.
"""
from typing import Iterator, List, Tuple

Vec = Tuple[int, int, int]


def _sgn(v: int) -> int:
    return (v > 0) - (v < 0)


def _add(*vs: Vec) -> Vec:
    return (sum(v[0] for v in vs), sum(v[1] for v in vs), sum(v[2] for v in vs))


def _neg(v: Vec) -> Vec:
    return (-v[0], -v[1], -v[2])


def _sub(u: Vec, v: Vec) -> Vec:
    return (u[0] - v[0], u[1] - v[1], u[2] - v[2])


def _half(v: Vec) -> Vec:
    return (v[0] // 2, v[1] // 2, v[2] // 2)  # floor division, as in the published algorithm


def _len(v: Vec) -> int:
    return abs(v[0] + v[1] + v[2])


def _unit(v: Vec) -> Vec:
    return (_sgn(v[0]), _sgn(v[1]), _sgn(v[2]))


def gilbert3d(width: int, height: int, depth: int) -> Iterator[Vec]:
    """Yields (x, y, z) for every cell of the box exactly once, along the curve."""
    if width >= height and width >= depth:
        root = ((0, 0, 0), (width, 0, 0), (0, height, 0), (0, 0, depth))
    elif height >= width and height >= depth:
        root = ((0, 0, 0), (0, height, 0), (width, 0, 0), (0, 0, depth))
    else:
        root = ((0, 0, 0), (0, 0, depth), (width, 0, 0), (0, height, 0))
    stack: List[Tuple[Vec, Vec, Vec, Vec]] = [root]
    while stack:
        p, a, b, c = stack.pop()
        w, h, d = _len(a), _len(b), _len(c)
        da, db, dc = _unit(a), _unit(b), _unit(c)
        line = da if (h == 1 and d == 1) else db if (w == 1 and d == 1) else dc if (w == 1 and h == 1) else None
        if line is not None:
            n = w if line is da else h if line is db else d
            x, y, z = p
            for _ in range(n):
                yield (x, y, z)
                x, y, z = x + line[0], y + line[1], z + line[2]
            continue
        a2, b2, c2 = _half(a), _half(b), _half(c)
        # prefer even steps
        if _len(a2) % 2 and w > 2:
            a2 = _add(a2, da)
        if _len(b2) % 2 and h > 2:
            b2 = _add(b2, db)
        if _len(c2) % 2 and d > 2:
            c2 = _add(c2, dc)
        if 2 * w > 3 * h and 2 * w > 3 * d:  # long box: halve along a only
            parts = [
                (p, a2, b, c),
                (_add(p, a2), _sub(a, a2), b, c),
            ]
        elif 3 * h > 4 * d:  # flat in c: do not split c
            parts = [
                (p, b2, c, a2),
                (_add(p, b2), a, _sub(b, b2), c),
                (_add(p, _sub(a, da), _sub(b2, db)), _neg(b2), c, _neg(_sub(a, a2))),
            ]
        elif 3 * d > 4 * h:  # flat in b: do not split b
            parts = [
                (p, c2, a2, b),
                (_add(p, c2), a, b, _sub(c, c2)),
                (_add(p, _sub(a, da), _sub(c2, dc)), _neg(c2), _neg(_sub(a, a2)), b),
            ]
        else:  # split along all three axes
            parts = [
                (p, b2, c2, a2),
                (_add(p, b2), c, a2, _sub(b, b2)),
                (_add(p, _sub(b2, db), _sub(c, dc)), a, _neg(b2), _neg(_sub(c, c2))),
                (_add(p, _sub(a, da), b2, _sub(c, dc)), _neg(c), _neg(_sub(a, a2)), _sub(b, b2)),
                (_add(p, _sub(a, da), _sub(b2, db)), _neg(b2), c2, _neg(_sub(a, a2))),
            ]
        stack.extend(reversed(parts))
