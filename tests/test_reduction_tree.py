"""The transposing wave reduction of the 4..16-row GEMV against the plain DPP tree, symbolically.

coffin_amd/csrc/common.hpp sums the 64 lane chains of a unit with a fixed tree
(wave_sum_to_lane63: lanes l^1, l^2, quads, half rows, rows, halves); a batched row must have the
bits of the single-row call (reference contract: models/qwen35/batch.py:19-22), so
wave_sum_transposed -- which reduces 8, 16 or 32 values per lane together, each lane keeping half
of its values per level -- has to build exactly that tree for every value.  Here both are run on
symbols, with fp32 addition modelled as an unordered pair (it commutes bit for bit and does not
associate), the cross-lane moves modelled after the ISA (DPP quad_perm / row_half_mirror /
row_mirror / row_bcast, v_permlane16_swap, v_permlane32_swap).  The GPU parity tests check the
kernel itself; this pins the lane -> value map and the choice of halves it relies on.
"""
import pytest


def add(a, b):
    """fp32 addition on symbols: commutative, not associative."""
    return frozenset([a, b]) if a != b else ("dup", a)


def dpp(vals, ctrl):
    """What each lane reads through a DPP control: quad_perm [1,0,3,2] / [2,3,0,1],
    row_half_mirror, row_mirror."""
    out = [None] * 64
    for lane in range(64):
        row, j = lane // 16, lane % 16
        if ctrl == 0xB1:
            src = row * 16 + (j ^ 1)
        elif ctrl == 0x4E:
            src = row * 16 + (j ^ 2)
        elif ctrl == 0x141:
            src = row * 16 + (j & 8) + (7 - (j & 7))
        else:
            assert ctrl == 0x140
            src = row * 16 + (15 - j)
        out[lane] = vals[src]
    return out


def original(vals):
    """wave_sum_to_lane63 of one value: the total as lane 63 holds it."""
    v = list(vals)
    for ctrl in (0xB1, 0x4E, 0x141, 0x140):
        d = dpp(v, ctrl)
        v = [add(v[lane], d[lane]) for lane in range(64)]
    w = list(v)
    for lane in range(64):      # row_bcast15 into rows 1 and 3
        row = lane // 16
        if row in (1, 3):
            w[lane] = add(v[lane], v[(row - 1) * 16 + 15])
    v, w = w, list(w)
    for lane in range(32, 64):  # row_bcast31 into rows 2 and 3
        w[lane] = add(v[lane], v[31])
    return w[63]


def swap16(a, b):
    """v_permlane16_swap: odd rows of the first operand <-> even rows of the second."""
    na, nb = list(a), list(b)
    for lane in range(64):
        row, j = lane // 16, lane % 16
        if row % 2 == 1:
            na[lane] = b[(row - 1) * 16 + j]
            nb[(row - 1) * 16 + j] = a[lane]
    return na, nb


def swap32(a, b):
    """v_permlane32_swap: upper half of the first operand <-> lower half of the second."""
    na, nb = list(a), list(b)
    for lane in range(32, 64):
        na[lane] = b[lane - 32]
        nb[lane - 32] = a[lane]
    return na, nb


def level(vals, ctrl, half, upper):
    """One transposing level: pair sums of values i and i + half, a lane keeps one of the two."""
    out = []
    for i in range(half):
        dl, dh = dpp(vals[i], ctrl), dpp(vals[i + half], ctrl)
        lo = [add(vals[i][lane], dl[lane]) for lane in range(64)]
        hi = [add(vals[i + half][lane], dh[lane]) for lane in range(64)]
        out.append([hi[lane] if upper(lane) else lo[lane] for lane in range(64)])
    return out


def transposed(nv, vals):
    """wave_sum_transposed<nv>: what every lane ends with."""
    a1 = level(vals, 0xB1, nv // 2, lambda l: (l ^ (l >> 2)) & 1)
    a2 = level(a1, 0x4E, nv // 4, lambda l: ((l >> 1) ^ (l >> 2)) & 1)
    a3 = level(a2, 0x141, nv // 8, lambda l: ((l >> 2) ^ (l >> 3)) & 1)
    if nv == 8:
        d = dpp(a3[0], 0x140)
        t = [add(a3[0][lane], d[lane]) for lane in range(64)]
    else:
        a4 = level(a3, 0x140, nv // 16, lambda l: (l >> 3) & 1)
        if nv == 32:
            x, y = swap16(a4[0], a4[1])
            t = [add(x[lane], y[lane]) for lane in range(64)]
        else:
            t = a4[0]
    if nv != 32:
        x, y = swap16(t, t)
        t = [add(x[lane], y[lane]) for lane in range(64)]
    x, y = swap32(t, t)
    return [add(x[lane], y[lane]) for lane in range(64)]


def index(nv, lane):
    """wave_sum_transposed_index<nv>."""
    s1 = (lane ^ (lane >> 2)) & 1
    s2 = ((lane >> 1) ^ (lane >> 2)) & 1
    s3 = ((lane >> 2) ^ (lane >> 3)) & 1
    s4 = (lane >> 3) & 1
    s5 = (lane >> 4) & 1
    return {8: s1 * 4 + s2 * 2 + s3,
            16: s1 * 8 + s2 * 4 + s3 * 2 + s4,
            32: s1 * 16 + s2 * 8 + s3 * 4 + s4 * 2 + s5}[nv]


@pytest.mark.parametrize("nv", [8, 16, 32])
def test_transposing_reduction_builds_the_plain_tree(nv):
    vals = [[(i, lane) for lane in range(64)] for i in range(nv)]
    want = [original(vals[i]) for i in range(nv)]
    got = transposed(nv, vals)
    for lane in range(64):
        assert got[lane] == want[index(nv, lane)], (nv, lane)
    # the lanes that store cover every value exactly once
    assert sorted(index(nv, lane) for lane in range(nv)) == list(range(nv))


def test_a_different_choice_of_halves_is_caught():
    """Keeping halves by the plain lane bit at the quad level pairs lanes that hold different
    values at the next level: the model must tell the two apart."""
    nv = 8
    vals = [[(i, lane) for lane in range(64)] for i in range(nv)]
    a1 = level(vals, 0xB1, 4, lambda l: l & 1)          # plain bit 0 instead of b0 ^ b2
    a2 = level(a1, 0x4E, 2, lambda l: (l >> 1) & 1)
    a3 = level(a2, 0x141, 1, lambda l: (l >> 2) & 1)
    want = [original(vals[i]) for i in range(nv)]
    d = dpp(a3[0], 0x140)
    t = [add(a3[0][l], d[l]) for l in range(64)]
    x, y = swap16(t, t)
    t = [add(x[l], y[l]) for l in range(64)]
    x, y = swap32(t, t)
    got = [add(x[l], y[l]) for l in range(64)]
    assert any(got[lane] not in want for lane in range(64))
