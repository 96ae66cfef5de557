"""CPU: the LDS layout of the depthwise_conv1d kernels that use two-term fp16 products (csrc/timex.hip).

Those kernels fill most of the 160 KiB of LDS and read the Toeplitz operand through two shifted copies of a
line, one element past the last tap being a legal read.  The constants are taken from the source text and the index
ranges are walked for every T the kernels accept: every read and write must stay inside its array, every multi-byte
access must be aligned as the instruction needs, and the window a lane reads must be the taps the product needs."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = open(os.path.join(ROOT, "rwkv_cuda_amd", "csrc", "timex.hip")).read()
LDS_BYTES = 160 * 1024


def _const(name):
    m = re.search(r"constexpr int %s = (\d+);" % name, SRC)
    assert m, name
    return int(m.group(1))


def _affine(fn):
    """`return T + c;` of a one-line helper."""
    m = re.search(r"inline int %s\(int T\) \{ return T \+ (\d+); \}" % fn, SRC)
    assert m, fn
    return int(m.group(1))


T_MAX3 = _const("T_H2_MAX")
MROWS = _const("MROWS")
GH2_ROWS = _const("GH2_ROWS")
ROW_PAD = _affine("h2_row_stride")
_m = re.search(r"inline int h2_line_len\(int T\) \{ return T \+ \(\(T & 32\) \? (\d+) : (\d+)\); \}", SRC)
assert _m, "h2_line_len"


def line_len(T):
    return T + (int(_m.group(1)) if T & 32 else int(_m.group(2)))


TS = [t for t in range(32, T_MAX3 + 1, 32)]


@pytest.mark.parametrize("T", TS)
def test_conv_planes_fit_and_are_aligned(T):
    rs, xl = T + ROW_PAD, line_len(T)
    total = (2 * MROWS * rs + 4 * xl) * 2 + 16 * 4            # two planes of rows, two planes x two copies of the line, the maxima
    assert total <= LDS_BYTES, (T, total)
    assert ((2 * MROWS * rs + 4 * xl) * 2) % 4 == 0            # the maxima are floats
    assert (rs * 2) % 16 == 0                       # a lane's eight slots of a row: one aligned 16-byte read
    assert (2 * MROWS * rs * 2) % 4 == 0 and (xl * 2) % 4 == 0     # the line copies start on dwords
    # the second copy sits 16 banks (of 4 bytes) away from the first, modulo 32 banks
    assert (xl // 2) % 32 == 16


@pytest.mark.parametrize("T", [32, 64, 96, 384, 736, 768, 992, 1024])
@pytest.mark.parametrize("mirror", [False, True])
def test_conv_tap_windows(T, mirror):
    """line[] as the kernel fills it, the two copies, and the window of every (output tile, input tile, lane, K block)."""
    nt, xl = T // 32, line_len(T)
    w = [1000 + tau for tau in range(T)]            # tap tau of the kernel row (w[c][tau]); 0 stands for "no tap"
    line = [0] * xl
    for tau in range(T):
        line[31 + (T - 1 - tau) if mirror else tau] = w[tau]
    copy = [list(line), line[1:] + [0]]
    for ot in range(nt):
        n_in = nt - ot if mirror else ot + 1
        for j2 in range(2 * n_in + 1):              # the step past the last one is fetched too (and never used)
            for ln in range(32):
                for kh in range(2):
                    start0 = (31 - ln if mirror else T - 1 - 32 * ot - ln) + 8 * kh
                    start = start0 + 16 * j2
                    e, dw = start & 1, (start >> 1)
                    assert 0 <= 2 * dw and 2 * dw + 7 < xl, (T, mirror, ot, j2, ln, kh)
                    got = copy[e][2 * dw:2 * dw + 8]
                    if j2 == 2 * n_in:
                        continue
                    j, ks = j2 >> 1, j2 & 1
                    it = ot + j if mirror else j
                    for i in range(8):
                        slot = 16 * ks + 8 * kh + i
                        if mirror:                   # row u = 32 ot + ln, slot t = 32 it + slot: tap of lag t - u
                            lag = 32 * it + slot - (32 * ot + ln)
                        else:                        # row t = 32 ot + ln, slot u = 32 it + slot
                            lag = (32 * ot + ln) - (32 * it + slot)
                        want = w[T - 1 - lag] if 0 <= lag < T else 0
                        assert got[i] == want, (T, mirror, ot, j2, ln, kh, i)


_g = re.search(r"inline int gw_row_stride\(int T\) \{ return T \+ \(\((\d+) - \(T & 127\)\) & 127\); \}", SRC)
assert _g, "gw_row_stride"


def gw_row_stride(T):
    return T + ((int(_g.group(1)) - (T & 127)) & 127)


@pytest.mark.parametrize("T", TS)
def test_gradient_planes_fit(T):
    """Planes [2 tensors][2 terms][16 rows][T + pad] fp16, the diagonal sums, the maxima; 8-byte stores of a lane's four
    steps and the two transposing reads of an operand (rows 8 kh + (l16 >> 2) and four further on, 8 bytes at step
    32 tile + 16 (ln >> 4) + 4 (l16 & 3)) stay inside their plane and are aligned."""
    rsg = gw_row_stride(T)
    assert rsg >= T + 8
    plane = GH2_ROWS * rsg
    total = 4 * plane * 2 + (2 * T + 16) * 4
    assert total <= LDS_BYTES, (T, total)
    assert (rsg * 2) % 8 == 0 and (4 * plane * 2) % 4 == 0
    for tile in range(T // 32):
        for lane in range(64):
            ln, kh, l16 = lane & 31, lane >> 5, lane & 15
            for extra in (0, 4):
                row = 8 * kh + (l16 >> 2) + extra
                step = 32 * tile + 16 * (ln >> 4) + 4 * (l16 & 3)
                assert row < GH2_ROWS and step + 3 < T
                assert ((row * rsg + step) * 2) % 8 == 0
    # the sixteen 8-byte pieces that the 16 lanes of a group read at once fall on different banks (64 banks of 4 bytes)
    for kh in range(2):
        banks = set()
        for l16 in range(16):
            a = ((8 * kh + (l16 >> 2)) * rsg + 4 * (l16 & 3)) * 2
            banks.update({(a // 4) % 64, (a // 4 + 1) % 64})
        assert len(banks) == 32, (T, kh)
    # a lane's eight K slots are the batch rows 8 kh .. 8 kh + 7 of step 32 tile + ln: the 16 lanes of a group ask for four
    # rows x 16 steps, and lane l16 gets step 16 (ln >> 4) + l16 of each
    for lane in range(64):
        ln, l16 = lane & 31, lane & 15
        assert 16 * (ln >> 4) + l16 == ln


def test_diagonal_sums_in_registers():
    """Lane p of a half-wave takes, for row t, the element of column (t - p) mod 32: diagonal p if t >= p, else p - 32;
    every element of the 32 x 32 tile is taken exactly once."""
    seen = set()
    for kh in range(2):
        for v in range(16):
            t = 8 * (v >> 2) + 4 * kh + (v & 3)
            for p in range(32):
                u = (t - p) & 31
                d = t - u
                assert d == (p if t >= p else p - 32)
                seen.add((t, u))
    assert len(seen) == 32 * 32
