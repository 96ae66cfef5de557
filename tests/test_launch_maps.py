"""CPU: two index maps that decide which workgroup computes what, checked as maps (bijections, exact covers) with the
expressions taken from the sources.

* wkv4: workgroups are renumbered so that the two that share every 128-byte line run on the same XCD (csrc/wkv4.hip,
  paired_workgroup).  Whatever the grid size, the renumbering must be a permutation of the workgroups.
* wkv5 at head size 128: every head runs as four heads of 64 in two launches; workgroup h of a launch takes its value
  channels from block h and its key channels from block h ^ cross (csrc/wkv6_fwd.hip and the two sweeps).  Every block
  (value half, key half) of every head must be computed exactly once, and every output block must receive exactly one
  term from each launch."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rwkv_cuda_amd", "csrc")


def test_wkv4_paired_workgroups_are_a_permutation():
    src = open(os.path.join(CSRC, "wkv4.hip")).read()
    m = re.search(r"DEVINL int paired_workgroup\(int launched, int n\) \{\s*return (.+?);\s*\}", src, re.S)
    assert m
    expr = m.group(1)                                # n % 16 == 0 ? (launched % 8) * (n / 8) + launched / 8 : launched
    cond, rest = expr.split("?")
    yes, no = rest.split(":")
    py = lambda e: e.replace("/", "//").strip()
    for n in list(range(1, 70)) + [96, 192, 256, 3072, 3088]:
        seen = set()
        for launched in range(n):
            env = {"launched": launched, "n": n}
            q = eval(py(yes), {}, env) if eval(py(cond), {}, env) else eval(py(no), {}, env)
            assert 0 <= q < n
            seen.add(q)
        assert len(seen) == n, n
        if n % 16 == 0:                              # neighbours in the new numbering were launched 8 apart: same XCD
            inv = {}
            for launched in range(n):
                inv[(launched % 8) * (n // 8) + launched // 8] = launched
            assert all(inv[q] % 8 == inv[q + 1] % 8 for q in range(0, n, 2))


def test_split_heads_cover_every_block_once():
    for f in ("wkv6_fwd.hip", "wkv6_bwd_a.hip", "wkv6_bwd_b.hip"):
        src = open(os.path.join(CSRC, f)).read()
        assert re.search(r"const int hk = (SPLIT( != 0)? \? )?h \^ a\.cross", src), f
    for H in (1, 2, 5):
        blocks = {}                                  # (head, value half, key half) -> launches that compute it
        for cross in (0, 1):
            for h in range(2 * H):                   # a launch treats the tensor as 2 H heads of 64
                hk = h ^ cross
                assert hk // 2 == h // 2             # both blocks belong to the same head of 128
                blocks.setdefault((h // 2, h % 2, hk % 2), []).append(cross)
        assert len(blocks) == 4 * H and all(len(v) == 1 for v in blocks.values())
        for head in range(H):
            for half in (0, 1):
                # outputs indexed by value channels (y, gv) and by key channels (gr, gk, gw, gu): one term per launch
                by_value = sorted(c for (hd, i, j), (c,) in ((k, tuple(v)) for k, v in blocks.items()) if hd == head and i == half)
                by_key = sorted(c for (hd, i, j), (c,) in ((k, tuple(v)) for k, v in blocks.items()) if hd == head and j == half)
                assert by_value == [0, 1] and by_key == [0, 1]
