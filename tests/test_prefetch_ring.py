"""CPU: the hand-counted waits of the chunked wkv5 / wkv6 kernels' input prefetch.

The prep waves of wkv6_fwd.hip, wkv6_bwd_a.hip and wkv6_bwd_b.hip load their inputs through inline asm into a ring of
register sets, several chunks ahead, and wait with `s_waitcnt vmcnt(younger * NLOADS)`: vector-memory operations
complete in order, so "at most n outstanding" means "all but the n youngest have landed".  That is right only if
  * NLOADS is the number of loads one `prefetch` call issues, in every decay mode,
  * `younger` is the number of `prefetch` calls issued after the one whose data is about to be read,
  * the ring slot read in an iteration holds the chunk that iteration expects,
  * the compiler adds no vector-memory operation of its own to those waves' loops (a spill would do that).
The first three are checked on the source text with a small model of the schedule, the last on the ISA that hipcc emits
(`-S`, cross-compiled, no GPU needed)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "rwkv_cuda_amd", "csrc")
MODES = {"W_HEAD": 0, "W_EW": 1, "W_RAW": 2}
KERNELS = {
    # file: (prefetch-depth constant, how the ring size follows from it per mode, extra loads per token beyond r k v)
    "wkv6_fwd.hip": "STAGES",
    "wkv6_bwd_a.hip": "STA",
    "wkv6_bwd_b.hip": "STB",
}


def _read(name):
    with open(os.path.join(CSRC, name)) as f:
        return f.read()


def _const(text, name):
    m = re.search(r"constexpr int %s = (\d+);" % name, text) or re.search(r"constexpr int %s = (\d+);" % name, _read("wkv6_chunk.h"))
    assert m, name
    return int(m.group(1))


def _lambda_body(text, name):
    """Source of `auto NAME = [&](...) ... { ... };` (brace matched)."""
    start = text.index("auto %s = [&]" % name)
    i = text.index("{", start)
    depth, j = 0, i
    while True:
        depth += {"{": 1, "}": -1}.get(text[j], 0)
        if depth == 0:
            return text[i:j + 1]
        j += 1


def _loads_per_call(body, mode):
    """Loads one prefetch call issues in `mode`: asm loads outside any `if constexpr`, plus those of the matching branch,
    times the trip count of the token loop they sit in."""
    trip = int(re.search(r"for \(int e = 0; e < (\d+); \+\+e\)", body).group(1))
    n = 0
    # split the loop body into the unconditional part and the `if constexpr (WMODE == X)` branches
    branches = list(re.finditer(r"if constexpr \(WMODE == (W_\w+)\) \{(.*?)\}", body, re.S))
    uncond = body
    for b in branches:
        uncond = uncond.replace(b.group(0), "")
    n += len(re.findall(r'asm volatile\("global_load_', uncond))
    for b in branches:
        if b.group(1) == mode:
            n += len(re.findall(r'asm volatile\("global_load_', b.group(2)))
    return n * trip


def _nloads_expr(text, mode):
    m = re.search(r"constexpr int NLOADS = WMODE == W_HEAD \? (\d+) : (\d+);", text)
    assert m
    return int(m.group(1)) if mode == "W_HEAD" else int(m.group(2))


def _ring_size(text, depth_name, mode):
    depth = _const(text, depth_name)
    m = re.search(r"constexpr int NST = WMODE == W_EW \? %s - 1 : %s;" % (depth_name, depth_name), text)
    if m:
        return depth - 1 if mode == "W_EW" else depth
    return depth


def _schedule(text, ring_name):
    """(arrived slot offset, younger expression, prefetch slot offset, prefetch chunk offset) of the main loop."""
    R = ring_name
    a = re.search(r"arrived\(ring\[\(z \+ (\d+)\) % " + R + r"\], std::integral_constant<int, " + R + r" - (\d+)>\{\}\);", text)
    p = re.search(r"prefetch\(i \+ (\d+) \+ " + R + r", ring\[\(z \+ (\d+)\) % " + R + r"\]\);", text)
    pro = re.search(r"prefetch\(%s, ring\[0\]\);" % ring_name, text)
    first = re.search(r"static_for<%s>\(\[&\]\(auto Z\) \{ prefetch\(decltype\(Z\)::value, ring\[decltype\(Z\)::value\]\); \}\);" % ring_name, text)
    wait0 = re.search(r"static_for<%s>\(\[&\]\(auto Z\) \{ arrived\(ring\[decltype\(Z\)::value\], std::integral_constant<int, 0>\{\}\); \}\);" % ring_name, text)
    assert a and p and pro and first and wait0, "the prefetch schedule no longer has the shape this test models"
    return int(a.group(1)), int(a.group(2)), int(p.group(2)), int(p.group(1))


@pytest.mark.parametrize("fname", sorted(KERNELS))
@pytest.mark.parametrize("mode", sorted(MODES))
def test_loads_per_prefetch_call_match_nloads(fname, mode):
    text = _read(fname)
    body = _lambda_body(text, "prefetch")
    assert _loads_per_call(body, mode) == _nloads_expr(text, mode), (fname, mode)
    # every wait names its count through the same constant
    waits = re.findall(r's_waitcnt vmcnt\(%\[n\]\)"[^;]*?\[n\] "n"\(([^)]*\)[^)]*)\)', text, re.S)
    assert waits, fname
    for w in waits:
        assert "decltype(younger)::value * NLOADS" in w, (fname, w)
    # and no wait in the prep role is written with a literal count
    dividers = [m.start() for m in re.finditer(r"^// -{20,}", text, re.M)]
    start = next(d for d in dividers if "prep waves" in text[d:text.index("\n", d)])
    prep = text[start:min(d for d in dividers if d > start)]
    assert not re.search(r"s_waitcnt vmcnt\(\d+\)", prep), fname


@pytest.mark.parametrize("fname", sorted(KERNELS))
@pytest.mark.parametrize("mode", sorted(MODES))
@pytest.mark.parametrize("nchunks", [1, 2, 3, 4, 5, 7, 12])
def test_younger_counts_and_slot_contents(fname, mode, nchunks):
    """Replays the order of prefetch / arrived calls of the prep waves and checks every wait against the model."""
    text = _read(fname)
    depth_name = KERNELS[fname]
    ring_name = "NST" if re.search(r"constexpr int NST =", text) else depth_name
    n = _ring_size(text, depth_name, mode)
    arr_off, younger_sub, pre_off, pre_chunk = _schedule(text, ring_name)
    assert n >= 3, "the loop reads slot z+1 and waits for slot z+2: the ring needs three slots"

    issued = []                 # program order of prefetch calls: (slot, chunk)
    landed = {}                 # slot -> index into `issued` of the newest prefetch known to have landed
    held = {}                   # slot -> chunk of its newest prefetch

    def prefetch(chunk, slot):
        issued.append((slot, min(chunk, nchunks - 1)))
        held[slot] = min(chunk, nchunks - 1)

    def arrived(slot, younger):
        idx = max(i for i, (s, _) in enumerate(issued) if s == slot)
        after = len(issued) - 1 - idx
        # in-order completion: waiting for "at most `younger` calls outstanding" covers this slot iff no more than
        # `younger` calls were issued after it; fewer would wait for data that is not needed yet
        assert after == younger, (fname, mode, nchunks, slot, after, younger)
        landed[slot] = idx

    def use(slot, chunk):
        idx = max(i for i, (s, _) in enumerate(issued) if s == slot)
        assert landed.get(slot) == idx, ("read before its wait", fname, mode, slot, chunk)
        assert held[slot] == chunk, ("slot holds another chunk", fname, mode, slot, held[slot], chunk)

    for z in range(n):
        prefetch(z, z)
    for z in range(n):
        landed[z] = z                          # the prologue waits with vmcnt(0): everything issued so far has landed
    use(0, 0)                                  # scan(0), operands(0)
    if nchunks > 1:
        use(1, min(1, nchunks - 1))            # scan(1)
    prefetch(n, 0)
    for i in range(nchunks):
        z = i % n
        arrived((z + arr_off) % n, n - younger_sub)
        if i + 2 < nchunks:
            use((z + arr_off) % n, i + 2)      # scan(i + 2)
        if i + 1 < nchunks:
            use((z + 1) % n, i + 1)            # operands(i + 1)
        prefetch(i + pre_chunk + n, (z + pre_off) % n)


def _isa(fname):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument", "-I", os.path.join(ROOT, "include"), "-I", CSRC,
           "-S", "--cuda-device-only", "-o", "-", os.path.join(CSRC, fname)]
    return subprocess.run(cmd, check=True, capture_output=True, text=True).stdout


def _kernels(asm):
    """name -> instruction lines (with labels) of each kernel in the listing."""
    out, cur = {}, None
    for line in asm.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            cur = out.setdefault(m.group(1), [])
            continue
        if cur is not None:
            if line.strip().startswith(".Lfunc_end"):
                cur = None
            else:
                cur.append(line.strip())
    return out


@pytest.mark.parametrize("fname", sorted(KERNELS))
def test_no_compiler_vmem_inside_the_prefetching_loops(fname):
    """A register spilled inside the prep waves' loop would put scratch loads and stores (counted by vmcnt like any
    other vector-memory operation) between a prefetch and its wait, and a spilled ring register would be saved before
    its load has landed.  The build tolerates a few spilled registers in sweep B (values of the state waves, saved
    before the roles part and reloaded by compiler-generated code with compiler-generated waits); none may sit in a
    loop that holds a hand-counted wait."""
    text = _read(fname)
    depth_name = KERNELS[fname]
    ring_name = "NST" if re.search(r"constexpr int NST =", text) else depth_name
    _, younger_sub, _, _ = _schedule(text, ring_name)
    for name, lines in _kernels(_isa(fname)).items():
        mode = next(m for m, v in MODES.items() if "ILi%dE" % v in name)
        want = (_ring_size(text, depth_name, mode) - younger_sub) * _nloads_expr(text, mode)
        wait = "s_waitcnt vmcnt(%d)" % want
        labels = {}
        for i, l in enumerate(lines):
            m = re.match(r"^(\.LBB\d+_\d+):", l)
            if m:
                labels[m.group(1)] = i
        loops = []
        for i, l in enumerate(lines):
            m = re.match(r"^s_c?branch\w*\s+(\.LBB\d+_\d+)", l)
            if m and labels.get(m.group(1), len(lines)) <= i:
                loops.append((labels[m.group(1)], i))
        prefetching = [(a, b) for a, b in loops if any(l == wait for l in lines[a:b + 1])]
        # the hand-counted wait survives into the ISA with the count the model expects, inside a loop
        assert prefetching, (name, wait)
        for a, b in prefetching:
            bad = [l for l in lines[a:b + 1] if l.startswith("scratch_")]
            assert not bad, (name, bad)



def _lambdas_over_raw(text):
    """name -> body of every lambda of the prep role that takes a ring slot (`Raw& x`)."""
    out = {}
    for m in re.finditer(r"auto (\w+) = \[&\]\([^)]*Raw& x[^)]*\)", text):
        out[m.group(1)] = _lambda_body(text, m.group(1))
    return out


@pytest.mark.parametrize("fname", sorted(KERNELS))
def test_ring_registers_are_only_touched_by_their_loads_their_wait_and_their_readers(fname):
    """The compiler takes the outputs of the asm loads as defined right after the asm statement: C++ that reads, copies or
    assigns a loaded field of a ring slot between its `prefetch` and its `arrived` would touch a register whose load has
    not landed, and neither the spill count nor the scratch scan would see the move.  On the source text:
      * `prefetch` and `arrived` name the loaded fields inside asm statements only (outputs of the loads, "+v" operands of
        the wait) and nothing else of a slot;
      * the only other code that sees a slot are the reader lambdas scan / operands_a / operands_b, and the ring is never
        copied, assigned or indexed outside calls of these five;
      * in the main loop a slot is waited for before its first reader and reloaded after its last one (which slot that
        is, and that the wait's count covers it, is the business of test_younger_counts_and_slot_contents)."""
    text = _read(fname)
    lam = _lambdas_over_raw(text)
    assert set(lam) == {"prefetch", "arrived", "scan", "operands_a", "operands_b"}, sorted(lam)
    loaded = set(re.findall(r'"=&v"\(x\.(\w+)\[', lam["prefetch"]))
    assert {"r", "k", "v"} <= loaded, loaded
    fields = set(re.search(r"struct Raw \{(.*?)\};", text, re.S).group(1).replace("[", " ").replace(";", " ").replace(",", " ").split())
    assert loaded <= fields
    for name in ("prefetch", "arrived"):
        body = lam[name]
        outside_asm = re.sub(r"asm volatile\(.*?\);", "", body, flags=re.S)
        assert not re.search(r"\bx\.", outside_asm), (fname, name, "a slot is touched outside the asm statements")
        for stmt in re.findall(r"asm volatile\((.*?)\);", body, re.S):
            named = set(re.findall(r"x\.(\w+)", stmt))
            assert named <= loaded, (fname, name, named - loaded)
    # the wait names every loaded field of the mode it is compiled for ("+v": the compiler must treat them as redefined there)
    for stmt in re.findall(r"asm volatile\((.*?)\);", lam["arrived"], re.S):
        assert set(re.findall(r'"\+v"\(x\.(\w+)', stmt)) >= {"r", "k", "v"}, (fname, stmt)
    # nobody else sees the ring
    start = text.index("Raw ring[")
    role_end = text.index("// ----------", start)
    role = text[start:role_end]
    for m in re.finditer(r"ring\[", role):
        if role[m.start() - 4:m.start()] == "Raw ":
            continue
        stmt_start = max(role.rfind(";", 0, m.start()), role.rfind("{", 0, m.start()), role.rfind("}", 0, m.start())) + 1
        stmt = role[stmt_start:role.index(";", m.start())]
        assert re.search(r"\b(prefetch|arrived|scan|operands_a|operands_b)\(", stmt), (fname, stmt.strip())
        assert not re.search(r"(^|[^=!<>])=[^=]", re.sub(r"\([^()]*\)", "", stmt).replace("exact_cur =", "").replace("exact_next =", "").replace("bool exact_cur", "").replace("bool exact_next", "")) \
            or re.search(r"exact_(cur|next) = operands_a\(", stmt), (fname, stmt.strip())
    assert not re.search(r"\bRaw\s+\w+\s*(=|\{|\()", role.replace("Raw ring[", "")), fname
    # order inside one iteration of the main loop
    loop = role[role.index("static_for<", role.index("for (int ib = 0")):]
    at = {k: loop.index(k) for k in ("arrived(ring[(z + 2)", "scan(i + 2, ring[(z + 2)", "operands_a(i + 1, ring[(z + 1)", "operands_b(i + 1, ring[(z + 1)", "prefetch(i + 1 +")}
    assert at["arrived(ring[(z + 2)"] < at["scan(i + 2, ring[(z + 2)"], fname                 # slot z + 2: waited for, then read
    assert max(at["operands_a(i + 1, ring[(z + 1)"], at["operands_b(i + 1, ring[(z + 1)"]) < at["prefetch(i + 1 +"], fname   # slot z + 1: read, then reloaded
    assert re.search(r"prefetch\(i \+ 1 \+ \w+, ring\[\(z \+ 1\)", loop), fname


@pytest.mark.parametrize("fname", ["wkv6_fwd_f.hip", "wkv6_bwd_f.hip"])
def test_one_sweep_kernels_leave_the_waits_to_the_compiler(fname):
    """The one-sweep kernels prefetch with ordinary loads into ordinary variables: the compiler knows which registers are in
    flight and places the waits itself, so there is no hand-counted wait to get wrong and no move it could place ahead of
    one.  What they owe the compiler instead is a loop in which every stage runs in every iteration (its wait counts are
    taken over all the ways into a wait): the prefetch, the staging and the stores sit outside any `if` of the prep loop
    that depends on the iteration."""
    text = _read(fname)
    assert "asm volatile(\"global_load" not in text and "buffer_load" not in text
    assert not re.search(r"s_waitcnt vmcnt", re.sub(r"//.*", "", text))
    m = re.search(r"for \(int it0 = 0; it0 < nit; it0 \+= (DEPTH|TRIP)\)", text)
    start = m.start()
    if m.group(1) == "TRIP":
        # a trip of the loop is a whole number of turns of the prefetch ring and of the registers kept for the finishing:
        # both are indexed by compile-time constants, so nothing in flight is ever copied
        depth, kept, trip = (int(re.search(rf"constexpr int {n} = (\d+);", text).group(1)) for n in ("DEPTH", "KEPT", "TRIP"))
        assert trip % depth == 0 and trip % kept == 0
        assert "static_for<TRIP>" in text and "% DEPTH" in text and "% KEPT" in text
    loop = text[start:text.index("__syncthreads();", start)]
    for call in re.findall(r"^\s*(?:if [^\n]*\))?\s*(fetch|stage_in)\(", loop, re.M):
        pass
    # fetch is unconditional; stage_in only chooses between its two forms
    assert re.search(r"^\s+fetch\(", loop, re.M), fname
    assert not re.search(r"if \([^\n]*\)\s*fetch\(", loop), fname
    assert re.search(r"stage_in\([^;]*part\); else stage_in\([^;]*full\);", loop), fname
