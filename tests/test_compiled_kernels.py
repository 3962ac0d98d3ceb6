"""Checks of the compiled gfx950 assembly of the attention kernels (hipcc cross-compiles without a GPU).

The counted waits of the streaming kernels (tests/test_counted_waits.py models them) are only right while a step of
their loops issues exactly the vector memory operations the count was made from: no register spill to scratch, no
split store, no load the compiler added.  And the LDS-direct loads write M0 from inline assembly without being able
to name it as a clobber, which is only safe while nothing else in the kernels uses M0.  Both are properties of the
compiler's output, so they are checked there."""
import importlib.util
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from tile_index_lib import BUILD, ROOT, lib

CSRC = os.path.join(ROOT, "sf-bert_amd", "csrc")
FILES = ["unfused_attention.hip", "fused_attention.hip", "fused_backward.hip"]
VMEM = re.compile(r"^\s+(global_|buffer_|scratch_|flat_)(\w+)")


def _device_flags():
    spec = importlib.util.spec_from_file_location("sfb_build_flags", os.path.join(ROOT, "sf-bert_amd", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.HIPCC, mod.DEVICE_FLAGS


def _assemble(name):
    """csrc/<name> -> assembly text of its device code (cached until a source changes)."""
    hipcc, flags = _device_flags()
    out = os.path.join(BUILD, name + ".s")
    sources = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))]
    sources.append(os.path.join(ROOT, "include", "sfbert_hip.h"))
    if not os.path.exists(out) or os.path.getmtime(out) < max(os.path.getmtime(s) for s in sources):
        os.makedirs(BUILD, exist_ok=True)
        subprocess.run([hipcc] + flags + ["-x", "hip", "--cuda-device-only", "-S", "-o", out, os.path.join(CSRC, name)],
                       check=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    with open(out) as f:
        return f.read()


@pytest.fixture(scope="module")
def kernels():
    """{demangled-ish symbol: list of assembly lines} over all three files."""
    with ThreadPoolExecutor(len(FILES)) as pool:
        texts = list(pool.map(_assemble, FILES))
    out = {}
    for text in texts:
        name, body = None, []
        for line in text.split("\n"):
            m = re.match(r"^(_Z\w+):", line)
            if m:
                name, body = m.group(1), []
                out[name] = body
            elif name is not None:
                body.append(line)          # up to the next symbol: the resource comments follow .Lfunc_end
    assert len(out) > 100
    return out


def find(kernels, *parts):
    hits = [k for k in kernels if all(p in k for p in parts)]
    assert len(hits) == 1, (parts, hits)
    return kernels[hits[0]]


def scratch_bytes(body):
    for line in body:
        m = re.match(r"^; ScratchSize: (\d+)", line)
        if m:
            return int(m.group(1))
    raise AssertionError("no ScratchSize line")


def loop_lines(body, innermost=False):
    """Lines inside any loop: the union of [label, backward branch to it] spans.  innermost: the shortest such span
    only (a block that the compiler laid out behind the loop and that jumps back to the code before it looks like a
    span around the loop)."""
    labels = {m.group(1): i for i, line in enumerate(body) if (m := re.match(r"^(\.LBB\w+):", line))}
    inside = [False] * len(body)
    spans = []
    for i, line in enumerate(body):
        m = re.match(r"^\s+s_c?branch\w*\s+(\.LBB\w+)", line)
        if m and labels.get(m.group(1), len(body)) < i:
            spans.append((i - labels[m.group(1)], labels[m.group(1)], i))
            for k in range(labels[m.group(1)], i + 1):
                inside[k] = True
    if innermost:
        _, first, last = min(spans)
        return body[first:last + 1]
    return [line for line, keep in zip(body, inside) if keep]


def events(lines):
    """Vector memory operations and vmcnt waits in text order: ('lds' | 'load' | 'store' | 'other', mnemonic) and
    ('wait', N)."""
    out = []
    for line in lines:
        m = re.match(r"^\s+s_waitcnt .*vmcnt\((\d+)\)", line)
        if m:
            out.append(("wait", int(m.group(1))))
            continue
        m = VMEM.match(line)
        if m:
            op = m.group(1) + m.group(2)
            kind = ("lds" if "load_lds" in op else "load" if "_load_" in op else "store" if "_store_" in op else "other")
            out.append((kind, op))
    return out


def between_counted_waits(ev, count):
    """For every wait of exactly `count`: the operations up to the next wait of any count (or the end)."""
    spans = []
    for i, e in enumerate(ev):
        if e == ("wait", count):
            span = []
            for f in ev[i + 1:]:
                if f[0] == "wait":
                    break
                span.append(f)
            spans.append(span)
    return spans


def kinds(span):
    out = {}
    for kind, _ in span:
        out[kind] = out.get(kind, 0) + 1
    return out


@pytest.mark.parametrize("elem,elem_bytes", [("DF16b", 2), ("f", 4)])
def test_sdd_stream_step_issues_what_its_wait_counts(kernels, elem, elem_bytes):
    L = lib()
    body = find(kernels, "sdd_nt_stream_kernelI" + elem + "E")
    assert scratch_bytes(body) == 0
    ev = events(loop_lines(body))
    count, loads, passes = L.ti_sdd_wait_count(elem_bytes), L.ti_sdd_wait_loads(elem_bytes), L.ti_slab_passes(elem_bytes)
    spans = between_counted_waits(ev, count)
    assert len(spans) == 1
    # a step issues the next tile's loads and the block's stores; the only other memory operations of the loop are
    # the four query fragments of a new block-row (the loop's first block in text order), drained at once
    assert [k for k, _ in spans[0]] == ["lds"] * loads + ["store"] * passes + ["load"] * 4
    assert ev.count(("wait", count)) == 1 and ev.count(("wait", 0)) == 1
    assert len([e for e in ev if e[0] != "wait"]) == len(spans[0])
    following = ev[ev.index(("wait", count)) + 1 + len(spans[0]):] + ev[:ev.index(("wait", count))]
    assert following[0] == ("wait", 0), "the query fragments are waited for before anything else is issued"


@pytest.mark.parametrize("elem,elem_bytes", [("DF16b", 2), ("f", 4)])
def test_sdd_softmax_stream_step_issues_what_its_waits_count(kernels, elem, elem_bytes):
    L = lib()
    body = find(kernels, "sdd_softmax_stream_kernelI" + elem + "E")
    assert scratch_bytes(body) == 0
    ev = events(loop_lines(body))
    count, loads, passes = L.ti_sdd_wait_count(elem_bytes), L.ti_sdd_wait_loads(elem_bytes), L.ti_slab_passes(elem_bytes)
    assert ("wait", count) in ev and ("wait", loads) in ev
    # a step: [wait] K tile loads, then possibly a mask word (drained at once), then the block's stores
    step = ev[ev.index(("wait", loads)) + 1:]
    assert [k for k, _ in step[:loads]] == ["lds"] * loads
    tail = step[loads:]
    if tail and tail[0][0] == "load":
        assert tail[1] == ("wait", 0)
        tail = tail[2:]
    assert [k for k, _ in tail[:passes]] == ["store"] * passes
    assert all(k == "wait" or k == "lds" for k, _ in ev[:ev.index(("wait", count))]), "pass prologue: tile loads only"
    assert kinds([e for e in ev if e[0] != "wait"]) in ({"lds": 3 * loads, "store": passes, "load": 1},
                                                        {"lds": 3 * loads, "store": passes})


# the streaming dsd kernel launched by block-rows and by work items
DSD_STREAM = ["dsd_nn_kernelILi64ELi64EDF16bDF16bLb0ELb0EE", "dsd_nn_kernelILi64ELi64EDF16bDF16bLb0ELb1EE"]


@pytest.mark.parametrize("name", DSD_STREAM)
def test_dsd_stream_steps_issue_what_their_wait_counts(kernels, name):
    L = lib()
    body = find(kernels, name)
    assert scratch_bytes(body) == 0
    ev = events(loop_lines(body, innermost=True))
    spans = between_counted_waits(ev, L.ti_dsd_wait_count())
    assert len(spans) == L.ti_dsd_depth() // 2
    for span in spans:
        assert [k for k, _ in span] == ["lds"] * (2 * L.ti_dsd_v_loads()) + ["load"] * (2 * L.ti_dsd_p_loads())
    assert sum(len(s) for s in spans) == len([e for e in ev if e[0] != "wait"]), "nothing else in the loop"


def registers(operand):
    """VGPR numbers an operand like v12 or v[8:11] names."""
    m = re.fullmatch(r"v(\d+)", operand)
    if m:
        return {int(m.group(1))}
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", operand)
    return set(range(int(m.group(1)), int(m.group(2)) + 1)) if m else set()


def in_flight_violations(code, laxer_by=0):
    """Walk a straight-line loop body twice in text order; loads into registers retire in issue order at every
    vmcnt wait (read as laxer_by more permissive than written, for the self-test below).  Returns (number of register
    loads seen, instructions that touch the destination registers of a load that may still be in flight)."""
    in_flight = []          # (sequence number, destination registers), oldest first
    issued = loads_seen = 0
    touched = []
    for sweep in range(2):
        for line in code:
            op, _, rest = line.partition(" ")
            operands = [o.strip() for o in rest.split(",")]
            m = re.match(r"s_waitcnt .*vmcnt\((\d+)\)", line)
            if m:
                in_flight = [(n, regs) for n, regs in in_flight if n > issued - (int(m.group(1)) + laxer_by)]
                continue
            used = set().union(*[registers(o.split()[0]) for o in operands if o]) if operands else set()
            busy = set().union(*[regs for _, regs in in_flight]) if in_flight else set()
            if VMEM.match("\t" + line):
                issued += 1
                if "_load_" in op and "lds" not in op:
                    # neither the address nor the destination of a new load may belong to a load still in flight
                    # (reloading registers whose previous load has been waited for is the normal case)
                    if used & busy:
                        touched.append(line)
                    in_flight.append((issued, registers(operands[0])))
                    loads_seen += 1
                    continue
            if used & busy:
                touched.append(line)
    return loads_seen, touched


@pytest.mark.parametrize("name", DSD_STREAM)
def test_registers_of_loads_in_flight_are_left_alone(kernels, name):
    """dsd (bf16): the P blocks are loaded into registers from inline assembly several blocks ahead and made valid by a
    counted wait, so the compiler believes them defined from the moment of issue: it must not read, copy or spill
    them before the wait that retires their loads.  Checked on the compiled loop (one straight-line block)."""
    body = loop_lines(find(kernels, name), innermost=True)
    code = [line.strip() for line in body if re.match(r"^\s+[a-z]", line)]
    assert not any(re.match(r"s_c?branch", c.split()[0]) for c in code[:-1]), "one straight-line block"
    loads_seen, touched = in_flight_violations(code)
    assert loads_seen == 2 * 16, "two sweeps over the four blocks' 16-byte loads"
    assert touched == [], touched[:5]
    # the walk does see a wait that retires too little.  (The count is set by the V tiles, which this walk does not
    # track -- test_dsd_stream_steps_issue_what_their_wait_counts does: behind the P registers a step reads stand
    # 8 tile loads and 8 loads of other P registers, so the registers only show up 9 operations laxer.)
    assert in_flight_violations(code, laxer_by=8)[1] == []
    assert in_flight_violations(code, laxer_by=9)[1] != []


def test_m0_is_only_written_for_the_lds_direct_loads(kernels):
    """Every instruction that names M0 is an s_mov into it, and the next instruction (after the s_nop of the same
    inline-assembly statement) is the LDS-direct load that reads it."""
    seen = 0
    for name, body in kernels.items():
        code = [line for line in body if re.match(r"^\s+[a-z]", line)]
        for i, line in enumerate(code):
            if not re.search(r"\bm0\b", line):
                continue
            assert re.match(r"^\s+s_mov_b32 m0, (s\d+|vcc_lo|vcc_hi|ttmp\d+)\s*$", line), (name, line)
            follow = [c.split()[0] for c in code[i + 1:i + 3]]
            assert follow == ["s_nop", "global_load_lds_dwordx4"], (name, line, follow)
            seen += 1
    assert seen > 1000


def test_the_model_of_a_step_is_not_vacuous(kernels):
    """The span extraction does see a count that does not match: the fp32 kernel's loop against the bf16 count."""
    L = lib()
    ev = events(loop_lines(find(kernels, "sdd_nt_stream_kernelIfE")))
    assert between_counted_waits(ev, L.ti_sdd_wait_count(2)) == []
    spans = between_counted_waits(ev, L.ti_sdd_wait_count(4))
    assert kinds(spans[0]) != {"lds": L.ti_sdd_wait_loads(2), "store": L.ti_slab_passes(2)}


def innermost_loops(body):
    """[label, backward branch] spans that contain no other such span."""
    labels = {m.group(1): i for i, line in enumerate(body) if (m := re.match(r"^(\.LBB\w+):", line))}
    spans = []
    for i, line in enumerate(body):
        m = re.match(r"^\s+s_c?branch\w*\s+(\.LBB\w+)", line)
        if m and labels.get(m.group(1), len(body)) < i:
            spans.append((labels[m.group(1)], i))
    return [body[a:b + 1] for a, b in spans if not any((c, d) != (a, b) and a <= c and d <= b for c, d in spans)]


def instruction_mix(lines):
    mix = {}
    for line in lines:
        m = re.match(r"^\s+([a-z][a-z0-9_]+)", line)
        if not m:
            continue
        op = m.group(1)
        kind = ("mfma" if op.startswith("v_mfma") else "exp" if op.startswith("v_exp") else
                "lds_direct" if op.startswith("global_load_lds") else "vmem" if op.startswith(("global_", "buffer_", "scratch_")) else
                "tr_read" if op.startswith("ds_read_b64_tr") else "ds_read" if op.startswith("ds_read") else
                "ds_write" if op.startswith("ds_write") else "barrier" if op == "s_barrier" else
                "valu" if op.startswith("v_") else "salu" if op.startswith("s_") else "other")
        mix[kind] = mix.get(kind, 0) + 1
    return mix


def test_instruction_mix_of_the_benchmarked_loop(kernels):
    """The loop that the benchmarked launch runs (bf16, block 64, head 64, no mask: scale and offset folded into the
    score product) handles two key blocks per trip (one per tile-buffer parity).  Per trip and wave: the 2 x 16 matrix
    instructions of the two products, one v_exp per probability and nothing more transcendental, 16 LDS-direct loads
    (a K and a V tile per block, four loads each), fragments read from LDS only as 128-bit and transposing reads, no
    LDS writes, no other memory traffic than the two look-up entries, two barriers; and a bounded count of ordinary
    vector instructions beside them (the softmax's share of the issue slots: about 5.5 per probability pair)."""
    body = find(kernels, "fused_attention_bf16_kernelILi64ELi64ELb0ELb0E")
    assert scratch_bytes(body) == 0
    lean = [loop for loop in innermost_loops(body) if instruction_mix(loop).get("mfma", 0) == 32]
    assert lean, "no loop with the matrix instructions of two key blocks"
    mix = instruction_mix(lean[0])
    assert mix["exp"] == 64 and mix["lds_direct"] == 16 and mix["ds_read"] == 16 and mix["tr_read"] == 32
    assert mix.get("ds_write", 0) == 0 and mix["barrier"] == 2 and mix.get("vmem", 0) <= 2
    assert mix["valu"] <= 190, mix
