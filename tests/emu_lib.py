"""Builds the library's kernel sources for the host and runs them there (no GPU): test infrastructure.

The .hip files are compiled as they are, as plain C++ against tests/emu/hip/hip_runtime.h, after a textual rewrite of
the three things that are not C++:

* ``kernel<<<grid, block, shared, stream>>>(args);``  ->  ``emu::launch(grid, block, shared, stream, [=]() { kernel(args); });``
* ``__shared__ T name[N];``  ->  a reference into the work-group's LDS arena
* ``asm volatile(...)``  ->  the model's function for the instructions it contains; an instruction sequence this
  file does not know stops the build, so a kernel change cannot silently leave the model behind.

Counted waits: the model keeps only LDS-direct loads in its queue (ordinary loads and stores execute at once), so a wait
whose count includes ordinary memory operations is mapped to the number of LDS-direct loads it is documented to
leave in flight (the kernels' own SddStreamWait / DsdStreamWait constants); that the count matches the compiled
sequence of memory operations is what test_counted_waits.py and test_compiled_kernels.py check.

The result, tests/_build/emu/libsfbert_emu.so, exports the C ABI of include/sfbert_hip.h (the GEMM entry points
included: tests/emu/hipblaslt, tests/emu/rocblas stand in for the libraries) with host pointers in place of
device pointers.
"""
import ctypes as C
import hashlib
import importlib.util
import os
import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "sf-bert_amd", "csrc")
EMU = os.path.join(HERE, "emu")
BUILD = os.path.join(HERE, "_build", "emu")
LIB = os.path.join(BUILD, "libsfbert_emu.so")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"

KERNEL_SOURCES = ["fused_attention.hip", "fused_backward.hip", "unfused_attention.hip", "layer_ops.hip", "runtime.hip",
                  "encoder_layer.hip"]
HOST_SOURCES = ["descriptors.cpp"]
HEADERS = ["common.hip.h", "tiles.hip.h", "tile_index.h"]

# plain x86-64 (no instruction-set extensions: the build runs wherever the tests do); products and sums are not
# contracted, so that host arithmetic rounds where the kernels' source says it does
HOST_FLAGS = ["-O1", "-g0", "-std=c++17", "-fPIC", "-I" + EMU, "-Wno-everything", "-ffp-contract=off"]

OPS = ["none", "block_barrier", "block_and", "wave_barrier", "mfma_bf16", "mfma_f32", "readfirstlane", "readlane",
       "ballot", "shfl_xor", "ds_read_tr16", "dpp", "yield"]


# ---------------------------------------------------------------------------------------------------------------
# source rewrite
# ---------------------------------------------------------------------------------------------------------------
def _balanced(text, start):
    """Index just past the parenthesis that closes the one at text[start]."""
    assert text[start] == "("
    depth, i, in_string = 0, start, False
    while i < len(text):
        ch = text[i]
        if in_string:
            if ch == "\\":
                i += 1
            elif ch == '"':
                in_string = False
        elif ch == '"':
            in_string = True
        elif ch == "(":
            depth += 1
        elif ch == ")":
            depth -= 1
            if depth == 0:
                return i + 1
        i += 1
    raise ValueError("unbalanced parenthesis")


def _split_asm(body):
    """asm body -> (template text, [output expressions], [input expressions])."""
    parts, depth, in_string, current = [], 0, False, ""
    i = 0
    while i < len(body):
        ch = body[i]
        if in_string:
            current += ch
            if ch == "\\":
                current += body[i + 1]
                i += 1
            elif ch == '"':
                in_string = False
        elif ch == '"':
            in_string = True
            current += ch
        elif ch in "([":
            depth += 1
            current += ch
        elif ch in ")]":
            depth -= 1
            current += ch
        elif ch == ":" and depth == 0:
            parts.append(current)
            current = ""
        else:
            current += ch
        i += 1
    parts.append(current)
    template = "".join(re.findall(r'"((?:[^"\\]|\\.)*)"', parts[0]))
    template = template.replace("\\n", "\n").replace("\\t", " ")

    def operands(text):
        out, j = [], 0
        while True:
            m = re.compile(r'\s*,?\s*"[^"]*"\s*\(').match(text, j)
            if not m:
                break
            end = _balanced(text, m.end() - 1)
            out.append(text[m.end():end - 1].strip())
            j = end
        return out

    outputs = operands(parts[1]) if len(parts) > 1 else []
    inputs = operands(parts[2]) if len(parts) > 2 else []
    return template, outputs, inputs


def _asm_replacement(template, outputs, inputs, where):
    ops = outputs + inputs

    def arg(token):
        return "(" + ops[int(token[1:])] + ")"

    lines = [ln.strip() for ln in template.split("\n") if ln.strip()]
    code = []
    i = 0
    while i < len(lines):
        ln = lines[i]
        m = re.fullmatch(r"s_waitcnt vmcnt\((%\d+|\d+)\)", ln)
        if m:
            n = m.group(1)
            count = arg(n) if n.startswith("%") else n
            # a count that includes ordinary loads and stores: the LDS-direct loads it leaves in flight
            count = re.sub(r"(SddStreamWait<[^;]*?>)::COUNT", r"\1::LOADS", count)
            count = count.replace("DsdStreamWait::COUNT", "0")   # only loads into registers stand behind it
            code.append("emu::s_waitcnt_vmcnt(%s);" % count)
        elif ln.startswith("s_mov_b32 m0,"):
            m0 = arg(ln.split(",")[1].strip())
            assert lines[i + 1] == "s_nop 0", (where, lines)
            i += 2
            n_loads = 0
            while i < len(lines) and lines[i].startswith("global_load_lds_dwordx4"):
                m = re.fullmatch(r"global_load_lds_dwordx4 (%\d+), (%\d+)(?: offset:(%\d+|-?\d+))?", lines[i])
                assert m, (where, lines[i])
                off = m.group(3) or "0"
                off = arg(off) if off.startswith("%") else off
                code.append("emu::global_load_lds_dwordx4(%s, %s, %s, %s);" % (m0, arg(m.group(1)), arg(m.group(2)), off))
                n_loads += 1
                i += 1
            assert n_loads > 0, (where, lines)
            continue
        elif ln.startswith("global_load_dwordx4"):
            m = re.fullmatch(r"global_load_dwordx4 (%\d+), (%\d+), (%\d+)(?: offset:(\d+))?", ln)
            assert m, (where, ln)
            code.append("memcpy(&%s, (const uint8_t*)(uintptr_t)%s + %s + %s, 16);"
                        % (arg(m.group(1)), arg(m.group(3)), arg(m.group(2)), m.group(4) or "0"))
        elif ln.startswith("global_store_dwordx4"):
            m = re.fullmatch(r"global_store_dwordx4 (%\d+), (%\d+), off sc1", ln)
            assert m, (where, ln)
            code.append("memcpy((void*)%s, &%s, 16);" % (arg(m.group(1)), arg(m.group(2))))
        else:
            raise AssertionError("%s: inline assembly the host model does not know: %r" % (where, ln))
        i += 1
    return "do { " + " ".join(code) + " } while (0)" if code else "((void)0)"


def rewrite(text, name):
    # attributes of the device compiler
    text = re.sub(r"__attribute__\(\(amdgpu_waves_per_eu\((?:[^()]|\([^()]*\))*\)\)\)", "", text)
    # inline assembly
    out, pos = "", 0
    for m in re.finditer(r"\basm\s+volatile\s*\(", text):
        if m.start() < pos:
            continue
        end = _balanced(text, m.end() - 1)
        template, outputs, inputs = _split_asm(text[m.end():end - 1])
        line = text.count("\n", 0, m.start()) + 1
        replacement = _asm_replacement(template, outputs, inputs, "%s:%d" % (name, line))
        # keep the line count, so that compiler messages point at the original lines
        newlines = text.count("\n", m.start(), end)
        continuation = "\\\n" if _inside_macro(text, m.start()) else "\n"
        out += text[pos:m.start()] + replacement + continuation * newlines
        pos = end
    text = out + text[pos:]
    assert "asm(" not in text and "asm volatile" not in text, name

    # __shared__ declarations
    def shared(m):
        align = m.group("align") or "16"
        ctype, var, dims = m.group("type"), m.group("name"), m.group("dims") or ""
        return ("typedef %s emu_lds_%s_t%s; static char emu_lds_%s_site; emu_lds_%s_t& %s = "
                "*(emu_lds_%s_t*)emu::lds_alloc(&emu_lds_%s_site, sizeof(emu_lds_%s_t), %s);"
                % (ctype, var, dims, var, var, var, var, var, var, align))
    text, n_shared = re.subn(
        r"__shared__\s+(?:__attribute__\(\(aligned\((?P<align>\d+)\)\)\)\s+)?(?P<type>[\w:]+)\s+(?P<name>\w+)"
        r"(?P<dims>(?:\[[^\]]+\])*)\s*;", shared, text)
    assert "__shared__" not in re.sub(r"//[^\n]*", "", text), name

    # kernel launches
    out, pos = "", 0
    while True:
        at = text.find("<<<", pos)
        if at < 0:
            break
        start = _kernel_name_start(text, at)
        close = text.index(">>>", at)
        paren = close + 3
        while text[paren] in " \t":
            paren += 1
        assert text[paren] == "(", (name, text[at:at + 80])
        end = _balanced(text, paren)
        out += text[pos:start] + "emu::launch(%s, [=]() { %s(%s); })" % (text[at + 3:close], text[start:at].strip(),
                                                                      text[paren + 1:end - 1])
        pos = end
    text = out + text[pos:]
    return text


def _kernel_name_start(text, at):
    """Start of `name` or `name<template arguments>` that ends at text[at]."""
    i = at - 1
    while text[i] in " \t":
        i -= 1
    if text[i] == ">":
        depth = 0
        while True:
            if text[i] == ">":
                depth += 1
            elif text[i] == "<":
                depth -= 1
                if depth == 0:
                    break
            i -= 1
        i -= 1
    while text[i].isalnum() or text[i] in "_:":
        i -= 1
    return i + 1


def _inside_macro(text, at):
    """Whether position `at` lies in a #define continued over several lines."""
    line_start = text.rfind("\n", 0, at) + 1
    prev_end = line_start - 1
    return prev_end > 0 and text[prev_end - 1] == "\\"


# ---------------------------------------------------------------------------------------------------------------
# build
# ---------------------------------------------------------------------------------------------------------------
def _digest():
    h = hashlib.sha256()
    files = [os.path.join(CSRC, f) for f in KERNEL_SOURCES + HOST_SOURCES + HEADERS]
    files += [os.path.join(EMU, "hipblaslt", "hipblaslt.h"), os.path.join(EMU, "hipblaslt", "hipblaslt-ext.hpp"),
              os.path.join(EMU, "rocblas", "rocblas.h")]
    files += [os.path.join(EMU, "hip", "hip_runtime.h"), os.path.join(EMU, "emu_runtime.cpp"), os.path.abspath(__file__),
              os.path.join(EMU, "selftest_kernels.hip"),
              os.path.join(ROOT, "include", "sfbert_hip.h")]
    for f in files:
        h.update(open(f, "rb").read())
    return h.hexdigest()


def build(verbose=False):
    os.makedirs(os.path.join(BUILD, "sf-bert_amd", "csrc"), exist_ok=True)
    stamp = os.path.join(BUILD, "digest")
    digest = _digest()
    if os.path.exists(LIB) and os.path.exists(stamp) and open(stamp).read() == digest:
        return LIB
    # the rewritten sources keep their relative position to include/, which they name in #include lines
    gen = os.path.join(BUILD, "sf-bert_amd", "csrc")
    os.makedirs(os.path.join(BUILD, "include"), exist_ok=True)
    with open(os.path.join(BUILD, "include", "sfbert_hip.h"), "w") as f:
        f.write(open(os.path.join(ROOT, "include", "sfbert_hip.h")).read())
    units = []
    for name in KERNEL_SOURCES + HEADERS:
        text = rewrite(open(os.path.join(CSRC, name)).read(), name)
        target = os.path.join(gen, name if name.endswith(".h") else name.replace(".hip", "_emu.cpp"))
        with open(target, "w") as f:
            f.write(text)
        if not name.endswith(".h"):
            units.append(target)
    selftest = os.path.join(gen, "selftest_kernels_emu.cpp")
    with open(selftest, "w") as f:
        f.write(rewrite(open(os.path.join(EMU, "selftest_kernels.hip")).read(), "selftest_kernels.hip"))
    units += [selftest] + [os.path.join(CSRC, f) for f in HOST_SOURCES] + [os.path.join(EMU, "emu_runtime.cpp")]
    flags = HOST_FLAGS

    def compile_unit(src):
        obj = os.path.join(BUILD, os.path.basename(src) + ".o")
        # (the scheduler itself, where the model spends its time, is optimised further)
        cmd = [CLANG, "-x", "c++"] + flags + (["-O2"] if src.endswith("emu_runtime.cpp") else []) + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=6) as pool:
        objects = list(pool.map(compile_unit, units))
    # linked under another name and moved into place: a process that has the old library loaded keeps it
    subprocess.check_call([CLANG, "-shared", "-o", LIB + ".new"] + objects + ["-lm"])
    os.replace(LIB + ".new", LIB)
    with open(os.path.join(BUILD, "objects"), "w") as f:
        f.write("\n".join(objects))
    with open(stamp, "w") as f:
        f.write(digest)
    return LIB


def build_sanitized(verbose=False):
    """Every unit of the host build compiled with the undefined-behaviour sanitizer (misaligned vector accesses,
    out-of-range shifts and indices of fixed arrays, signed overflow): tests/_build/emu/libsfbert_emu_ubsan.so.
    Findings are printed to stderr and counted by the runtime's own handler; see test_emulated_kernels.py."""
    build()
    lib = os.path.join(BUILD, "libsfbert_emu_ubsan.so")
    stamp = os.path.join(BUILD, "digest_ubsan")
    digest = _digest()
    if os.path.exists(lib) and os.path.exists(stamp) and open(stamp).read() == digest:
        return lib
    gen = os.path.join(BUILD, "sf-bert_amd", "csrc")
    units = [os.path.join(gen, name.replace(".hip", "_emu.cpp")) for name in KERNEL_SOURCES]
    units += [os.path.join(gen, "selftest_kernels_emu.cpp")] + [os.path.join(CSRC, f) for f in HOST_SOURCES]
    units += [os.path.join(EMU, "emu_runtime.cpp")]
    flags = [f if f != "-g0" else "-g1" for f in HOST_FLAGS] + [
             "-fsanitize=undefined", "-fno-sanitize=vptr,function", "-fno-sanitize-recover=undefined",
             "-fsanitize-trap=undefined"]

    def compile_unit(src):
        obj = os.path.join(BUILD, os.path.basename(src) + ".ubsan.o")
        subprocess.check_call([CLANG, "-x", "c++"] + flags + ["-c", src, "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=6) as pool:
        objects = list(pool.map(compile_unit, units))
    subprocess.check_call([CLANG, "-shared", "-o", lib + ".new"] + objects + ["-lm"])
    os.replace(lib + ".new", lib)
    with open(stamp, "w") as f:
        f.write(digest)
    return lib


def build_host_program(name):
    """A C++ host program of sf-bert_amd/host/ (they drive the library through the reference-named launchers) built
    against the stand-in runtime and the host build: tests/_build/emu/<name>."""
    lib = build()
    src = os.path.join(ROOT, "sf-bert_amd", "host", name + ".cpp")
    exe = os.path.join(BUILD, name)
    if os.path.exists(exe) and os.path.getmtime(exe) > max(os.path.getmtime(src), os.path.getmtime(lib)):
        return exe
    subprocess.check_call([CLANG, "-O1", "-std=c++17", "-w", "-I" + EMU, "-o", exe, "-x", "c++", src, "-x", "none", lib,
                           "-Wl,-rpath," + BUILD, "-lm"])
    return exe


def build_mutant(tag, source, old, new, count=1):
    """The host build with one deliberate mistake: the text `old` of the rewritten kernel source (or of a rewritten
    header, when `source` is one) replaced by `new`.  tests/_build/emu/mutants/<tag>/libsfbert_emu.so.  For the check
    that the tests on the host model notice mistakes in the real kernels (test_host_model_mutants.py)."""
    build()
    gen = os.path.join(BUILD, "sf-bert_amd", "csrc")
    out = os.path.join(BUILD, "mutants", tag)
    mgen = os.path.join(out, "sf-bert_amd", "csrc")
    os.makedirs(mgen, exist_ok=True)
    os.makedirs(os.path.join(out, "include"), exist_ok=True)
    with open(os.path.join(out, "include", "sfbert_hip.h"), "w") as f:
        f.write(open(os.path.join(ROOT, "include", "sfbert_hip.h")).read())
    lib = os.path.join(out, "libsfbert_emu.so")
    stamp = os.path.join(out, "digest")
    digest = _digest() + repr((source, old, new))
    if os.path.exists(lib) and os.path.exists(stamp) and open(stamp).read() == digest:
        return lib
    changed = source if source.endswith(".h") else source.replace(".hip", "_emu.cpp")
    for name in HEADERS:   # every header beside the units that include it
        text = open(os.path.join(gen, name)).read()
        if name == changed:
            assert text.count(old) == count, (tag, text.count(old))
            text = text.replace(old, new)
        with open(os.path.join(mgen, name), "w") as f:
            f.write(text)
    flags = HOST_FLAGS
    objects = open(os.path.join(BUILD, "objects")).read().split("\n")
    # a header is included by the three attention sources; a source stands for itself
    units = (["fused_attention_emu.cpp", "fused_backward_emu.cpp", "unfused_attention_emu.cpp"] if source.endswith(".h")
             else [changed])

    def compile_unit(unit):
        text = open(os.path.join(gen, unit)).read()
        if unit == changed:
            assert text.count(old) == count, (tag, text.count(old))
            text = text.replace(old, new)
        src = os.path.join(mgen, unit)
        with open(src, "w") as f:
            f.write(text)
        obj = os.path.join(out, unit + ".o")
        subprocess.check_call([CLANG, "-x", "c++"] + flags + ["-c", src, "-o", obj])
        return unit, obj

    with ThreadPoolExecutor(max_workers=3) as pool:
        rebuilt = dict(pool.map(compile_unit, units))
    linked = [rebuilt.get(os.path.basename(o)[:-2], o) for o in objects]
    subprocess.check_call([CLANG, "-shared", "-o", lib + ".new"] + linked + ["-lm"])
    os.replace(lib + ".new", lib)
    with open(stamp, "w") as f:
        f.write(digest)
    return lib


def build_variant(tag, defines, source="fused_attention.hip"):
    """The host build with one kernel source compiled under other preprocessor definitions (the opt-in kernel
    variants of sf-bert_amd/build.py): tests/_build/emu/libsfbert_emu_<tag>.so."""
    build()
    lib = os.path.join(BUILD, "libsfbert_emu_%s.so" % tag)
    stamp = os.path.join(BUILD, "digest_" + tag)
    digest = _digest() + " " + " ".join(defines)
    if os.path.exists(lib) and os.path.exists(stamp) and open(stamp).read() == digest:
        return lib
    src = os.path.join(BUILD, "sf-bert_amd", "csrc", source.replace(".hip", "_emu.cpp"))
    obj = os.path.join(BUILD, "%s_%s.o" % (os.path.basename(src), tag))
    flags = HOST_FLAGS + ["-D" + d for d in defines]
    subprocess.check_call([CLANG, "-x", "c++"] + flags + ["-c", src, "-o", obj])
    others = [o for o in open(os.path.join(BUILD, "objects")).read().split("\n")
              if os.path.basename(o) != os.path.basename(src) + ".o"]
    subprocess.check_call([CLANG, "-shared", "-o", lib + ".new", obj] + others + ["-lm"])
    os.replace(lib + ".new", lib)
    with open(stamp, "w") as f:
        f.write(digest)
    return lib


# ---------------------------------------------------------------------------------------------------------------
# use
# ---------------------------------------------------------------------------------------------------------------
_modules = {}


def load(tag="", defines=()):
    """The package's ctypes binding (capi.py), bound to the host build instead of libsfbert_hip.so (tag, defines: to
    a variant of it, see build_variant)."""
    if tag in _modules:
        return _modules[tag]
    if isinstance(defines, dict):   # a mutant: dict(source=, old=, new=[, count=])
        lib_path = build_mutant(tag, **defines)
    else:
        lib_path = build_sanitized() if tag == "ubsan" else build_variant(tag, defines) if tag else build()
    saved = os.environ.get("SFBERT_HIP_LIB")
    os.environ["SFBERT_HIP_LIB"] = lib_path
    try:
        spec = importlib.util.spec_from_file_location("sfb_emulated" + ("_" + tag if tag else ""),
                                                      os.path.join(ROOT, "sf-bert_amd", "capi.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    finally:
        if saved is None:
            del os.environ["SFBERT_HIP_LIB"]
        else:
            os.environ["SFBERT_HIP_LIB"] = saved
    mod._stream = lambda: None
    mod.to_device = lambda a: tensor(np.ascontiguousarray(a).view(np.uint8).reshape(-1))
    lib = mod.lib
    lib.emu_guarded_alloc.restype = C.c_void_p
    lib.emu_guarded_alloc.argtypes = [C.c_size_t]
    lib.emu_message.restype = C.c_char_p
    lib.emu_count.restype = C.c_uint64
    lib.emu_partial_count.restype = C.c_uint64
    _modules[tag] = mod
    return mod


def configure(order=0, lazy_loads=True, resident=64):
    """Lane order (0 ascending, 1 descending, n > 1 shuffled with seed n and waves held back at random), whether
    LDS-direct loads land only at the wait that asks for them, and the work-groups in flight; for every build loaded."""
    load()
    for mod in _modules.values():
        mod.lib.emu_configure(int(order), int(bool(lazy_loads)), int(resident))


def counts():
    lib = load().lib
    return {name: (int(lib.emu_count(i)), int(lib.emu_partial_count(i))) for i, name in enumerate(OPS)}


def message():
    return load().lib.emu_message().decode()


_keep = []


def tensor(array, bf16=False):
    """A torch CPU tensor holding `array` in memory that ends at an inaccessible page: a kernel that reads or writes
    past the end of a tensor takes a segmentation fault instead of going unnoticed."""
    import torch
    array = np.ascontiguousarray(array)
    if bf16:
        t = torch.from_numpy(array.astype(np.float32)).to(torch.bfloat16)
        out = empty(t.shape, torch.bfloat16)
        out.copy_(t)
        return out
    out = empty(array.shape, torch.from_numpy(array[:0].reshape(-1)).dtype)
    out.copy_(torch.from_numpy(array))
    return out


def empty(shape, dtype, fill=None):
    import torch
    lib = load().lib
    n = int(np.prod(shape)) if len(shape) else 1
    item = torch.finfo(dtype).bits // 8 if dtype.is_floating_point else torch.iinfo(dtype).bits // 8
    nbytes = max(n * item, 16)
    ptr = lib.emu_guarded_alloc(nbytes)
    assert ptr
    buf = (C.c_uint8 * nbytes).from_address(ptr)
    _keep.append(buf)
    t = torch.frombuffer(buf, dtype=dtype, count=n).reshape(tuple(shape))
    if fill is not None:
        t.fill_(fill)
    return t


def install(monkeypatch=None):
    """Makes the tests marked gpu run on the host build: the package name resolves to the binding of the host build,
    'device' tensors are host tensors in guarded memory, and the few torch.cuda calls the tests make are inert.
    With a pytest MonkeyPatch the changes to torch are undone with it (and the package name is left alone)."""
    import sys
    import torch
    mod = load()
    mod.capi = mod
    if monkeypatch is None:
        sys.modules["sf-bert_amd"] = mod

        def put(owner, name, value):
            setattr(owner, name, value)
    else:
        put = monkeypatch.setattr

    def to_guarded(t):
        if t.numel() * t.element_size() > (1 << 30):
            return t.clone()
        out = empty(t.shape, t.dtype)
        out.copy_(t)
        return out

    put(torch.Tensor, "cuda", lambda self, *a, **k: to_guarded(self))
    put(torch.cuda, "synchronize", lambda *a, **k: None)
    put(torch.cuda, "memory_allocated", lambda *a, **k: 0)

    class _Stream:
        cuda_stream = 0
    put(torch.cuda, "current_stream", lambda *a, **k: _Stream())

    def host(factory, guarded):
        def make(*args, **kwargs):
            on_device = "device" in kwargs
            if str(kwargs.get("device", "cpu")).startswith("cuda"):
                kwargs["device"] = "cpu"
            t = factory(*args, **kwargs)
            return to_guarded(t) if (on_device and guarded) else t
        return make
    for name in ("zeros", "empty", "ones", "full", "randn", "rand", "randint", "tensor", "arange", "zeros_like", "empty_like"):
        put(torch, name, host(getattr(torch, name), name != "tensor"))
    return mod
