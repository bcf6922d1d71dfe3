"""The Go sources under integration/go (the files a go-metal maintainer copies over a checkout) against the C
header they bind: no Go toolchain exists here, so they cannot be compiled; what can be checked mechanically is
that every C function they call is declared in include/gometal_hip.h with the number of arguments they pass, and
that every error string and hook they rely on is the one the tested C++ mirror uses."""
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GO = os.path.join(ROOT, "integration", "go")
C_TYPES = {"int", "float", "uintptr_t", "double", "char", "size_t", "uint64_t"}


def split_top_level(args):
    """Arguments of a call or a prototype, split at commas outside parentheses and brackets."""
    parts, depth, cur = [], 0, ""
    for ch in args:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        parts.append(cur.strip())
    return parts


def header_prototypes(with_types=False):
    text = open(os.path.join(ROOT, "include", "gometal_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    protos = {}
    for m in re.finditer(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(([^()]*)\)\s*;", text):
        name, args = m.group(1), m.group(2).strip()
        params = [] if args in ("", "void") else split_top_level(args)
        protos[name] = [c_kind(p) for p in params] if with_types else len(params)
    return protos


def c_kind(param):
    """pointer / float / int / uintptr_t of a C parameter declaration."""
    if "*" in param:
        return "pointer"
    for kind in ("float", "uintptr_t", "int"):
        if re.search(rf"\b{kind}\b", param):
            return kind
    return param


def go_kind(arg):
    """The same classification of an argument expression of a cgo call."""
    arg = arg.strip()
    if arg.startswith("&") or arg.startswith("first("):
        return "pointer"
    m = re.match(r"C\.([A-Za-z_0-9]+)\(", arg)
    return m.group(1) if m else arg


def go_c_calls(path):
    """(name, number of arguments, line) of every C.name(...) call in a Go file, casts to C types left out."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", lambda m: "\n" * m.group(0).count("\n"), text, flags=re.S)    # the cgo preamble
    text = re.sub(r"//[^\n]*", "", text)
    calls = []
    for m in re.finditer(r"\bC\.([A-Za-z_][A-Za-z0-9_]*)\s*\(", text):
        name = m.group(1)
        if name in C_TYPES:
            continue
        depth, i = 1, m.end()
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        args = split_top_level(text[m.end():i - 1])
        calls.append((name, len(args), text.count("\n", 0, m.start()) + 1, args))
    return calls


def go_files():
    files = sorted(glob.glob(os.path.join(GO, "**", "*.go"), recursive=True))
    assert len(files) >= 5
    return files


def test_every_c_function_the_go_wrappers_call_is_declared_with_that_arity():
    protos = header_prototypes()
    assert protos["execute_adam_amp_step"] == 18 and protos["execute_adam_amp_step_fused"] == 22
    assert protos["gm_allocate_buffer_phased"] == 4 and protos["gm_amp_state_query"] == 5
    seen = set()
    for path in go_files():
        for name, nargs, line, _ in go_c_calls(path):
            where = f"{os.path.relpath(path, ROOT)}:{line}"
            assert name in protos, f"{where}: C.{name} is not declared in include/gometal_hip.h"
            assert nargs == protos[name], f"{where}: C.{name} called with {nargs} arguments, declared with {protos[name]}"
            seen.add(name)
    assert {"execute_adam_amp_step", "execute_adam_amp_step_async", "execute_adam_amp_step_fused",
            "execute_adam_amp_step_fused_async", "gm_allocate_buffer_phased", "gm_amp_state_create",
            "gm_amp_state_destroy", "gm_amp_state_query", "gm_amp_state_set", "gm_amp_state_set_step_count",
            "gm_amp_state_current_set", "gm_amp_state_set_current_set", "gm_synchronize"} <= seen


def test_every_argument_of_a_cgo_call_has_the_kind_the_header_declares():
    """Position by position: a pointer where the header has a pointer, C.float where it has float, C.int where it has
    int, C.uintptr_t where it has uintptr_t (two arguments swapped in a call would compile in C and fail here)."""
    protos = header_prototypes(with_types=True)
    checked = 0
    for path in go_files():
        for name, _, line, args in go_c_calls(path):
            got = [go_kind(a) for a in args]
            assert got == protos[name], f"{os.path.relpath(path, ROOT)}:{line}: C.{name}({got}) against {protos[name]}"
            checked += len(args)
    assert checked > 90


def test_go_files_are_plausible_go():
    """Balanced braces and parentheses, a package clause, the build tag on the files that need the library."""
    for path in go_files():
        text = open(path).read()
        code = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        code = re.sub(r"//[^\n]*", "", code)
        code = re.sub(r'"(\\.|[^"\\])*"', '""', code)
        for a, b in ("()", "{}", "[]"):
            assert code.count(a) == code.count(b), (path, a)
        package = os.path.basename(os.path.dirname(path))
        assert re.search(rf"^package {package}$", text, flags=re.M), path
        if "C." in code or "cgo_bridge.AMPSet" in code or "AllocateMetalBufferPhased" in code:
            assert text.startswith("//go:build linux && amd64\n"), path


def test_go_error_strings_are_the_mirrors():
    """The Go methods were written from the C++ mirror the GPU tests drive (host/optimizer.cpp, host/bridge.cpp):
    every error string of theirs must occur there too (format verbs aside: %v in Go where C++ has %s)."""
    mirror = "".join(open(os.path.join(ROOT, "go-metal_amd", "host", f)).read()
                     for f in ("optimizer.cpp", "bridge.cpp", "memory_manager.cpp"))
    mirror = mirror.replace('"\n', '"').replace("%s", "%v")
    mirror = re.sub(r'"\s*\n\s*"', "", mirror)
    own = {"loss-scale state query failed with error code: %d", "loss-scale state update failed with error code: %d",
           "loss-scale state step count update failed with error code: %d", "failed to create loss-scale state",
           "device synchronisation failed with error code: %d",
           "failed to allocate Metal buffer of size %d at phase %d"}          # the wrappers' own, one per new C call
    for name in ("optimizer/adam_amp.go", "cgo_bridge/bridge_amp_linux.go"):
        text = open(os.path.join(GO, name)).read()
        for m in re.finditer(r'fmt\.Errorf\("((?:\\.|[^"\\])*)"', text):
            msg = m.group(1)
            assert msg in own or msg in mirror, (name, msg)


def test_hooks_named_in_the_go_files_exist():
    """adam_amp.go tells the maintainer which lines of adam.go call into it; those functions are defined."""
    text = open(os.path.join(GO, "optimizer", "adam_amp.go")).read()
    for fn in ("beforeStep", "cleanupAMP", "CurrentWeightBuffers", "CurrentMomentumBuffers", "CurrentVarianceBuffers",
               "finishPendingAMP", "EnableMixedPrecision", "EnablePingPong", "StepAMP", "StepAMPAsync", "SyncAMP"):
        assert re.search(rf"^func \(adam \*AdamOptimizerState\) {fn}\(", text, flags=re.M), fn
    mem = open(os.path.join(GO, "memory", "manager_state.go")).read()
    for fn in ("AllocateStateBuffer", "AllocateBufferAtPhase", "releasePlaced"):
        assert re.search(rf"^func \(mm \*MemoryManager\) {fn}\(", mem, flags=re.M), fn
    # the constants are the C++ mirror's
    hpp = open(os.path.join(ROOT, "go-metal_amd", "host", "memory_manager.hpp")).read()
    assert "kStatePhases[3] = {512 << 10, 1536 << 10, 1 << 20}" in hpp and "[3]int{512 << 10, 1536 << 10, 1 << 20}" in mem
    assert "kShadowWeightPhase = 1 << 20" in hpp and "ShadowWeightPhase = 1 << 20" in mem
    assert "kPhasedMinBytes = 16 << 20" in hpp and "PhasedMinBytes = 16 << 20" in mem


def test_go_oracle_restates_every_statement_the_c_oracle_cites():
    """oracle_cpu.go is the Go form of oracle/oracle.c's update rules (it cannot be run here).  Both annotate every
    statement with the line of bridge_optimizer.m it follows: each citation of the C rules must appear in the Go file,
    the same number of times, so a statement dropped or doubled in the translation shows."""
    c_text = open(os.path.join(ROOT, "oracle", "oracle.c")).read()
    rules = c_text[c_text.index("void gm_oracle_sgd_step"):c_text.index("/* ---- fp16 casts")]
    go_text = open(os.path.join(GO, "optimizer", "oracle_cpu.go")).read()
    go_rules = go_text[go_text.index("func OracleSGDStep"):go_text.index("// Float16ToFloat32")]
    cite = lambda text, pattern: sorted(re.findall(pattern, text))
    c_cites = cite(rules, r"/\* :(\d+(?:-\d+)?) \*/")
    go_cites = sorted(a or b for a, b in re.findall(r"// :(\d+(?:-\d+)?)[ \t]*\n|// :(\d+(?:-\d+)?)$", go_rules, flags=re.M))
    assert len(c_cites) > 80
    assert go_cites == c_cites, (sorted(set(c_cites) - set(go_cites)), sorted(set(go_cites) - set(c_cites)))
    # and the same operators in the same order, statement by statement, for the Adam element
    c_adam = c_text[c_text.index("static inline void adam_element"):c_text.index("/* bridge_optimizer.m:360-641 */")]
    go_adam = go_text[go_text.index("func adamElement"):go_text.index("// OracleAdamStep")]
    ops = lambda text, marker: re.findall(r"= [^;\n]*?([*/+-])[^;\n]*?" + marker, text)
    assert ops(c_adam, r";\s*/\* :") == ops(go_adam, r"\)\s*// :") and len(ops(c_adam, r";\s*/\* :")) >= 12
