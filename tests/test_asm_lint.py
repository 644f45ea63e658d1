"""A source check of the inline assembly in the HIP kernels (runs on the CPU, reads the sources only).

The compiler takes the outputs of an asm statement as valid the moment the statement ends.  A vector-memory load that
is still in flight behind its own statement can therefore find its destination registers copied, or handed to
something else (an address), before the data lands: wrong data at best, a wild address at worst.  The rule the kernels
follow, and this test enforces for every `asm volatile` statement under csrc/: a statement that loads from memory into
registers waits for its loads itself (`s_waitcnt` with a vmcnt field in the same statement) and marks every register
output early-clobber (`=&v`), so that no address operand shares a register with a destination.
"""
import re
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "flashsvd_amd" / "csrc"
LOAD = re.compile(r"\b(global|flat|buffer|scratch)_load_(?!lds)\w+")     # loads into registers (not the LDS-direct forms)


def _asm_statements(text: str):
    """(line number, text between the parentheses) of every `asm volatile( ... )` statement."""
    for m in re.finditer(r"\basm\s+volatile\s*\(", text):
        depth, i, in_str = 1, m.end(), False
        while i < len(text) and depth:
            c = text[i]
            if in_str:
                if c == "\\":
                    i += 1
                elif c == '"':
                    in_str = False
            elif c == '"':
                in_str = True
            elif c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
            i += 1
        yield text.count("\n", 0, m.start()) + 1, text[m.end():i - 1]


def _string_macros(text: str) -> dict:
    return {m.group(1): m.group(2) for m in re.finditer(r'^\s*#\s*define\s+(\w+)\s+("(?:[^"\\]|\\.)*")\s*$', text, re.M)}


def check_source(text: str, name: str = "<text>") -> list:
    problems = []
    macros = _string_macros(text)
    for line, body in _asm_statements(text):
        for k, v in macros.items():
            body = re.sub(rf"\b{k}\b", v, body)
        template = body.split(":", 1)[0]
        code = "".join(re.findall(r'"((?:[^"\\]|\\.)*)"', template))
        if not LOAD.search(code):
            continue
        if not re.search(r"s_waitcnt[^\\]*vmcnt\(", code):
            problems.append(f"{name}:{line}: a load without an s_waitcnt vmcnt(...) in the same asm statement")
        outputs = body.split(":")[1] if body.count(":") >= 1 else ""
        for cons in re.findall(r'"(=[^"]*)"', outputs):
            if "v" in cons and "&" not in cons:
                problems.append(f"{name}:{line}: register output {cons!r} of a load is not early-clobber")
    return problems


def test_every_inline_load_waits_for_itself():
    sources = sorted([*CSRC.glob("*.hip"), *CSRC.glob("*.hpp")])
    assert sources, f"no sources under {CSRC}"
    problems = []
    n_loads = 0
    for src in sources:
        text = src.read_text()
        problems += check_source(text, src.name)
        macros = _string_macros(text)
        for _, body in _asm_statements(text):
            for k, v in macros.items():
                body = re.sub(rf"\b{k}\b", v, body)
            n_loads += bool(LOAD.search(body))
    assert not problems, "\n".join(problems)
    assert n_loads >= 3, "the check no longer finds the coherent-load statements of the step kernel: has their form changed?"


def test_the_check_catches_the_two_mistakes():
    bad_wait = 'asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=&v"(v) : "v"(a) : "memory");'
    bad_clobber = 'asm volatile("global_load_dwordx4 %0, %1, off\\n\\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(a) : "memory");'
    good = '#define L "global_load_dwordx4 %"\nasm volatile(L "0, %1, off\\n\\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(a) : "memory");'
    lds = 'asm volatile("global_load_lds_dwordx4 %0, off" :: "v"(a) : "memory");'
    assert len(check_source(bad_wait)) == 1 and "s_waitcnt" in check_source(bad_wait)[0]
    assert len(check_source(bad_clobber)) == 1 and "early-clobber" in check_source(bad_clobber)[0]
    assert check_source(good) == [] and check_source(lds) == []
    assert check_source('#define L "global_load_dwordx4 %"\nasm volatile(L "0, %1, off" : "=&v"(v) : "v"(a));') != []
