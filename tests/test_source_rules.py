"""Rules the kernel sources keep, checked on their text (no GPU, no compiler).

A memory instruction inside an `asm` statement is opaque to the compiler's hazard
recogniser: a store of more than 64 bits followed by a vector write of the registers
that held its data needs wait states between the two, and the compiler inserts them
only for stores it emitted itself. A hand-written `global_store_dwordx4 ... sc1` in
the GEMM epilogue once lost a float4 of a product now and then for exactly that
reason. Every load and store of the kernels therefore comes from a builtin or plain
C++, and the only `asm` statements allowed are empty ones (argument pinning)."""
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tfjs_amd", "csrc")

ASM = re.compile(r"\b(?:asm|__asm__|__asm)\b\s*(?:volatile|__volatile__)?\s*\(")
STRING = re.compile(r'"((?:[^"\\]|\\.)*)"')
MEMORY_WORDS = ("store", "load", "global_", "buffer_", "ds_", "flat_", "scratch_", "atomic")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", lambda m: "\n" * m.group(0).count("\n"), text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _asm_statements(text):
    """(line, instruction template) of every asm statement: the string literals that
    precede the first colon (or the closing parenthesis) of the statement."""
    out = []
    for m in ASM.finditer(text):
        depth, i = 1, m.end()
        while i < len(text) and depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        body = text[m.end():i - 1]
        head, in_string, k = [], False, 0
        while k < len(body):                     # cut at the first ':' outside a string literal
            ch = body[k]
            if ch == "\\" and in_string:
                k += 1
            elif ch == '"':
                in_string = not in_string
            elif ch == ":" and not in_string:
                break
            k += 1
        template = "".join(STRING.findall(body[:k]))
        out.append((text.count("\n", 0, m.start()) + 1, template))
    return out


def _sources():
    files = sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.h")) +
                   glob.glob(os.path.join(CSRC, "*.cc")))
    assert len(files) >= 15
    return files


def test_no_asm_statement_carries_an_instruction():
    seen = 0
    for path in _sources():
        for line, template in _asm_statements(_strip_comments(open(path).read())):
            seen += 1
            where = "%s:%d" % (os.path.relpath(path, ROOT), line)
            assert template.strip() == "", "%s: asm with an instruction template %r; use a builtin" % (where, template)
            assert not any(w in template for w in MEMORY_WORDS), where
    assert seen >= 1, "the argument-pinning asm of gemm_kernel.h was expected"


def test_the_checker_sees_what_it_is_meant_to_refuse():
    bad = 'void f() { asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory"); }'
    (line, template), = _asm_statements(_strip_comments(bad))
    assert line == 1 and "global_store_dwordx4" in template and any(w in template for w in MEMORY_WORDS)
    ok = '// asm("ds_read_b32") in a comment\nvoid g() { asm volatile("" ::"s"(x)); }'
    assert _asm_statements(_strip_comments(ok)) == [(2, "")]
    two = 'void h() { __asm__ __volatile__("s_nop 0\\n" "s_nop 1" ::: "memory"); }'
    assert _asm_statements(_strip_comments(two))[0][1] == "s_nop 0\\ns_nop 1"
