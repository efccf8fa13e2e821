"""The C-ABI library loads and exports every function include/ccfuser_moe.h declares;
argument checks that need no GPU return error codes instead of crashing."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ccfuser_moe.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ccf_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from ccfuser_amd import _lib
    if not _lib.LIB_PATH.exists():
        from ccfuser_amd import build
        build.build(verbose=False)
    return _lib.lib()


def test_header_and_binding_agree(lib):
    from ccfuser_amd import _lib
    names = declared_functions()
    assert len(names) >= 18
    assert set(names) == set(_lib.SIGNATURES), "binding table and header differ"
    for n in names:
        assert hasattr(lib, n), f"{n} is declared but not exported"


def test_every_declaration_cites_the_reference_or_says_it_has_none():
    text = open(HEADER).read()
    blocks = re.findall(r"/\*(.*?)\*/\s*(?:int|size_t|const char \*)\s*(ccf_[a-z0-9_]+)\s*\(", text, flags=re.S)
    assert blocks
    for comment, name in blocks:
        ok = ("mix_moe/" in comment) or ("no counterpart" in comment) or name in (
            "ccf_version", "ccf_last_error", "ccf_route_workspace_bytes", "ccf_ffn_workspace_bytes",
            "ccf_moe_workspace_bytes", "ccf_segments_workspace_bytes")
        assert ok, f"{name}: declaration comment names no reference interface"


def _split_args(text, start):
    """Arguments of the call whose opening parenthesis is at text[start]: split at top-level commas."""
    depth, args, cur = 0, [], []
    for ch in text[start:]:
        if ch in "([{":
            depth += 1
            if depth == 1:
                continue
        elif ch in ")]}":
            depth -= 1
            if depth == 0:
                break
        if ch == "," and depth == 1:
            args.append("".join(cur).strip())
            cur = []
        else:
            cur.append(ch)
    last = "".join(cur).strip()
    if last and last != "void":
        args.append(last)
    return args


def header_arity():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return {m.group(1): len(_split_args(text, m.end() - 1)) for m in re.finditer(r"\b(ccf_[a-z0-9_]+)\s*\(", text)}


def test_integration_guide_calls_match_the_header():
    """Every ccf_*( call inside a code block of INTEGRATION.md passes as many arguments as the
    header declares for that function, so the guide's snippets cannot drift from the ABI."""
    arity = header_arity()
    guide = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```(?:cpp|c)\n(.*?)```", guide, flags=re.S)
    assert blocks, "no C/C++ code block found in INTEGRATION.md"
    seen = 0
    for code in blocks:
        code = re.sub(r"/\*.*?\*/", "", code, flags=re.S)
        code = re.sub(r"//[^\n]*", "", code)
        for m in re.finditer(r"\b(ccf_[a-z0-9_]+)\s*\(", code):
            name = m.group(1)
            assert name in arity, f"INTEGRATION.md calls {name}, which the header does not declare"
            got = len(_split_args(code, m.end() - 1))
            assert got == arity[name], f"INTEGRATION.md passes {got} arguments to {name}; the header declares {arity[name]}"
            seen += 1
    assert seen >= 4


def test_version_and_sizes(lib):
    assert lib.ccf_version() >= 100
    assert lib.ccf_route_workspace_bytes(32768, 32) > 0
    assert lib.ccf_ffn_workspace_bytes(8192, 8, 4096, 14336) > 0
    need = lib.ccf_moe_workspace_bytes(4096, 4096, 14336, 8, 2)
    # dominated by h [8192, 14336] and y_flat [8192, 4096] in fp16, plus 64 MiB of fp32 partial
    # tiles for the split last round of the grouped GEMMs and 64 MiB for skinny tiles cut along K
    assert 8192 * (14336 + 4096) * 2 + (128 << 20) <= need <= 8192 * (14336 + 4096) * 2 + (128 << 20) + (1 << 21)
    assert lib.ccf_moe_workspace_bytes(-1, 64, 64, 2, 1) == 0


def test_argument_errors_are_codes_not_crashes(lib):
    # null pointers and bad sizes are rejected before anything touches the GPU
    rc = lib.ccf_gate_topk_softmax(None, None, None, 4, 64, 4, 2, 0, None, None, None, None)
    assert rc == 1 and b"null" in lib.ccf_last_error()
    rc = lib.ccf_set_option(b"gemm_variant", 999)
    assert rc == 1
    rc = lib.ccf_set_option(b"no_such_option", 0)
    assert rc == 1 and b"unknown option" in lib.ccf_last_error()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    rc = lib.ccf_gate_topk_softmax(p, p, None, 4, 60, 4, 2, 0, p, p, None, None)
    assert rc == 2 and b"multiple of 8" in lib.ccf_last_error()
    rc = lib.ccf_combine(p, p, None, p, 4, 9, 64, None)
    assert rc == 2
    rc = lib.ccf_ffn1_forward(p, None, None, p, 8, 2, 64, 64, p, p, 1, p, None, 0, None)
    assert rc == 3 and b"workspace" in lib.ccf_last_error()
    rc = lib.ccf_moe_forward(p, p, p, p, p, p, p, 4, 64, 64, 2, 1, -1, p, None, None, None, None,
                             None, p, 16, None)
    assert rc == 3
    # backward entry points and the block planner
    assert lib.ccf_ffn_backward_workspace_bytes(8192, 8, 4096, 14336) > 8 * 4096 * 14336 * 2
    assert lib.ccf_ffn_backward_workspace_bytes(8192, 0, 4096, 14336) == 0
    rc = lib.ccf_ffn2_backward(None, p, None, None, p, 8, 2, 64, 64, p, p, p, p, p, 1 << 30, None)
    assert rc == 1 and b"null" in lib.ccf_last_error()
    rc = lib.ccf_ffn2_backward(p, p, None, None, p, 8, 2, 64, 96, p, p, p, p, p, 1 << 30, None)
    assert rc == 2 and b"multiples of 64" in lib.ccf_last_error()
    rc = lib.ccf_ffn1_backward(p, p, None, None, p, 8, 2, 64, 64, p, p, p, p, p, 16, None)
    assert rc == 3 and b"workspace" in lib.ccf_last_error()
    rc = lib.ccf_ffn1_forward_keep(p, None, p, 8, 2, 64, 64, p, p, None, p, p, 1 << 30, None)
    assert rc == 1
    rc = lib.ccf_combine_backward(p, p, p, None, 4, 2, 60, p, p, None)
    assert rc == 2
    rc = lib.ccf_plan_blocks(p, 2000, 64, 0, 8, p, p, p, p, p, p, p, None)
    assert rc == 2 and b"exceeds" in lib.ccf_last_error()
    rc = lib.ccf_plan_blocks(None, 4, 64, 0, 8, p, p, p, p, p, p, p, None)
    assert rc == 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from ccfuser_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libccfuser_moe.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()
