"""The integration notes at the repository root quote tandem_amd/hip_engine.py, the binding a tandem
maintainer would copy into the reference tree: the quotation and the file must be the same text, and the file must
offer what the reference's Group calls on its native engine (tandem/comm.py:149-160,326-452 and
the pybind surface tandem/csrc/engine.cpp:103-122 there)."""

import ast
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def quoted_block():
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    section = text[text.index("## 2. The binding"):text.index("## 3. The patch")]
    start = section.index("```python\n") + len("```python\n")
    return section[start:section.rindex("```")]


def test_the_document_quotes_the_file_verbatim():
    assert quoted_block() == open(os.path.join(ROOT, "tandem_amd", "hip_engine.py")).read()


def test_the_binding_has_the_surface_the_reference_calls():
    tree = ast.parse(open(os.path.join(ROOT, "tandem_amd", "hip_engine.py")).read())
    classes = {n.name: n for n in tree.body if isinstance(n, ast.ClassDef)}
    def methods(cls):
        return {f.name: [a.arg for a in f.args.args] for f in classes[cls].body if isinstance(f, ast.FunctionDef)}
    engine = methods("Engine")
    assert engine["__init__"] == ["self", "job", "rank", "size", "slots", "slot_bytes", "timeout", "device"]
    want = {"connect": ["self"], "close": ["self"], "all_reduce": ["self", "t", "average"],
            "reduce_scatter": ["self", "t", "sizes", "average"], "all_gather": ["self", "t", "sizes"],
            "broadcast": ["self", "t", "root"], "send": ["self", "t", "dst"], "recv": ["self", "t", "src"],
            "sendrecv": ["self", "send", "dst", "recv", "src"], "barrier": ["self"]}
    for name, args in want.items():
        assert engine[name] == args, name
    handle = methods("Handle")
    assert {"wait", "done"} <= set(handle)
    source = open(os.path.join(ROOT, "tandem_amd", "hip_engine.py")).read()
    assert "started = property" in source and "finished = property" in source and "\ncuda = True" in source
    # every entry point it binds is declared in the header
    header = open(os.path.join(ROOT, "include", "tandem_hip.h")).read()
    import re
    for sym in set(re.findall(r"\btdm_[a-z0-9_]+", source)):
        assert re.search(rf"\b{sym}\s*\(", header), sym
