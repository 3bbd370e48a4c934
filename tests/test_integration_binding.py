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


def test_a_handle_dropped_before_its_collective_ran_leaves_its_tensors_with_the_engine(monkeypatch):
    """The binding's handle keeps the tensors alive (the C ABI has only addresses). Dropped without a wait while the
    collective has not run, it parks (work, tensors) on its engine, which frees the work and lets go of the tensors
    once the collective is done: at the next call, or in close(). A handle that was waited for, or whose collective
    has finished, is freed at once. The reference's engine holds its tensor until the job has run
    (tandem/csrc/collectives.cpp:314-324). The library is replaced by a recorder here; tests/test_gpu_integration.py
    drops a handle on the GPU."""
    from tandem_amd import hip_engine

    class Recorder:
        def __init__(self):
            self.done, self.freed, self.closed = set(), [], []

        def tdm_work_done(self, p):
            return int(p in self.done)

        def tdm_work_free(self, p):
            self.freed.append(p)

        def tdm_work_wait(self, p, stream):
            return 0

        def tdm_engine_close(self, e):
            self.closed.append(e)
            return 0

        def tdm_engine_destroy(self, e):
            pass

        def tdm_barrier(self, e, out):
            return 0

    lib = Recorder()
    monkeypatch.setattr(hip_engine, "_L", lib)
    monkeypatch.setattr(hip_engine, "_stream", lambda device: None)
    engine = hip_engine.Engine.__new__(hip_engine.Engine)
    engine._e, engine._device, engine._orphans = "engine", None, []
    tensor = object()
    hip_engine.Handle("w1", None, (tensor,), engine)  # dropped at once, not run, never waited for
    assert engine._orphans == [("w1", (tensor,))] and lib.freed == []
    waited = hip_engine.Handle("w2", None, (tensor,), engine)
    waited.wait()
    del waited
    finished = hip_engine.Handle("w3", None, (tensor,), engine)
    lib.done.add("w3")
    del finished
    hip_engine.Handle("w4", None, (), engine)  # a barrier's handle keeps nothing alive
    assert lib.freed == ["w2", "w3", "w4"] and len(engine._orphans) == 1
    engine.barrier()  # w1 still not done: stays parked
    assert len(engine._orphans) == 1
    lib.done.add("w1")
    h = engine.barrier()
    assert engine._orphans == [] and "w1" in lib.freed
    del h
    hip_engine.Handle("w5", None, (tensor,), engine)
    assert [p for p, _ in engine._orphans] == ["w5"]
    engine.close()  # close runs what is queued, then frees what was parked
    assert lib.closed == ["engine"] and "w5" in lib.freed and engine._orphans == []
