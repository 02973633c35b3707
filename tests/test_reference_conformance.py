"""Static conformance of the lane's plug-in code with the host it plugs into.

`tessera_amd.install.install()` registers candidates, execution-matrix rows, executor
functions and a native launcher into objects the host owns, and the GPU tests exercise those
seams against `tests/standin_host.py`, a small host written for the tests.  This file makes
sure the stand-in and the lane cannot drift from the real host unnoticed: it PARSES the
host's source files (`ast`, nothing is imported or executed) and asserts every name,
attribute and parameter the lane relies on.  CPU only; skipped where the host's checkout
is not mounted.
"""
import ast
import dataclasses
import inspect
from pathlib import Path

import pytest

from tessera_amd import candidates, executors, native_launcher

HOST = Path("/root/reference/python/tessera")
pytestmark = pytest.mark.skipif(not HOST.is_dir(), reason="the host's source checkout is not mounted")


def _module(rel):
    return ast.parse((HOST / rel).read_text())


def _top(tree, kind, name):
    for node in tree.body:
        if isinstance(node, kind) and getattr(node, "name", None) == name:
            return node
    raise AssertionError(f"{name} not found")


def _assigned_names(tree):
    out = set()
    for node in tree.body:
        targets = node.targets if isinstance(node, ast.Assign) else [node.target] if isinstance(node, ast.AnnAssign) else []
        out.update(t.id for t in targets if isinstance(t, ast.Name))
    return out


def _class_attrs(cls):
    attrs, methods = set(), {}
    for node in cls.body:
        if isinstance(node, ast.AnnAssign) and isinstance(node.target, ast.Name):
            attrs.add(node.target.id)
        elif isinstance(node, ast.Assign):
            attrs.update(t.id for t in node.targets if isinstance(t, ast.Name))
        elif isinstance(node, ast.FunctionDef):
            methods[node.name] = node
    return attrs, methods


def _params(fn):
    a = fn.args
    return [p.arg for p in a.posonlyargs + a.args], [p.arg for p in a.kwonlyargs], a.vararg and a.vararg.arg


def test_candidate_module_has_what_the_candidates_use():
    tree = _module("compiler/emit/candidate.py")
    names = _assigned_names(tree)
    # op tags the candidate classes read from the host API by attribute
    for cls_name, op_ref, attrs in candidates._SPECS:
        if isinstance(op_ref, str) and op_ref.startswith("OP_"):
            assert op_ref in names, op_ref
    tier = _top(tree, ast.ClassDef, "Tier")
    assert "HAND_TUNED" in _class_attrs(tier)[0]
    cand = _top(tree, ast.ClassDef, "Candidate")
    attrs, methods = _class_attrs(cand)
    # every class attribute / method the lane's candidates set must exist on the base class
    set_by_lane = {"target", "tier", "accuracy_atol", "available", "op"}
    for _, _, body in candidates._SPECS:
        set_by_lane.update(k for k in body if not k.startswith("__"))
    missing = set_by_lane - attrs - set(methods)
    assert not missing, f"Candidate has no {sorted(missing)}"
    # call shapes the arbiter uses on a candidate
    assert _params(methods["available"])[0] == ["self"]
    assert _params(methods["applies_to"])[0] == ["self", "region"]
    pos, kwonly, var = _params(methods["run"])
    assert pos == ["self", "region"] and var == "inputs"
    pos, kwonly, var = _params(methods["measure_device_latency"])
    assert pos == ["self", "region"] and var == "inputs" and {"reps", "warmup"} <= set(kwonly)
    assert _params(methods["mma_dtype"])[0] == ["self", "region"]
    # the lane's own methods take what the base class's take
    for _, _, body in candidates._SPECS:
        for meth in ("applies_to", "run", "measure_device_latency", "mma_dtype"):
            fn = body.get(meth)
            if callable(fn):
                got = list(inspect.signature(fn).parameters)
                assert got[:2] == ["self", "region"], (meth, got)


def test_registry_and_arbiter_signatures():
    tree = _module("compiler/emit/candidate.py")
    assert _params(_top(tree, ast.FunctionDef, "register_op_kind"))[0] == ["op", "verify_fn"]
    assert _params(_top(tree, ast.FunctionDef, "register_candidate"))[0] == ["candidate"]
    assert _params(_top(tree, ast.FunctionDef, "candidates_for"))[0] == ["target", "op"]
    pos, kwonly, _ = _params(_top(tree, ast.FunctionDef, "arbitrate"))
    assert pos == ["region", "op", "target"] and kwonly == ["verify", "force", "measure"]
    pos, kwonly, var = _params(_top(tree, ast.FunctionDef, "run_arbitrated"))
    assert pos == ["region", "op", "target"] and var == "inputs" and {"verify", "force", "measure"} <= set(kwonly)
    # the stand-in host the GPU tests register into exposes the same entry points
    import standin_host
    host = standin_host.CandidateHost()
    for fn, want in (("register_op_kind", ["op", "verify_fn"]), ("register_candidate", None),
                     ("candidates_for", ["target", "op"])):
        got = list(inspect.signature(getattr(host, fn)).parameters)
        if want is not None:
            assert got == want, (fn, got)
    sig = inspect.signature(host.arbitrate)
    kw = [n for n, p in sig.parameters.items() if p.kind is p.KEYWORD_ONLY]
    assert list(sig.parameters)[:3] == ["region", "op", "target"] and kw == ["verify", "force", "measure"]
    base_attrs, base_methods = _class_attrs(_top(tree, ast.ClassDef, "Candidate"))
    for name in base_attrs | set(base_methods):
        if not name.startswith("_"):
            assert hasattr(standin_host.Candidate, name), f"stand-in Candidate lacks {name}"


def test_execution_row_fields_and_tables():
    tree = _module("compiler/execution_matrix.py")
    row = _top(tree, ast.ClassDef, "ExecutionRow")
    fields, required = [], []
    for node in row.body:
        if isinstance(node, ast.AnnAssign) and isinstance(node.target, ast.Name):
            fields.append(node.target.id)
            if node.value is None:
                required.append(node.target.id)
    for f in executors.ROW_FIELDS:
        assert set(f) <= set(fields), f"row fields the host does not have: {sorted(set(f) - set(fields))}"
        assert set(required) <= set(f), f"row lacks required fields {sorted(set(required) - set(f))}"
    # the lane's own row class (used by its stand-alone launch) has the host's leading fields in order
    own = [f.name for f in dataclasses.fields(executors.ExecutionRow)]
    assert own == fields[:len(own)]
    names = _assigned_names(tree)
    assert {"_MATRIX", "KNOWN_EXECUTORS"} <= names
    assert _params(_top(tree, ast.FunctionDef, "lookup"))[0] == ["target", "compiler_path"]
    # every row names an executor the lane provides and documents
    table = executors.executor_table()
    for f in executors.ROW_FIELDS:
        assert f["executor_id"] in table and f["executor_id"] in executors.KNOWN_EXECUTORS


def test_runtime_seams():
    tree = _module("runtime.py")
    table = _top(tree, ast.FunctionDef, "_executor_table")
    assert _params(table) == ([], [], None)          # install wraps a zero-argument function
    pos, kwonly, _ = _params(_top(tree, ast.FunctionDef, "launch"))
    assert pos[:2] == ["kernel", "args"]
    pos, kwonly, _ = _params(_top(tree, ast.FunctionDef, "register_native_launcher"))
    assert pos == ["target"] and kwonly == ["binary_formats", "submit", "replace"]
    # the hook the lane registers takes the five things the host submits
    assert len(inspect.signature(native_launcher.submit).parameters) == 5
    art = _top(tree, ast.ClassDef, "RuntimeArtifact")
    host_fields = _class_attrs(art)[0]
    own = {f.name for f in dataclasses.fields(executors.RuntimeArtifact)}
    assert own <= host_fields, sorted(own - host_fields)
    # an executor is called as executor(artifact, args)
    for fn in executors.executor_table().values():
        assert list(inspect.signature(fn).parameters)[:2] == ["artifact", "args"]
