"""The stand-in for the reference's compiled extension against the reference's own call sites, read as text.

`wall_x/fusions/backend.py` is the only importer of the extension (`import wallx_csrc as backend`, backend.py:13).
When the reference tree is present, its source is parsed (never imported or executed) and every `backend.<name>(...)`
call is checked against the signature of the same name in this repository's `wallx_csrc` module: the name exists, the
call's positional arguments bind, and no keyword is used that the stand-in lacks.  The same walk over
`wall_x/fusions/ops.py` checks its `backend.<name>(...)` calls against `wallx_mi355.fusions.backend`."""

import ast
import inspect
import os

import pytest

import wallx_csrc
from wallx_mi355.fusions import backend as our_backend

REF = "/root/reference/wall_x/fusions"

pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not present on this machine")


def _calls(path, receiver):
    tree = ast.parse(open(path).read())
    out = []
    for node in ast.walk(tree):
        if isinstance(node, ast.Call) and isinstance(node.func, ast.Attribute) and \
                isinstance(node.func.value, ast.Name) and node.func.value.id == receiver:
            assert not any(isinstance(a, ast.Starred) for a in node.args), "a starred call cannot be counted"
            out.append((node.func.attr, len(node.args), [k.arg for k in node.keywords], node.lineno))
    return out


def _binds(fn, n_positional, keywords):
    sig = inspect.signature(fn)
    sig.bind(*([None] * n_positional), **{k: None for k in keywords})  # raises TypeError when the call would not bind


def test_every_native_call_site_of_the_reference_binds_to_the_stand_in():
    calls = _calls(os.path.join(REF, "backend.py"), "backend")
    names = {name for name, *_ in calls}
    assert names == set(wallx_csrc.__all__), f"call sites {sorted(names)} vs exported {sorted(wallx_csrc.__all__)}"
    for name, n_pos, keywords, line in calls:
        try:
            _binds(getattr(wallx_csrc, name), n_pos, keywords)
        except TypeError as exc:
            raise AssertionError(f"backend.py:{line}: backend.{name} with {n_pos} positional arguments and keywords "
                                 f"{keywords} does not bind: {exc}")
    # the positional counts the reference uses today (csrc/*.h): a change on either side shows here
    assert {name: n for name, n, _, _ in calls} == {
        "asym_dual_gmm": 8, "permute": 5, "unpermute": 5, "unpermute_bwd": 4, "rope": 7, "rope_bwd": 9,
        "rope_index": 10, "rot_pos_emb": 3, "get_window_index": 5}


def test_every_backend_call_of_the_reference_ops_binds_to_this_backend():
    calls = _calls(os.path.join(REF, "ops.py"), "backend")
    assert calls
    for name, n_pos, keywords, line in calls:
        fn = getattr(our_backend, name, None)
        assert fn is not None, f"ops.py:{line}: backend.{name} has no counterpart"
        try:
            _binds(fn, n_pos, keywords)
        except TypeError as exc:
            raise AssertionError(f"ops.py:{line}: backend.{name} does not bind: {exc}")
