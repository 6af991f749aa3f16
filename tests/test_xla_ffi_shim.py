"""The XLA FFI binding (gla_jax_amd/xla_ffi) cannot be compiled or run without jaxlib, which neither the build
machine nor the GPU box has.  What can be held here: the handler source calls only entry points that
include/gla_hip.h declares, with the declared number of arguments; the Python side registers exactly the
handlers the source defines, with as many operands and results as each handler binds; and the module refuses
to import without jax instead of degrading."""
import ast
import importlib
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CC = os.path.join(ROOT, "gla_jax_amd", "xla_ffi", "gla_xla_ffi.cc")
PY = os.path.join(ROOT, "gla_jax_amd", "xla_ffi", "gla_jax.py")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _call_args(text, start):
    """Number of top-level comma-separated arguments of the call whose '(' is at text[start]."""
    depth, n, i, seen = 0, 0, start, False
    while True:
        ch = text[i]
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
            if depth == 0:
                return n + (1 if seen else 0)
        elif ch == "," and depth == 1:
            n += 1
        elif depth >= 1 and not ch.isspace():
            seen = True
        i += 1


def declared():
    text = _strip_comments(open(os.path.join(ROOT, "include", "gla_hip.h")).read())
    out = {}
    for m in re.finditer(r"\b(gla_[a-z0-9_]+)\s*\(", text):
        n = _call_args(text, m.end() - 1)
        args = text[m.end():text.index(")", m.end())].strip()
        out[m.group(1)] = 0 if args == "void" else n
    return out


def test_handlers_call_the_c_abi_as_declared():
    decl = declared()
    text = _strip_comments(open(CC).read())
    calls = [(m.group(1), _call_args(text, m.end() - 1)) for m in re.finditer(r"\b(gla_[a-z0-9_]+)\s*\(", text)]
    used = {n for n, _ in calls}
    assert {"gla_chunk_fwd", "gla_chunk_bwd", "gla_recurrent_fwd_ws", "gla_recurrent_bwd_ws", "gla_cumsum_f32",
            "gla_rnn_scan_f32", "gla_status_string"} <= used
    for name, nargs in calls:
        assert name in decl, f"{name} is not declared in include/gla_hip.h"
        assert nargs == decl[name], f"{name}: called with {nargs} arguments, declared with {decl[name]}"


def bindings():
    """handler symbol -> (number of .Arg, number of .Ret, attribute names) from the source."""
    text = _strip_comments(open(CC).read())
    out = {}
    for m in re.finditer(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)\s*,\s*(\w+)\s*,(.*?)\);\s*(?=XLA_FFI|\Z)", text, flags=re.S):
        body = m.group(3)
        out[m.group(1)] = (body.count(".Arg<"), body.count(".Ret<"), re.findall(r'\.Attr<[^>]+>\("(\w+)"\)', body))
    return out


def test_python_side_matches_the_handlers():
    b = bindings()
    assert set(b) == {"GlaChunkFwd", "GlaChunkBwd", "GlaRecurrentFwd", "GlaRecurrentBwd", "GlaCumsum", "GlaRnnScan"}
    tree = ast.parse(open(PY).read())
    registered = None
    calls = {}
    for node in ast.walk(tree):
        if isinstance(node, ast.For) and isinstance(node.iter, ast.Tuple) and all(
                isinstance(e, ast.Constant) and str(e.value).startswith("Gla") for e in node.iter.elts):
            registered = {e.value for e in node.iter.elts}
        # jax.ffi.ffi_call("Name", results, ...)(operands..., attr=...)
        if isinstance(node, ast.Call) and isinstance(node.func, ast.Call):
            inner = node.func
            if isinstance(inner.func, ast.Attribute) and inner.func.attr == "ffi_call":
                name = inner.args[0].value
                res = inner.args[1]
                n_res = len(res.elts) if isinstance(res, ast.Tuple) else 1
                calls[name] = (len(node.args), n_res, sorted(k.arg for k in node.keywords))
    assert registered == set(b)
    assert set(calls) == set(b)
    for name, (n_arg, n_ret, attrs) in b.items():
        assert calls[name] == (n_arg, n_ret, sorted(attrs)), f"{name}: python passes {calls[name]}, handler binds {(n_arg, n_ret, sorted(attrs))}"


def test_module_refuses_to_import_without_jax():
    if importlib.util.find_spec("jax") is not None:
        pytest.skip("jax is installed here")
    with pytest.raises(ImportError, match="jax"):
        importlib.import_module("gla_jax_amd.xla_ffi.gla_jax")
    from gla_jax_amd import build
    assert build.jaxlib_include() is None and build.build_xla_ffi(verbose=False) is None


# The reference's public signatures (gla.py:657-669, 405-416, 26; ops.py:234-240, 396-403): name -> list of
# (parameter, default or REQUIRED), in order.
REQUIRED = object()
REFERENCE_SIGNATURES = {
    "chunk_gla": [("hidden_init", REQUIRED), ("log_fgate", REQUIRED), ("value", REQUIRED), ("key", REQUIRED),
                  ("query", REQUIRED), ("chunk_size", REQUIRED), ("block_size_t", 64), ("block_size_d", 64),
                  ("interpret", False), ("num_warps", 4), ("num_stages", 2)],
    "recurrent_gla": [("hidden_init", REQUIRED), ("log_fgate", REQUIRED), ("value", REQUIRED), ("key", REQUIRED),
                      ("query", REQUIRED), ("reverse", False), ("max_block_size", 64), ("num_warps", 1),
                      ("num_stages", 1), ("interpret", False)],
    "recurrent_gla_naive": [("hidden", REQUIRED), ("log_fgate", REQUIRED), ("value", REQUIRED), ("key", REQUIRED),
                            ("query", REQUIRED), ("reverse", REQUIRED)],
    "cumsum_recursive": [("src", REQUIRED), ("axis", REQUIRED), ("init", None), ("reverse", False),
                         ("block_size_t", 2048)],
    "rnn_recursive": [("log_fgate", REQUIRED), ("kv", REQUIRED), ("init_log_fgate", None), ("init_kv", None),
                      ("block_size_t", 256), ("reverse", False)],
}


def _parsed_signatures(path):
    """name -> [(parameter, default or REQUIRED)] of every top-level public function, from the source text."""
    out = {}
    for node in ast.parse(open(path).read()).body:
        if isinstance(node, ast.FunctionDef) and not node.name.startswith("_"):
            a = node.args
            assert not a.posonlyargs and not a.kwonlyargs and a.vararg is None and a.kwarg is None
            names = [x.arg for x in a.args]
            defaults = [REQUIRED] * (len(names) - len(a.defaults)) + [ast.literal_eval(d) for d in a.defaults]
            out[node.name] = list(zip(names, defaults))
    return out


def test_public_signatures_are_the_reference_ones_in_both_front_ends():
    """Every public function of the JAX module (parsed, it cannot be imported here) and of the torch front-end
    (inspect.signature) takes the reference's parameters, in the reference's order, with the reference's
    defaults: a positional call written for the reference means the same thing in both."""
    import inspect

    from gla_jax_amd import gla, ops
    jax_side = _parsed_signatures(PY)
    for name, want in REFERENCE_SIGNATURES.items():
        assert jax_side.get(name) == want, f"xla_ffi/gla_jax.py::{name}: {jax_side.get(name)}"
        fn = getattr(gla, name, None) or getattr(ops, name)
        got = [(p.name, REQUIRED if p.default is inspect.Parameter.empty else p.default)
               for p in inspect.signature(fn).parameters.values()]
        assert got == want, f"torch front-end {name}: {got}"
    # nothing public in the JAX module beyond those and the two custom_vjp functions of the reference
    assert set(jax_side) - set(REFERENCE_SIGNATURES) <= {"chunk_gla_forward_backward",
                                                         "recurrent_gla_forward_backward"}
