"""The JAX front end (gpu_ragged_dot_amd/jax_adapter.py + csrc/rd_xla_ffi.cc) cannot be imported or compiled in an
image without JAX.  What can be checked on the CPU: the Python parses and mirrors the reference's surface
(gpu_ragged_dot.py:347-428: names, positional order, defaults, static-argument positions, the custom_vjp wiring), and the
handlers pass their arguments to rd_gmm / rd_tgmm in the order include/ragged_dot_hip.h declares."""

import ast
import inspect
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ADAPTER = os.path.join(ROOT, "gpu_ragged_dot_amd", "jax_adapter.py")
SHIM = os.path.join(ROOT, "gpu_ragged_dot_amd", "csrc", "rd_xla_ffi.cc")
HEADER = os.path.join(ROOT, "include", "ragged_dot_hip.h")

GMM_PARAMS = ["x", "A", "group_sizes", "block_m", "block_k", "block_n", "trans_rhs", "interpret", "compute_dtype",
              "acc_dtype", "num_warps", "num_stages", "chunk_m"]  # gpu_ragged_dot.py:362-376
TGMM_PARAMS = ["x", "y", "group_sizes", "block_m", "block_k", "block_n", "interpret", "compute_dtype", "acc_dtype",
               "num_warps", "num_stages", "chunk_m"]  # gpu_ragged_dot.py:411-424


def _tree():
    with open(ADAPTER) as f:
        return ast.parse(f.read())


def _func(tree, name):
    return next(n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == name)


def _decorator_sources(fn):
    return [ast.unparse(d) for d in fn.decorator_list]


def test_adapter_parses_and_mirrors_the_reference_surface():
    tree = _tree()
    gmm, tgmm = _func(tree, "gmm"), _func(tree, "tgmm")
    assert [a.arg for a in gmm.args.args] == GMM_PARAMS
    assert [a.arg for a in tgmm.args.args] == TGMM_PARAMS
    # hyper-parameters are static under jit and non-differentiable under custom_vjp (:360-361, :409-410)
    d = _decorator_sources(gmm)
    assert any("jax.custom_vjp" in s and "NONDIFF_ARGNAMES + ('trans_rhs',)" in s for s in d), d
    assert any("jax.jit" in s and "static_argnums=list(range(3, 13))" in s for s in d), d
    d = _decorator_sources(tgmm)
    assert any("jax.custom_vjp" in s and "nondiff_argnames=NONDIFF_ARGNAMES" in s for s in d), d
    assert any("jax.jit" in s and "static_argnums=list(range(3, 12))" in s for s in d), d
    src = ast.unparse(tree)
    assert "gmm.defvjp(_gmm_fwd_rule, _gmm_bwd_rule)" in src and "tgmm.defvjp(_tgmm_fwd, _tgmm_bwd_rule)" in src
    assert "ragged_dot = gmm" in src and "trans_ragged_dot = tgmm" in src
    nondiff = next(n for n in tree.body if isinstance(n, ast.Assign) and n.targets[0].id == "NONDIFF_ARGNAMES")
    assert list(ast.literal_eval(nondiff.value)) == GMM_PARAMS[3:6] + GMM_PARAMS[7:]
    # bwd rules take the non-differentiable arguments first, in positional order, then (res, do) (:383-396)
    assert [a.arg for a in _func(tree, "_gmm_bwd_rule").args.args] == GMM_PARAMS[3:] + ["res", "do"]
    assert [a.arg for a in _func(tree, "_tgmm_bwd_rule").args.args] == TGMM_PARAMS[3:] + ["res", "do"]


def test_adapter_and_torch_front_end_agree_on_signatures_and_defaults():
    from gpu_ragged_dot_amd import ops

    tree = _tree()
    for name, fn in (("gmm", ops.gmm), ("tgmm", ops.tgmm)):
        node = _func(tree, name)
        sig = inspect.signature(fn)
        ref_names = [a.arg for a in node.args.args]
        # the torch front end has the reference's parameters first, in order; what follows are the slice-of-groups
        # keywords of jax.lax.ragged_dot, which the reference does not have
        assert list(sig.parameters)[:len(ref_names)] == ref_names
        assert set(list(sig.parameters)[len(ref_names):]) <= {"group_offset", "num_actual_groups"}
        defaults = [ast.unparse(dflt) for dflt in node.args.defaults]
        torch_defaults = [p.default for nm, p in sig.parameters.items()
                          if p.default is not inspect.Parameter.empty and nm in ref_names]
        assert len(defaults) == len(torch_defaults)
        for a, b in zip(defaults, torch_defaults):
            if a in ("DEFAULT_BLOCK_M", "DEFAULT_BLOCK_K", "DEFAULT_BLOCK_N"):
                assert b == 64
            elif a == "CHUNK_M":
                assert b == 512
            elif a == "jnp.float32":
                assert str(b) == "torch.float32"
            else:
                assert ast.literal_eval(a) == b


def _c_params(header_text, name):
    m = re.search(r"\bint\s+" + name + r"\s*\(([^;]*?)\)\s*;", header_text, re.S)
    assert m, name
    params = []
    for p in re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S).split(","):
        params.append(re.findall(r"[A-Za-z_][A-Za-z_0-9]*", p)[-1])
    return params


def test_handlers_pass_arguments_in_header_order():
    with open(HEADER) as f:
        header = f.read()
    with open(SHIM) as f:
        shim = f.read()
    for name in ("rd_gmm", "rd_tgmm"):
        call = re.search(r"status\(" + name + r"\(([^;]*?)\)\)\s*;", shim, re.S)
        assert call, f"{name} call not found in rd_xla_ffi.cc"
        args = [a.strip() for a in call.group(1).split(",")]
        assert args == _c_params(header, name), (name, args)
    # both targets are defined, bound to the platform stream, and registered by the Python side under the same names
    for symbol in ("RdGmm", "RdTgmm"):
        assert re.search(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*" + symbol, shim)
    with open(ADAPTER) as f:
        adapter = f.read()
    assert '("rd_gmm", "RdGmm")' in adapter and '("rd_tgmm", "RdTgmm")' in adapter
    # every attribute the Python side sends is bound by the handler, and vice versa
    for target, symbol in (("rd_gmm", "RdGmm"), ("rd_tgmm", "RdTgmm")):
        block = shim[shim.index("XLA_FFI_DEFINE_HANDLER_SYMBOL(" + symbol):]
        block = block[:block.index(";")]
        bound = set(re.findall(r'\.Attr<[^>]+>\("([a-z_0-9]+)"\)', block))
        want = {"compute_bf16", "variant", "group_m", "group_n", "decode_nb", "split_k", "chunk_m"}
        if target == "rd_gmm":
            want.add("trans_rhs")
        assert bound == want, (symbol, bound)
    # element type comes from the buffer, never hard-coded
    assert "element_type()" in shim and not re.search(r"rd_t?gmm\([^;]*RD_DTYPE_BF16", shim)


def _shim_function(shim, name):
    """Body of a free function of the shim, braces balanced."""
    start = re.search(r"\b" + name + r"\s*\([^)]*\)\s*\{", shim)
    assert start, name
    depth, i = 1, start.end()
    while depth:
        depth += {"{": 1, "}": -1}.get(shim[i], 0)
        i += 1
    return shim[start.end():i - 1]


def test_result_element_type_rule_matches_the_python_side():
    """The handlers must accept exactly the result buffer jax_adapter declares (gpu_ragged_dot.py:210,324: the operands'
    type; float8 operands give bfloat16).  The shim's rule is evaluated from its source for every element type
    dtype_code() knows and compared with jax_adapter._out_dtype evaluated from its source."""
    with open(SHIM) as f:
        shim = f.read()
    # element types the shim accepts
    known = re.findall(r"t == ffi::DataType::([A-Z0-9]+)", _shim_function(shim, "dtype_code"))
    assert sorted(known) == ["BF16", "F16", "F32", "F8E4M3FN"], known
    # result_type(): `if (t == ffi::DataType::X) return ffi::DataType::Y;` lines, then `return t;`
    body = _shim_function(shim, "result_type")
    special = dict(re.findall(r"if \(t == ffi::DataType::([A-Z0-9]+)\) return ffi::DataType::([A-Z0-9]+);", body))
    assert re.search(r"return t;\s*$", body.strip())
    shim_rule = {t: special.get(t, t) for t in known}
    # jax_adapter._out_dtype evaluated with stand-ins for jnp
    names = {"BF16": "bfloat16", "F16": "float16", "F32": "float32", "F8E4M3FN": "float8_e4m3fn"}

    class _Jnp:
        bfloat16, float16, float32, float8_e4m3fn = "bfloat16", "float16", "float32", "float8_e4m3fn"
        dtype = staticmethod(lambda d: d)

    fn = _func(_tree(), "_out_dtype")
    scope = {"jnp": _Jnp}
    exec(compile(ast.Module(body=[fn], type_ignores=[]), ADAPTER, "exec"), scope)
    for t in known:
        assert names[shim_rule[t]] == scope["_out_dtype"](names[t]), (t, shim_rule[t])
    # both handlers check the result against that rule, and the operands against each other
    for impl, res, other in (("GmmImpl", "y_buf", "A_buf"), ("TgmmImpl", "dA_buf", "dy_buf")):
        body = _shim_function(shim, impl)
        assert f"{res}->element_type() != result_type(x_buf.element_type())" in body, impl
        assert f"{other}.element_type() != x_buf.element_type()" in body, impl
        assert f"{res}->element_type() != x_buf.element_type()" not in body, impl
