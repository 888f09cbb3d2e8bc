"""Payload modules from MLIR text, for the matmul forms the reference's own fixtures use.

The reference parses any MLIR module and lowers it with pass pipelines
(lighthouse/pipeline/driver.py, lighthouse/lh_run.py:87-110).  This target has kernels, not a
compiler, so the text front end recognises the linalg programs that map onto one kernel call and
rejects everything else with ``ValueError``:

* ``linalg.add`` of two arguments into a third (examples/basic/compile_and_run.py:25-31);
* ``linalg.matmul`` (test/run/pipeline-check.mlir:8-14), optionally followed by a broadcast bias
  add and a ReLU in named form (``linalg.broadcast`` + ``linalg.add``, ``linalg.max`` against a
  zero fill: the ops of lighthouse/ingress/mlir_gen/named.py:5-32);
* the same chain written as ``linalg.generic`` ops (test/opt/pipeline-check.mlir:27-46):
  mulf+addf contraction, addf of a 1-D operand, maximumf against a zero constant.

The matmul accumulates into its ``outs`` operand when that is a function argument (the in-place
result of bufferisation) and starts from zero when it is a zero ``linalg.fill`` / ``tensor.empty``,
also when that fill is itself an in-place operation on the argument buffer (memref form, where
operations have no results and a buffer's contents depend on the program order).
The function's argument order is kept: callers pass buffers in signature order.
"""

from __future__ import annotations

import re
from dataclasses import dataclass

from .. import _lib
from ..utils.numpy import lh_dtype
from .payloads import ArgSpec, PayloadFunction, PayloadModule

_TYPE_RE = re.compile(r"(?:tensor|memref)<((?:\d+x)*)([a-zA-Z0-9]+)>")
_FUNC_RE = re.compile(r"func\.func\s+(?:private\s+|public\s+)?@([\w.$-]+)\s*\(([^)]*)\)([^{]*)\{")
_MAP_RE = re.compile(r"(#\w+)\s*=\s*affine_map<\(([^)]*)\)\s*->\s*\(([^)]*)\)>")


@dataclass
class _Value:
    kind: str               # arg | const | empty | fill | matmul | bias | relu | bcast
    data: tuple = ()


def _parse_type(text: str):
    m = _TYPE_RE.search(text)
    if not m:
        raise ValueError(f"unsupported argument type '{text.strip()}': ranked static tensor/memref expected")
    dims = tuple(int(d) for d in m.group(1).split("x") if d)
    return dims, m.group(2)


def _function_body(text: str, start: int) -> str:
    depth, i = 1, start
    while i < len(text) and depth:
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    if depth:
        raise ValueError("unbalanced braces in function body")
    return text[start:i - 1]


def _split_statements(body: str) -> list[str]:
    """Top-level operations of a function body; a linalg.generic keeps its region."""
    out, cur, depth = [], [], 0
    for line in body.splitlines():
        stripped = line.split("//")[0].strip()
        if not stripped:
            continue
        # an operation may continue on the next line with its ins(...) / outs(...) / result type
        if not cur and out and re.match(r"(ins|outs)\s*\(|->|:\s", stripped):
            out[-1] += " " + stripped
            continue
        cur.append(stripped)
        depth += stripped.count("{") - stripped.count("}")
        # attribute dictionaries open and close on one line; a region stays open across lines
        if depth <= 0:
            out.append(" ".join(cur))
            cur, depth = [], 0
    if cur:
        out.append(" ".join(cur))
    return out


def _operands(stmt: str, key: str) -> list[str]:
    m = re.search(key + r"\s*\(([^:)]*)(?::[^)]*)?\)", stmt)
    return [o.strip() for o in m.group(1).split(",") if o.strip()] if m else []


def _maps_of(stmt: str, maps: dict[str, tuple[str, ...]]) -> list[tuple[str, ...]]:
    m = re.search(r"indexing_maps\s*=\s*\[([^\]]*)\]", stmt)
    if not m:
        return []
    found = []
    for item in re.findall(r"#\w+|affine_map<\([^)]*\)\s*->\s*\([^)]*\)>", m.group(1)):
        if item.startswith("#"):
            if item not in maps:
                raise ValueError(f"unknown affine map {item}")
            found.append(maps[item])
        else:
            mm = re.search(r"->\s*\(([^)]*)\)", item)
            found.append(tuple(x.strip() for x in mm.group(1).split(",") if x.strip()))
    return found


def _is_zero(v: _Value | None) -> bool:
    return v is not None and v.kind == "const" and float(v.data[0]) == 0.0


def parse_function(text: str, name: str, maps: dict[str, tuple[str, ...]]) -> PayloadFunction:
    m = next((f for f in _FUNC_RE.finditer(text) if f.group(1) == name), None)
    if m is None:
        raise ValueError(f"no function named '{name}' in payload module")
    arg_names, arg_types = [], []
    for a in [x for x in m.group(2).split(",") if x.strip()]:
        nm, _, ty = a.partition(":")
        arg_names.append(nm.strip())
        arg_types.append(_parse_type(ty))
    env: dict[str, _Value] = {n: _Value("arg", (i,)) for i, n in enumerate(arg_names)}
    # A buffer (memref) is rewritten in place by operations that have no SSA result.  Each such
    # write makes a new version of the buffer's name, and operands are read through `cur`, so a
    # value always refers to the contents its operands had at that point of the program.
    cur: dict[str, str] = {}
    versions: dict[str, int] = {}
    returned = None
    for stmt in _split_statements(_function_body(text, m.end())):
        res = re.match(r"(%[\w.#-]+)(?::\d+)?\s*=\s*(.*)", stmt)
        result, rest = (res.group(1), res.group(2)) if res else (None, stmt)
        op = rest.split()[0].split("(")[0]
        raw_outs = _operands(rest, "outs")
        ins = [cur.get(x, x) for x in _operands(rest, "ins")]
        outs = [cur.get(x, x) for x in raw_outs]
        val = None
        if op == "arith.constant":
            c = re.search(r"arith\.constant\s+(dense<)?([-+0-9.eE]+|true|false)", rest)
            val = _Value("const", (float(c.group(2)) if c and c.group(2) not in ("true", "false") else 1.0,))
        elif op == "tensor.empty" or op == "memref.alloc":
            val = _Value("empty")
        elif op == "linalg.fill":
            src = env.get(ins[0])
            if src is None or src.kind != "const":
                raise ValueError(f"linalg.fill with a non-constant value: {stmt}")
            val = _Value("fill", (src.data[0], outs[0]))
        elif op == "linalg.matmul":
            val = _Value("matmul", (ins[0], ins[1], outs[0], False, False))
        elif op == "linalg.broadcast":
            val = _Value("bcast", (ins[0],))
        elif op == "linalg.add":
            a, b = (env.get(x) for x in ins)
            if b is not None and b.kind == "bcast":
                val = _Value("bias", (ins[0], b.data[0]))
            elif a is not None and a.kind == "bcast":
                val = _Value("bias", (ins[1], a.data[0]))
            else:
                val = _Value("add2", (ins[0], ins[1], outs[0] if outs else None))  # plain elementwise sum
        elif op == "linalg.max":
            a, b = (env.get(x) for x in ins)
            zero = lambda v: v is not None and v.kind == "fill" and float(v.data[0]) == 0.0  # noqa: E731
            if zero(b):
                val = _Value("relu", (ins[0],))
            elif zero(a):
                val = _Value("relu", (ins[1],))
            else:
                raise ValueError(f"linalg.max against something other than a zero fill: {stmt}")
        elif op == "linalg.generic":
            val = _classify_generic(rest, ins, outs, env, maps)
        elif op in ("return", "func.return"):
            ops_ = [o.strip() for o in rest.split(":")[0].split()[1:]]
            returned = ops_[0].rstrip(",") if ops_ else None
            returned = cur.get(returned, returned) if returned else None
            continue
        else:
            raise ValueError(f"unsupported operation '{op}' in @{name}; this target runs matmul(+bias)(+relu) payloads")
        if result is not None:
            env[result] = val
        elif raw_outs and op.startswith("linalg."):
            # in-place write to a buffer: later reads of raw_outs[0] see this value
            versions[raw_outs[0]] = versions.get(raw_outs[0], 0) + 1
            versioned = f"{raw_outs[0]}@{versions[raw_outs[0]]}"
            env[versioned] = val
            cur[raw_outs[0]] = versioned
        last = val if val.kind in ("matmul", "bias", "relu", "add2") else None
        if last is not None:
            env["__last__"] = val
    root = env.get(returned) if returned else env.get("__last__")
    if root is None:
        raise ValueError(f"@{name} computes nothing this target recognises")
    if root.kind == "add2":
        return _elementwise_add(name, root, env, arg_types)
    has_relu = has_bias = False
    bias_name = None
    if root.kind == "relu":
        has_relu, root = True, env[root.data[0]]
    if root.kind == "bias":
        has_bias, bias_name, root = True, root.data[1], env[root.data[0]]
    if root.kind != "matmul":
        raise ValueError(f"@{name}: expected relu?(bias?(matmul)), found '{root.kind}' at its root")
    a_name, b_name, c_name, ta, tb = root.data
    cval = env.get(c_name)
    while cval is not None and cval.kind == "fill":
        if float(cval.data[0]) != 0.0:
            raise ValueError("matmul accumulating into a non-zero fill is not supported")
        c_name = cval.data[1]
        zero_init = True
        cval = env.get(c_name)
        if cval is not None and cval.kind in ("arg", "empty"):
            break
    else:
        zero_init = cval is not None and cval.kind == "empty"
    for nm in (a_name, b_name) + ((bias_name,) if has_bias else ()):
        if env.get(nm) is None or env[nm].kind != "arg":
            raise ValueError(f"@{name}: operand {nm} of the matmul chain is not a function argument")
    if cval is None or cval.kind != "arg":
        raise ValueError(f"@{name}: the matmul result is not written to a function argument; "
                         "pass the output buffer as an argument (results-to-arguments convention)")
    idx = {n: env[n].data[0] for n in (a_name, b_name, c_name)}
    a_dims, a_elem = arg_types[idx[a_name]]
    b_dims, b_elem = arg_types[idx[b_name]]
    c_dims, c_elem = arg_types[idx[c_name]]
    if len(a_dims) != 2 or len(b_dims) != 2 or len(c_dims) != 2 or a_elem != b_elem:
        raise ValueError(f"@{name}: matmul operands must be 2-D tensors of one element type")
    M, K = (a_dims[1], a_dims[0]) if ta else a_dims
    N = b_dims[0] if tb else b_dims[1]
    if (b_dims[1] if tb else b_dims[0]) != K or c_dims != (M, N):
        raise ValueError(f"@{name}: inconsistent matmul shapes {a_dims} x {b_dims} -> {c_dims}")
    flags = ((_lib.GEMM_HAS_BIAS if has_bias else 0) | (_lib.GEMM_HAS_RELU if has_relu else 0)
             | (0 if zero_init else _lib.GEMM_ACCUMULATE_C)
             | (_lib.GEMM_TRANSPOSE_A if ta else 0) | (_lib.GEMM_TRANSPOSE_B if tb else 0))
    order = [idx[c_name], idx[a_name], idx[b_name]]
    if has_bias:
        order.append(env[bias_name].data[0])
        if arg_types[order[3]] != ((N,), c_elem):
            raise ValueError(f"@{name}: bias must be a 1-D tensor of {N} {c_elem} values")
    args = [ArgSpec(d, e, writable=(i == order[0])) for i, (d, e) in enumerate(arg_types)]
    unused = sorted(set(range(len(args))) - set(order))
    if unused:
        raise ValueError(f"@{name}: arguments {unused} take no part in the matmul chain")
    attrs = _lib.MatmulAttrs(lh_dtype(a_elem), lh_dtype(c_elem), flags)
    flops = 2 * M * N * K + (M * N if has_bias else 0) + (M * N if has_relu else 0)
    return PayloadFunction(name, "matmul", attrs, args, flops, 0, arg_order=order)


def _elementwise_add(name: str, root: _Value, env: dict, arg_types: list) -> PayloadFunction:
    """`linalg.add ins(%a, %b) outs(%out)` on three function arguments of one shape and type: the
    kernel of examples/basic/compile_and_run.py:25-31 (memref<16x32xf32>)."""
    a, b, out = root.data
    vals = [env.get(x) for x in (a, b, out)]
    if any(v is None or v.kind != "arg" for v in vals):
        raise ValueError(f"@{name}: linalg.add must read two function arguments and write a third "
                         "(results-to-arguments convention)")
    ia, ib, io = (v.data[0] for v in vals)
    if not (arg_types[ia] == arg_types[ib] == arg_types[io]) or io in (ia, ib):
        raise ValueError(f"@{name}: linalg.add needs three distinct arguments of one shape and element type")
    dims, elem = arg_types[io]
    if len(dims) != 2:
        raise ValueError(f"@{name}: linalg.add runs on 2-D buffers, got rank {len(dims)}")
    if elem not in ("f32", "bf16", "f16"):
        raise ValueError(f"@{name}: linalg.add on {elem} is not supported")
    unused = sorted(set(range(len(arg_types))) - {ia, ib, io})
    if unused:
        raise ValueError(f"@{name}: arguments {unused} take no part in the sum")
    n = 1
    for d in dims:
        n *= d
    args = [ArgSpec(d, e, writable=(i == io)) for i, (d, e) in enumerate(arg_types)]
    attrs = _lib.ElementwiseAttrs(_lib.EW_ADD, lh_dtype(elem), lh_dtype(elem), 0)
    return PayloadFunction(name, "elementwise", attrs, args, n, 3 * n * (4 if elem == "f32" else 2), arg_order=[io, ia, ib])


def _classify_generic(stmt, ins, outs, env, maps) -> _Value:
    imaps = _maps_of(stmt, maps)
    iters = re.findall(r'"(parallel|reduction)"', stmt.split("ins(")[0].split("outs(")[0])
    region = stmt[stmt.index("^bb0"):] if "^bb0" in stmt else ""
    body_ops = re.findall(r"=\s*(arith\.\w+)", region)
    if iters.count("reduction") == 1 and body_ops == ["arith.mulf", "arith.addf"] and len(ins) == 2 and len(outs) == 1:
        if len(imaps) != 3:
            raise ValueError("contraction generic needs three indexing maps")
        red = None
        # The reduction dimension is the one the output map does not mention.
        dims_all = {d for mp in imaps for d in mp}
        red = (dims_all - set(imaps[2])).pop()
        m_dim, n_dim = imaps[2]
        ta = imaps[0] == (red, m_dim)
        tb = imaps[1] == (n_dim, red)
        if not (ta or imaps[0] == (m_dim, red)) or not (tb or imaps[1] == (red, n_dim)):
            raise ValueError(f"contraction with unsupported indexing maps {imaps}")
        return _Value("matmul", (ins[0], ins[1], outs[0], ta, tb))
    if iters and all(i == "parallel" for i in iters) and body_ops == ["arith.addf"] and len(ins) == 1:
        if len(imaps) == 2 and len(imaps[0]) == 1 and imaps[0][0] == imaps[1][-1]:
            return _Value("bias", (outs[0], ins[0]))
        raise ValueError(f"elementwise add that is not a row-broadcast bias: maps {imaps}")
    if iters and all(i == "parallel" for i in iters) and body_ops == ["arith.maximumf"]:
        consts = re.findall(r"arith\.maximumf\s+(%[\w.#-]+)\s*,\s*(%[\w.#-]+)", region)
        if consts and any(_is_zero(env.get(c)) for c in consts[0]):
            src = outs[0] if not ins else ins[0]
            return _Value("relu", (src,))
        raise ValueError("maximumf against something other than a zero constant")
    raise ValueError(f"unsupported linalg.generic (iterators {iters}, body {body_ops})")


def parse_payload_module(text: str, entry_points: list[str] | None = None) -> PayloadModule:
    """Build a payload module from MLIR text; `entry_points` limits which functions are read."""
    maps = {m.group(1): tuple(x.strip() for x in m.group(3).split(",") if x.strip()) for m in _MAP_RE.finditer(text)}
    names = entry_points or [f.group(1) for f in _FUNC_RE.finditer(text)]
    if not names:
        raise ValueError("no func.func found in the payload module")
    module = PayloadModule()
    for n in names:
        module.add(parse_function(text, n, maps))
    return module


def load_payload_module(path: str, entry_points: list[str] | None = None) -> PayloadModule:
    with open(path) as f:
        return parse_payload_module(f.read(), entry_points)
