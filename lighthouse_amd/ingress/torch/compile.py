"""``torch.compile`` backend that routes FX graphs onto the HIP kernels.

Same contract as the MLIR backend of lighthouse/ingress/torch/compile.py:154-496:
``gpu_backend(fn_compile, device, ...)`` returns a callable ``(GraphModule, example_inputs)
-> JITFunction``; shapes are static (``dynamic=False``, compile.py:378-382); the compiled
function takes the graph's input tensors and returns the list of its outputs
(``JITFunction.__call__`` :108-126) and has ``benchmark(*tensors, nruns, nwarmup)`` returning
seconds per call (:128-151).  Where the reference imports the graph into MLIR with torch-mlir and
JIT-compiles it, this backend lowers the graph to a plan: every compute node becomes one call
into liblighthouse_hip.so (Linear with its ReLU / tanh-GELU fused into the GEMM epilogue,
LayerNorm, scaled-dot-product attention on strided head views, residual adds, softmax, GELU),
shape-only nodes (view, transpose, split, ...) stay tensor metadata operations.  A compute node
with no kernel raises ``ValueError`` at compile time unless ``allow_torch_fallback`` is set; there
is no CPU path.
"""

from __future__ import annotations

import operator
import time
from collections.abc import Callable, Sequence
from dataclasses import dataclass, field

import numpy as np
import torch
import torch.nn.functional as F

from ... import ops

# Shape-only tensor methods / functions: executed as torch metadata operations (no kernel, except
# the copy a `contiguous()` / `reshape()` of a non-contiguous view needs).
_METADATA_METHODS = {
    "view", "reshape", "transpose", "permute", "split", "chunk", "contiguous", "size", "flatten", "unflatten",
    "squeeze", "unsqueeze", "t", "detach", "expand", "unbind", "dim", "view_as", "reshape_as", "__getitem__",
}
_METADATA_FUNCTIONS = {
    operator.getitem, torch.transpose, torch.permute, torch.reshape, torch.flatten, torch.split, torch.chunk,
    torch.squeeze, torch.unsqueeze, torch.t, torch.unbind,
}


@dataclass
class PlanStep:
    """One node of the lowered graph: `kind` names the kernel ("hip.gemm", "hip.layer_norm", ...) or
    "meta.<op>" for shape-only nodes; `run(env)` computes the node's value from the environment."""

    name: str
    kind: str
    run: Callable[[dict], object]
    detail: dict = field(default_factory=dict)


@dataclass(frozen=True)
class _Ref:
    """Names an environment entry produced by a synthetic plan step (a module's parameter)."""

    name: str


def _has_node(a) -> bool:
    if isinstance(a, (torch.fx.Node, _Ref)):
        return True
    if isinstance(a, dict):
        return any(_has_node(v) for v in a.values())
    if isinstance(a, (tuple, list)):
        return any(_has_node(x) for x in a)
    if isinstance(a, slice):
        return any(_has_node(x) for x in (a.start, a.stop, a.step))
    return False


def _resolver(a) -> Callable[[dict], object]:
    """A function env -> value for one FX argument (nodes nested in tuples / lists / dicts / slices
    are looked up in the environment), built at lowering time so that a call of the compiled
    function does no type dispatch over its arguments: constants are returned as they are, a node
    is one dictionary lookup."""
    if not _has_node(a):
        return lambda env: a
    if isinstance(a, (torch.fx.Node, _Ref)):
        name = a.name
        return lambda env: env[name]
    if isinstance(a, dict):
        items = [(k, _resolver(v)) for k, v in a.items()]
        return lambda env: {k: f(env) for k, f in items}
    if isinstance(a, (tuple, list)):
        parts, ctor = [_resolver(x) for x in a], type(a)
        return lambda env: ctor(f(env) for f in parts)
    start, stop, step = _resolver(a.start), _resolver(a.stop), _resolver(a.step)  # a slice
    return lambda env: slice(start(env), stop(env), step(env))


def _call_resolver(args, kwargs) -> Callable[[dict], tuple]:
    """Resolvers of a call's positional and keyword arguments."""
    return _resolver(tuple(args)), (_resolver(dict(kwargs)) if kwargs else None)


class _WeightCache:
    """Per-compiled-function cache of prepared parameters (a Linear weight stored [out, in] is kept
    as a contiguous [in, out] matrix so the GEMM streams it untransposed; LayerNorm parameters are
    kept in float32).  Keyed by storage address and version, so an optimizer step refreshes it."""

    def __init__(self):
        self._store: dict = {}

    def get(self, t: torch.Tensor, tag: str, make: Callable[[torch.Tensor], torch.Tensor]) -> torch.Tensor:
        key = (tag, t.data_ptr(), tuple(t.shape), t.dtype)
        hit = self._store.get(key)
        if hit is not None and hit[0] == t._version:
            return hit[1]
        prepared = make(t.detach())
        self._store[key] = (t._version, prepared)
        return prepared


def _as_2d(x: torch.Tensor) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    return x2 if x2.is_contiguous() else x2.contiguous()


class _Lowering:
    def __init__(self, gm: torch.fx.GraphModule, allow_torch_fallback: bool):
        self.gm = gm
        self.allow_torch_fallback = allow_torch_fallback
        self.cache = _WeightCache()
        self.steps: list[PlanStep] = []
        self.fused: dict[str, str] = {}  # activation / residual-add node name -> name of the linear it is fused into
        self.order = {n: i for i, n in enumerate(gm.graph.nodes)}

    # -- helpers -------------------------------------------------------------------------
    @staticmethod
    def _kwarg(node, name, pos, default=None):
        if name in node.kwargs:
            return node.kwargs[name]
        if len(node.args) > pos:
            return node.args[pos]
        return default

    def _single_user_activation(self, node):
        """(activation kind, activation node) if `node` feeds exactly one ReLU / tanh-GELU."""
        users = list(node.users)
        if len(users) != 1:
            return None, None
        u = users[0]
        if u.op == "call_function" and u.target in (F.relu, torch.relu) and u.args[0] is node:
            if not self._kwarg(u, "inplace", 1, False):
                return "relu", u
        if u.op == "call_method" and u.target == "relu" and u.args[0] is node:
            return "relu", u
        if u.op == "call_function" and u.target is F.gelu and u.args[0] is node:
            if self._kwarg(u, "approximate", 1, "none") == "tanh":
                return "gelu", u
        if u.op == "call_module":
            mod = self.gm.get_submodule(u.target)
            if isinstance(mod, torch.nn.ReLU) and not mod.inplace:
                return "relu", u
            if isinstance(mod, torch.nn.GELU) and mod.approximate == "tanh":
                return "gelu", u
        return None, None

    def _single_user_residual_add(self, node):
        """(add node, residual operand) if `node` feeds exactly one `r + node` / `node + r` whose other
        operand is a tensor computed before `node`: the GEMM then starts its accumulation from r."""
        users = list(node.users)
        if len(users) != 1:
            return None, None
        u = users[0]
        is_add = (u.op == "call_function" and u.target in (operator.add, torch.add, operator.iadd)) or \
                 (u.op == "call_method" and u.target in ("add", "__add__"))
        if not is_add or len(u.args) < 2 or self._kwarg(u, "alpha", 2, 1) != 1:
            return None, None
        other = u.args[1] if u.args[0] is node else u.args[0]
        if not isinstance(other, torch.fx.Node) or other is node or self.order[other] > self.order[node]:
            return None, None
        return u, other

    def _emit(self, name, kind, run, **detail):
        self.steps.append(PlanStep(name, kind, run, detail))

    def _param(self, node, attr, mod) -> _Ref:
        ref = _Ref(f"{node.name}__{attr}")
        self._emit(ref.name, "meta.get_attr", lambda env: getattr(mod, attr))
        return ref

    # -- compute nodes -------------------------------------------------------------------
    def _linear(self, node, x_arg, w_arg, b_arg):
        act, act_node = self._single_user_activation(node)
        add_node, res_arg = (None, None) if act_node is not None else self._single_user_residual_add(node)
        if act_node is not None:
            self.fused[act_node.name] = node.name
        if add_node is not None:
            self.fused[add_node.name] = node.name
        cache = self.cache

        x_f, w_f, b_f, r_f = _resolver(x_arg), _resolver(w_arg), _resolver(b_arg), _resolver(res_arg)

        def run(env, act=act):
            x, w, b, r = x_f(env), w_f(env), b_f(env), r_f(env)
            # A 16-bit [out, in] weight is read in place as a transposed B (the direct kernels take its
            # panel like A's); an f32 weight is transposed once and cached.
            in_place = w.dtype != torch.float32 and w.dim() == 2 and w.stride(1) == 1
            wt = w.detach() if in_place else cache.get(w, "linear_weight", lambda t: t.t().contiguous())
            x2 = _as_2d(x)
            n_out = wt.shape[0] if in_place else wt.shape[1]
            shape = (*x.shape[:-1], n_out)
            if r is not None:
                # x + linear(y): the accumulation starts from the residual, which is only read.
                if not isinstance(r, torch.Tensor) or tuple(r.shape) != shape or r.dtype != x.dtype:
                    raise ValueError(f"{node.name}: broadcasting / mixed-type add is not supported")
                r = _as_2d(r)
            # (a Linear multiplies by its [out, in] weight transposed)
            _check_schedule(node.name, schedule, x2.shape[0], n_out, x2.shape[1], False, True)
            out = ops.gemm(x2, wt, b.detach() if b is not None else None, relu=act == "relu", gelu=act == "gelu",
                           residual=r, transpose_b=in_place, tile=schedule.get("tile"), split_k=schedule.get("split_k"))
            return out.view(shape)

        schedule: dict = {}
        self._emit(node.name, "hip.gemm", run, bias=b_arg is not None, activation=act, residual=add_node is not None,
                   schedule=schedule)

    def _matmul(self, node, a_arg, b_arg, bias_arg=None):
        """torch.matmul / mm / `@` with a 2-D right operand (and addmm with a vector bias): one GEMM.
        A transposed view of a row-major matrix (`w.t()`) goes to the kernel as a transpose flag, not
        as a copy; a following ReLU / tanh-GELU with no other user is fused into the epilogue."""
        act, act_node = self._single_user_activation(node)
        if act_node is not None:
            self.fused[act_node.name] = node.name
        a_f, b_f, bias_f = _resolver(a_arg), _resolver(b_arg), _resolver(bias_arg)

        def operand(t):
            """-> (matrix with unit inner stride, transposed?)"""
            if t.stride(1) == 1 and t.stride(0) >= t.shape[1]:
                return t, False
            if t.stride(0) == 1 and t.stride(1) >= t.shape[0]:
                return t.t(), True
            return t.contiguous(), False

        def run(env, act=act):
            a, b, bias = a_f(env), b_f(env), bias_f(env)
            if not (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)) or a.dim() < 2 or b.dim() != 2:
                raise ValueError(f"{node.name}: matmul needs a [..., K] left and a [K, N] right operand "
                                 "(batched right operands are not supported)")
            if a.dtype != b.dtype:
                raise ValueError(f"{node.name}: mixed-type matmul ({a.dtype} @ {b.dtype}) is not supported")
            if bias is not None and (bias.dim() != 1 or bias.shape[0] != b.shape[1] or bias.dtype != a.dtype):
                raise ValueError(f"{node.name}: addmm needs a vector bias of the result's width and type")
            shape = (*a.shape[:-1], b.shape[1])
            a2, ta = operand(a) if a.dim() == 2 else (_as_2d(a), False)
            b2, tb = operand(b)
            _check_schedule(node.name, schedule, a2.shape[1] if ta else a2.shape[0], b.shape[1], b.shape[0], ta, tb)
            out = ops.gemm(a2, b2, bias.detach().contiguous() if bias is not None else None, relu=act == "relu",
                           gelu=act == "gelu", transpose_a=ta, transpose_b=tb, tile=schedule.get("tile"),
                           split_k=schedule.get("split_k"))
            return out.view(shape)

        schedule: dict = {}
        self._emit(node.name, "hip.gemm", run, bias=bias_arg is not None, activation=act, residual=False,
                   schedule=schedule)

    def _layer_norm(self, node, x_arg, shape, w_arg, b_arg, eps):
        if len(tuple(shape)) != 1:
            raise ValueError(f"{node.name}: LayerNorm over {tuple(shape)}: only the last dimension is supported")
        cache = self.cache

        x_f, w_f, b_f = _resolver(x_arg), _resolver(w_arg), _resolver(b_arg)

        def run(env):
            x = x_f(env)
            n = x.shape[-1]
            w, b = w_f(env), b_f(env)
            gamma = cache.get(w, "ln", lambda t: t.float().contiguous()) if w is not None else \
                cache.get(x.new_empty(0), f"ones{n}", lambda t: torch.ones(n, device=x.device))
            beta = cache.get(b, "ln", lambda t: t.float().contiguous()) if b is not None else \
                cache.get(x.new_empty(0), f"zeros{n}", lambda t: torch.zeros(n, device=x.device))
            return ops.layer_norm(_as_2d(x), gamma, beta, eps).view(x.shape)

        self._emit(node.name, "hip.layer_norm", run)

    def _sdpa(self, node):
        q_arg, k_arg, v_arg = node.args[:3]
        if self._kwarg(node, "attn_mask", 3) is not None:
            raise ValueError(f"{node.name}: attention masks other than is_causal are not supported")
        if self._kwarg(node, "dropout_p", 4, 0.0) != 0.0:
            raise ValueError(f"{node.name}: attention dropout is not supported")
        causal = bool(self._kwarg(node, "is_causal", 5, False))
        scale = self._kwarg(node, "scale", 6)

        q_f, k_f, v_f = _resolver(q_arg), _resolver(k_arg), _resolver(v_arg)

        def run(env):
            q, k, v = q_f(env), k_f(env), v_f(env)
            if q.dim() != 4:
                raise ValueError("scaled_dot_product_attention expects [batch, heads, seq, head_dim] tensors")
            z, h, t, d = q.shape
            # Heads stored innermost ([batch, seq, heads, d] viewed transposed, the layout a fused QKV
            # Linear produces): write the result in that layout too, so the transpose + contiguous
            # that follows in the model is free.
            if q.stride(1) < q.stride(2):
                out = torch.empty((z, t, h, d), dtype=q.dtype, device=q.device).transpose(1, 2)
            else:
                out = torch.empty((z, h, t, d), dtype=q.dtype, device=q.device)
            return ops.attention(q, k, v, causal=causal, scale=scale, out=out)

        self._emit(node.name, "hip.attention", run, causal=causal)

    def _binary_add(self, node):
        a_arg, b_arg = node.args[:2]
        if node.name in self.fused:
            src = self.fused[node.name]
            self._emit(node.name, "fused", lambda env, src=src: env[src], into=src)
            return
        if self._kwarg(node, "alpha", 2, 1) != 1:
            raise ValueError(f"{node.name}: add with alpha is not supported")

        a_f, b_f = _resolver(a_arg), _resolver(b_arg)

        def run(env):
            a, b = a_f(env), b_f(env)
            if not (isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor)):
                return a + b  # Python scalars / sizes
            if a.shape != b.shape or a.dtype != b.dtype:
                raise ValueError(f"{node.name}: broadcasting / mixed-type add is not supported "
                                 f"({tuple(a.shape)} {a.dtype} + {tuple(b.shape)} {b.dtype})")
            a = a if a.is_contiguous() else a.contiguous()
            b = b if b.is_contiguous() else b.contiguous()
            return ops.add(a, b)

        self._emit(node.name, "hip.add", run)

    def _unary(self, node, kind, x_arg):
        if node.name in self.fused:
            src = self.fused[node.name]
            self._emit(node.name, "fused", lambda env, src=src: env[src], into=src)
            return

        x_f = _resolver(x_arg)

        def run(env):
            x = x_f(env)
            x = x if x.is_contiguous() else x.contiguous()
            if kind == "gelu":
                return ops.gelu_tanh(x)
            if kind == "softmax":
                return ops.softmax(x.view(-1, x.shape[-1])).view(x.shape)
            zero = x.new_zeros(x.shape[-1])  # ReLU = bias_act with a zero bias
            return ops.bias_act(x.view(-1, x.shape[-1]), zero, relu=True).view(x.shape)

        self._emit(node.name, f"hip.{kind}", run)

    def _fallback(self, node, what):
        if not self.allow_torch_fallback:
            raise ValueError(f"no HIP kernel for graph node '{node.name}' ({what}); "
                             "pass allow_torch_fallback=True to run it with torch on the device")
        if node.op == "call_function":
            run = self._call(node.target, node.args, node.kwargs)
        elif node.op == "call_method":
            run = self._method_call(node)
        else:
            run = self._call(self.gm.get_submodule(node.target), node.args, node.kwargs)
        self._emit(node.name, f"torch.{what}", run)

    @staticmethod
    def _call(fn, args, kwargs):
        args_f, kwargs_f = _call_resolver(args, kwargs)
        if kwargs_f is None:
            return lambda env: fn(*args_f(env))
        return lambda env: fn(*args_f(env), **kwargs_f(env))

    @staticmethod
    def _method_call(node):
        self_f, method = _resolver(node.args[0]), node.target
        args_f, kwargs_f = _call_resolver(node.args[1:], node.kwargs)
        if kwargs_f is None:
            return lambda env: getattr(self_f(env), method)(*args_f(env))
        return lambda env: getattr(self_f(env), method)(*args_f(env), **kwargs_f(env))

    # -- dispatch ------------------------------------------------------------------------
    def lower(self) -> tuple[list[str], list[PlanStep], object]:
        placeholders: list[str] = []
        output_spec = None
        for node in self.gm.graph.nodes:
            if node.op == "placeholder":
                placeholders.append(node.name)
            elif node.op == "get_attr":
                obj = self.gm
                for part in node.target.split("."):
                    obj = getattr(obj, part)
                self._emit(node.name, "meta.get_attr", lambda env, obj=obj: obj)
            elif node.op == "output":
                output_spec = node.args[0]
            elif node.op == "call_function":
                self._call_function(node)
            elif node.op == "call_method":
                self._call_method(node)
            elif node.op == "call_module":
                self._call_module(node)
            else:
                raise ValueError(f"unsupported FX opcode {node.op}")
        return placeholders, self.steps, output_spec

    def _meta(self, node):
        if node.op == "call_function":
            run = self._call(node.target, node.args, node.kwargs)
            label = getattr(node.target, "__name__", str(node.target))
        else:
            run = self._method_call(node)
            label = node.target
        self._emit(node.name, f"meta.{label}", run)

    def _call_function(self, node):
        t = node.target
        if t in (torch._C._nn.linear, F.linear):
            return self._linear(node, node.args[0], node.args[1], self._kwarg(node, "bias", 2))
        if t in (torch.matmul, operator.matmul, torch.mm):
            return self._matmul(node, node.args[0], node.args[1])
        if t is torch.addmm:
            if self._kwarg(node, "beta", 3, 1) != 1 or self._kwarg(node, "alpha", 4, 1) != 1:
                return self._fallback(node, "addmm(alpha, beta)")
            return self._matmul(node, node.args[1], node.args[2], node.args[0])
        if t is F.layer_norm:
            return self._layer_norm(node, node.args[0], node.args[1], self._kwarg(node, "weight", 2),
                                    self._kwarg(node, "bias", 3), self._kwarg(node, "eps", 4, 1e-5))
        if t is F.scaled_dot_product_attention:
            return self._sdpa(node)
        if t in (operator.add, torch.add, operator.iadd):
            return self._binary_add(node)
        if t in (F.relu, torch.relu):
            return self._unary(node, "relu", node.args[0])
        if t is F.gelu:
            if self._kwarg(node, "approximate", 1, "none") != "tanh":
                return self._fallback(node, "gelu(erf)")
            return self._unary(node, "gelu", node.args[0])
        if t in (F.softmax, torch.softmax):
            dim = self._kwarg(node, "dim", 1, -1)
            if dim not in (-1,):
                return self._fallback(node, f"softmax(dim={dim})")
            return self._unary(node, "softmax", node.args[0])
        if t is F.dropout and (self._kwarg(node, "p", 1, 0.5) == 0.0 or not self._kwarg(node, "training", 2, True)):
            return self._emit(node.name, "meta.identity", _resolver(node.args[0]))
        if t in _METADATA_FUNCTIONS:
            return self._meta(node)
        return self._fallback(node, getattr(t, "__name__", str(t)))

    def _call_method(self, node):
        if node.target in _METADATA_METHODS:
            return self._meta(node)
        if node.target == "relu":
            return self._unary(node, "relu", node.args[0])
        if node.target in ("add", "__add__"):
            return self._binary_add(node)
        if node.target in ("matmul", "mm", "__matmul__"):
            return self._matmul(node, node.args[0], node.args[1])
        return self._fallback(node, f"Tensor.{node.target}")

    def _call_module(self, node):
        mod = self.gm.get_submodule(node.target)
        x = node.args[0]
        if isinstance(mod, torch.nn.Linear):
            # Parameters of a call_module node are read from the module at run time.
            w_ref = self._param(node, "weight", mod)
            b_ref = self._param(node, "bias", mod) if mod.bias is not None else None
            return self._linear(node, x, w_ref, b_ref)
        if isinstance(mod, torch.nn.LayerNorm):
            w_ref = self._param(node, "weight", mod) if mod.elementwise_affine else None
            b_ref = self._param(node, "bias", mod) if mod.elementwise_affine and mod.bias is not None else None
            return self._layer_norm(node, x, mod.normalized_shape, w_ref, b_ref, mod.eps)
        if isinstance(mod, torch.nn.ReLU) and not mod.inplace:
            return self._unary(node, "relu", x)
        if isinstance(mod, torch.nn.GELU) and mod.approximate == "tanh":
            return self._unary(node, "gelu", x)
        if isinstance(mod, torch.nn.Dropout) and (mod.p == 0.0 or not mod.training):
            return self._emit(node.name, "meta.identity", _resolver(x))
        if isinstance(mod, torch.nn.Identity):
            return self._emit(node.name, "meta.identity", _resolver(x))
        return self._fallback(node, type(mod).__name__)


class JITFunction:
    """Callable produced by the backend (lighthouse/ingress/torch/compile.py:47-151)."""

    def __init__(self, placeholders: list[str], plan: list[PlanStep], output_spec, device: torch.device,
                 entry_func: str = "main"):
        self.placeholders = placeholders
        self.plan = plan
        self.output_spec = output_spec
        self._output = _resolver(output_spec)
        self.device = device
        self.entry_func = entry_func

    @property
    def kinds(self) -> list[str]:
        """Kernel / operation kind of every plan step that does work, in execution order."""
        return [s.kind for s in self.plan if not s.kind.startswith("meta.") and s.kind != "fused"]

    def __call__(self, *args: torch.Tensor) -> list[torch.Tensor]:
        if len(args) != len(self.placeholders):
            raise ValueError(f"{self.entry_func}: expected {len(self.placeholders)} tensors, got {len(args)}")
        for a in args:
            if isinstance(a, torch.Tensor) and a.device.type != self.device.type:
                raise ValueError(f"{self.entry_func}: tensor on {a.device}, compiled for {self.device}")
        env = dict(zip(self.placeholders, args))
        with torch.no_grad():
            for step in self.plan:
                env[step.name] = step.run(env)
        out = self._output(env)
        return list(out) if isinstance(out, (tuple, list)) else [out]

    def benchmark(self, *args: torch.Tensor, nruns: int = 500, nwarmup: int = 500) -> np.ndarray:
        """`nwarmup` untimed calls, then `nruns` calls timed one by one (wall clock around call +
        device synchronisation, like the reference's benchmark wrapper); seconds per call."""
        for _ in range(nwarmup):
            self(*args)
        torch.cuda.synchronize()
        times = np.zeros(nruns, dtype=np.float64)
        for i in range(nruns):
            t0 = time.perf_counter()
            self(*args)
            torch.cuda.synchronize()
            times[i] = time.perf_counter() - t0
        return times



def _check_schedule(name: str, schedule: dict, M: int, N: int, K: int, ta: bool, tb: bool) -> None:
    """A layer's schedule parameters may state the problem they were chosen for (shape, and which
    operands are stored transposed); running them on another one is an error, not a silent fallback."""
    want = schedule.get("mnk")
    if want is not None and tuple(want) != (M, N, K):
        raise ValueError(f"{name}: schedule parameters are for a {want[0]}x{want[1]}x{want[2]} matmul, the layer is "
                         f"{M}x{N}x{K}")
    for key, have in (("transpose_a", ta), ("transpose_b", tb)):
        if key in schedule and bool(schedule[key]) != bool(have):
            raise ValueError(f"{name}: schedule parameters were chosen for {key}={bool(schedule[key])}, the layer's "
                             f"operand is {'stored transposed' if have else 'not transposed'}")


_SCHEDULE_KEYS = {"layer_kind", "m", "n", "k", "wg_m", "wg_n", "split_k", "transpose_a", "transpose_b", "source"}


def with_schedule_parameters(parameters: Sequence[dict]) -> Callable[[list[PlanStep]], list[PlanStep]]:
    """An `fn_compile` that gives the i-th GEMM of the lowered graph the i-th entry of `parameters`,
    the per-layer dictionaries of the reference's ScheduleParameters
    (lighthouse/schedule/parameters.py; examples/xegpu/torch_matmul.py:219-262: layer_kind, m, n, k,
    wg_m, wg_n, ...).  This target's kernels take `wg_m` x `wg_n` (the workgroup tile) and `split_k`;
    `m`, `n`, `k`, `transpose_a` and `transpose_b` state the problem the entry was chosen for and are
    checked against the layer when it runs (`source` is informational);
    every other tiling key of the XeGPU schedule has no counterpart and is an error, as is a count of
    entries that differs from the graph's GEMMs."""
    parameters = [dict(p) for p in parameters]
    for p in parameters:
        unknown = sorted(set(p) - _SCHEDULE_KEYS)
        if unknown:
            raise ValueError(f"schedule parameter(s) {unknown} have no counterpart on this target; it takes "
                             f"{sorted(_SCHEDULE_KEYS)}")
        if p.get("layer_kind", "matmul") != "matmul":
            raise ValueError(f"schedule parameters for layer kind '{p['layer_kind']}' are not supported")
        if ("wg_m" in p) != ("wg_n" in p):
            raise ValueError("wg_m and wg_n come together")

    def fn_compile(plan: list[PlanStep]) -> list[PlanStep]:
        gemms = [st for st in plan if st.kind == "hip.gemm"]
        if len(gemms) != len(parameters):
            raise ValueError(f"{len(parameters)} schedule parameter entries for a graph of {len(gemms)} matmul layers")
        for st, p in zip(gemms, parameters):
            sched = st.detail["schedule"]
            if "wg_m" in p:
                sched["tile"] = (int(p["wg_m"]), int(p["wg_n"]))
            if "split_k" in p:
                sched["split_k"] = int(p["split_k"])
            if all(key in p for key in ("m", "n", "k")):
                sched["mnk"] = (int(p["m"]), int(p["n"]), int(p["k"]))
            for key in ("transpose_a", "transpose_b"):
                if key in p:
                    sched[key] = bool(p[key])
        return plan

    return fn_compile


class HipBackend:
    """A PyTorch backend onto liblighthouse_hip.so; `backend(gm, example_inputs) -> JITFunction`."""

    def __init__(self, device: torch.device, fn_compile: Callable[[list[PlanStep]], list[PlanStep]] | None = None,
                 entry_func: str = "main", allow_torch_fallback: bool = False):
        self.device = device
        self.fn_compile = fn_compile
        self.entry_func = entry_func
        self.allow_torch_fallback = allow_torch_fallback
        self._last_jit_function: JITFunction | None = None

    @staticmethod
    def is_symbolic(t) -> bool:
        return isinstance(t, torch.SymInt) or (
            isinstance(t, torch.Tensor) and any(isinstance(d, torch.SymInt) for d in t.shape))

    def __call__(self, model: torch.fx.GraphModule, example_inputs: Sequence[torch.Tensor]) -> JITFunction:
        if any(self.is_symbolic(t) for t in example_inputs):
            raise ValueError("Dynamic shapes are not supported - consider using 'torch.compile(..., dynamic=False)'")
        placeholders, plan, output_spec = _Lowering(model, self.allow_torch_fallback).lower()
        if self.fn_compile is not None:
            plan = self.fn_compile(plan)
        jit_fn = JITFunction(placeholders, plan, output_spec, self.device, self.entry_func)
        self._last_jit_function = jit_fn
        return jit_fn

    @property
    def last_jit_function(self) -> JITFunction | None:
        return self._last_jit_function

    @property
    def jit_function(self) -> JITFunction:
        """The last JITFunction created (lighthouse/ingress/torch/compile.py:202-217); ValueError
        before the first compilation."""
        if self._last_jit_function is None:
            raise ValueError("The backend does not have a JITFunction available. Compile the torch model first.")
        return self._last_jit_function


def gpu_backend(fn_compile: Callable[[list[PlanStep]], list[PlanStep]] | None = None,
                device: torch.device | str = "cuda", entry_func: str = "main",
                allow_torch_fallback: bool = False) -> HipBackend:
    """GPU backend for `torch.compile(model, backend=gpu_backend(...), dynamic=False)`
    (lighthouse/ingress/torch/compile.py:453-496).  `fn_compile` may rewrite the lowered plan."""
    device = torch.device(device)
    assert device.type in ("cuda", "rocm", "xpu"), "Expected a GPU device"
    return HipBackend(device, fn_compile, entry_func, allow_torch_fallback)
