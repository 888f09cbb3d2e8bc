"""Payload generators of the HIP target.

The reference's generators build a linalg ``ir.Module`` that is later lowered by MLIR
(lighthouse/ingress/mlir_gen/gpu_*_payload.py).  This target runs hand-written kernels, so
a payload "module" is a plain description: for every function its name, the static types of
its arguments (output first, void return, as in the reference) and the C ABI entry point
plus attribute block that computes it.  Generator names and parameters follow the
reference so workload code reads the same; element types are names ("f32", "bf16", ...)
where the reference takes ``ir.Type`` objects.
"""

from __future__ import annotations

import ctypes
import math
from dataclasses import dataclass, field

from .. import _lib
from ..utils.numpy import elem_name, lh_dtype


@dataclass
class ArgSpec:
    shape: tuple[int, ...]
    elem: str
    writable: bool = False


@dataclass
class PayloadFunction:
    name: str
    entry: str                      # C entry point suffix: lh_hip_payload_<entry>
    attrs: ctypes.Structure
    args: list[ArgSpec]             # in the order the caller passes buffers
    flops: int = 0
    bytes_moved: int = 0
    # For each argument of the C entry point (output first), its position in `args`; None when the
    # function already has the entry point's order.  Set for functions read from MLIR text, whose
    # signature fixes the caller's order.
    arg_order: list[int] | None = None

    @property
    def outputs(self) -> list[int]:
        return [i for i, a in enumerate(self.args) if a.writable]


@dataclass
class PayloadModule:
    """A set of payload functions; what ``Runner`` executes."""

    functions: dict[str, PayloadFunction] = field(default_factory=dict)

    def add(self, fn: PayloadFunction) -> "PayloadModule":
        if fn.name in self.functions:
            raise ValueError(f"function '{fn.name}' already defined")
        self.functions[fn.name] = fn
        return self

    def lookup(self, name: str) -> PayloadFunction:
        if name not in self.functions:
            raise ValueError(f"no function named '{name}' in payload module")
        return self.functions[name]

    def __str__(self) -> str:
        lines = ["payload.module {"]
        for fn in self.functions.values():
            sig = ", ".join(
                f"memref<{'x'.join(str(d) for d in a.shape)}x{a.elem}>" + (" {writable}" if a.writable else "")
                for a in fn.args
            )
            lines.append(f"  func @{fn.name}({sig}) -> lh_hip_payload_{fn.entry}")
        lines.append("}")
        return "\n".join(lines)


def _single(fn: PayloadFunction) -> PayloadModule:
    return PayloadModule().add(fn)


def generate_gpu_matmul_payload(
    func_name: str,
    M: int,
    N: int,
    K: int,
    ab_type: str,
    c_type: str,
    transpose_a: bool = False,
    transpose_b: bool = False,
    has_bias: bool = False,
    has_relu: bool = False,
    accumulate_c: bool = False,
    result_type: str | None = None,
    has_gelu: bool = False,
) -> PayloadModule:
    """``payload(out, A, B[, bias])``; lighthouse/ingress/mlir_gen/gpu_matmul_payload.py:5-36.

    ``c_type`` is the accumulator type (must be f32 on this target); the output and bias
    have ``result_type`` when given, else ``c_type``.
    """
    ab, acc = elem_name(ab_type), elem_name(c_type)
    res = acc if result_type is None else elem_name(result_type)
    if acc != "f32":
        raise ValueError("Only f32 accumulation is supported on the HIP target")
    if ab not in ("f32", "bf16", "f16"):
        raise ValueError(f"Unsupported A/B element type {ab}")
    if res not in ("f32", ab):
        raise ValueError(f"result type {res} must be f32 or the A/B type {ab}")
    flags = 0
    flags |= _lib.GEMM_HAS_BIAS if has_bias else 0
    flags |= _lib.GEMM_HAS_RELU if has_relu else 0
    flags |= _lib.GEMM_HAS_GELU if has_gelu else 0
    flags |= _lib.GEMM_ACCUMULATE_C if accumulate_c else 0
    flags |= _lib.GEMM_TRANSPOSE_A if transpose_a else 0
    flags |= _lib.GEMM_TRANSPOSE_B if transpose_b else 0
    args = [
        ArgSpec((M, N), res, writable=True),
        ArgSpec((K, M) if transpose_a else (M, K), ab),
        ArgSpec((N, K) if transpose_b else (K, N), ab),
    ]
    if has_bias:
        args.append(ArgSpec((N,), res))
    sa, sc = _size(ab), _size(res)
    # examples/xegpu/matmul.py:41-64
    flops = 2 * M * N * K + (M * N if has_bias else 0) + (M * N if has_relu or has_gelu else 0)
    nbytes = (M * K + K * N) * sa + M * N * sc + (N * sc if has_bias else 0) + (M * N * sc if accumulate_c else 0)
    attrs = _lib.MatmulAttrs(lh_dtype(ab), lh_dtype(res), flags)
    return _single(PayloadFunction(func_name, "matmul", attrs, args, flops, nbytes))


def generate_gpu_mlp_payload(
    func_name: str,
    batch_size: int,
    input_size: int,
    output_size: int,
    hidden_layer_sizes: list[int],
    ab_type: str,
    acc_type: str,
    bias_type: str,
    result_type: str,
    transpose_a: bool = False,
    transpose_b: bool = False,
    has_bias: bool = False,
    has_relu: bool = False,
    accumulate_c: bool = False,
    relu_on_final_layer: bool = False,
) -> PayloadModule:
    """``payload(out, in, W_0 .. W_n[, bias_0 .. bias_n])``;
    lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:10-107.  Hidden activations have ``ab_type`` and
    get the ReLU; the last layer has ``result_type`` and gets it only with ``relu_on_final_layer``;
    ``transpose_a`` applies to the first layer's input, ``accumulate_c`` to the last layer."""
    ab, acc, bt, res = (elem_name(t) for t in (ab_type, acc_type, bias_type, result_type))
    if acc != "f32":
        raise ValueError("Only f32 accumulation is supported on the HIP target")
    if ab not in ("f32", "bf16", "f16"):
        raise ValueError(f"Unsupported A/B element type {ab}")
    if res not in ("f32", ab) or (has_bias and bt not in ("f32", ab)):
        raise ValueError(f"result type {res} and bias type {bt} must be f32 or the A/B type {ab}")
    sizes = [input_size, *hidden_layer_sizes, output_size]
    features = list(zip(sizes[:-1], sizes[1:]))
    args = [ArgSpec((batch_size, output_size), res, writable=True),
            ArgSpec((input_size, batch_size) if transpose_a else (batch_size, input_size), ab)]
    args += [ArgSpec((o, i) if transpose_b else (i, o), ab) for i, o in features]
    if has_bias:
        args += [ArgSpec((o,), bt) for _, o in features]
    flags = ((_lib.GEMM_HAS_BIAS if has_bias else 0) | (_lib.GEMM_HAS_RELU if has_relu else 0)
             | (_lib.GEMM_ACCUMULATE_C if accumulate_c else 0) | (_lib.GEMM_TRANSPOSE_A if transpose_a else 0)
             | (_lib.GEMM_TRANSPOSE_B if transpose_b else 0))
    attrs = _lib.MlpAttrs(lh_dtype(ab), lh_dtype(res), lh_dtype(bt if has_bias else res), flags, len(features),
                          1 if relu_on_final_layer else 0)
    # examples/xegpu/mlp.py sums the per-layer matmul complexity.
    flops = sum(2 * batch_size * i * o + (batch_size * o if has_bias else 0) for i, o in features)
    nbytes = sum((batch_size * i + i * o) * _size(ab) for i, o in features) + batch_size * output_size * _size(res)
    return _single(PayloadFunction(func_name, "mlp", attrs, args, flops, nbytes))


def generate_gpu_matmul_fp8_payload(
    func_name: str, M: int, N: int, K: int, scale_a: float, scale_b: float, result_type: str = "bf16"
) -> PayloadModule:
    """``payload(out, Aq, Bq)``: e4m3 inputs with per-tensor scales (no reference counterpart)."""
    res = elem_name(result_type)
    if res not in ("bf16", "f32"):
        raise ValueError("fp8 matmul result type must be bf16 or f32")
    args = [ArgSpec((M, N), res, writable=True), ArgSpec((M, K), "f8E4M3FN"), ArgSpec((K, N), "f8E4M3FN")]
    attrs = _lib.MatmulFp8Attrs(lh_dtype(res), float(scale_a), float(scale_b))
    return _single(PayloadFunction(func_name, "matmul_fp8", attrs, args, 2 * M * N * K,
                                   M * K + K * N + M * N * _size(res)))


def generate_gpu_attention_payload(
    func_name: str, Z: int, H: int, n_ctx: int, n_head: int, dtype: str, causal: bool = False
) -> PayloadModule:
    """``payload(out, Q, K, V)`` on [Z,H,n_ctx,n_head] tensors, scale 1/sqrt(n_head);
    lighthouse/ingress/mlir_gen/gpu_attention_payload.py:12-132 (``n_head`` is the head
    dimension there too).  ``causal`` adds the -inf upper-triangular mask."""
    dt = elem_name(dtype)
    if dt not in ("bf16", "f16", "f32"):
        raise ValueError(f"Unsupported attention element type {dt}")
    shape = (Z, H, n_ctx, n_head)
    args = [ArgSpec(shape, dt, writable=True)] + [ArgSpec(shape, dt) for _ in range(3)]
    attrs = _lib.AttentionAttrs(lh_dtype(dt), 1 if causal else 0, 1.0 / math.sqrt(n_head))
    flops = Z * H * 4 * n_ctx * n_ctx * n_head  # examples/xegpu/fused_attention.py:26-43
    if causal:
        flops //= 2
    return _single(PayloadFunction(func_name, "attention", attrs, args, flops, 4 * Z * H * n_ctx * n_head * _size(dt)))


def generate_gpu_layer_norm_payload(
    func_name: str, M: int, N: int, dtype: str, eps: float = 1e-5, result_type: str | None = None
) -> PayloadModule:
    """``payload(out, x, gamma, beta)``; lighthouse/ingress/mlir_gen/gpu_layer_norm_payload.py:90-143.
    gamma and beta are f32; ``result_type`` optionally fuses the conversion of the output."""
    dt = elem_name(dtype)
    res = dt if result_type is None else elem_name(result_type)
    args = [ArgSpec((M, N), res, writable=True), ArgSpec((M, N), dt), ArgSpec((N,), "f32"), ArgSpec((N,), "f32")]
    attrs = _lib.LayerNormAttrs(lh_dtype(dt), lh_dtype(res), float(eps))
    # examples/xegpu/layer_norm.py:27-40
    return _single(PayloadFunction(func_name, "layer_norm", attrs, args, 8 * M * N,
                                   M * N * _size(dt) + 2 * N * 4 + M * N * _size(res)))


def generate_gpu_softmax_payload(func_name: str, M: int, N: int, dtype: str) -> PayloadModule:
    """``payload(out, x)``; lighthouse/ingress/mlir_gen/gpu_softmax_payload.py:11-65."""
    return generate_gpu_elementwise_payload(func_name, "softmax", M, N, dtype)


_EW_KINDS = {"softmax": _lib.EW_SOFTMAX, "gelu": _lib.EW_GELU, "bias": _lib.EW_BIAS, "bias_relu": _lib.EW_BIAS,
             "add": _lib.EW_ADD, "cast": _lib.EW_CAST}


def generate_gpu_elementwise_payload(
    func_name: str, kind: str, M: int, N: int, dtype: str, dst_dtype: str | None = None
) -> PayloadModule:
    """Elementwise / row kernels of the nanoGPT payload builder
    (examples/xegpu/nanoGPT_payload.py:123-181) plus softmax and tanh-GELU."""
    if kind not in _EW_KINDS:
        raise ValueError(f"unknown elementwise kind '{kind}'")
    dt = elem_name(dtype)
    dst = dt if dst_dtype is None else elem_name(dst_dtype)
    args = [ArgSpec((M, N), dst if kind == "cast" else dt, writable=True), ArgSpec((M, N), dt)]
    if kind in ("bias", "bias_relu"):
        args.append(ArgSpec((N,), dt))
    if kind == "add":
        args.append(ArgSpec((M, N), dt))
    attrs = _lib.ElementwiseAttrs(_EW_KINDS[kind], lh_dtype(dt), lh_dtype(dst), 1 if kind == "bias_relu" else 0)
    flops = {"softmax": 5 * M * N}.get(kind, M * N)  # examples/xegpu/softmax.py:25-39
    nbytes = sum(_numel(a.shape) * _size(a.elem) for a in args)
    return _single(PayloadFunction(func_name, "elementwise", attrs, args, flops, nbytes))


def generate_nanogpt_block_payload(
    func_name: str, B: int, T: int, C: int, n_head: int, dtype: str, eps: float = 1e-5
) -> PayloadModule:
    """``payload(y, x, ln1_g, ln1_b, w_qkv, b_qkv, w_o, b_o, ln2_g, ln2_b, w_fc, b_fc, w_proj, b_proj,
    workspace)``: one pre-LayerNorm GPT-2 block (op order of ``_emit_block_fused``,
    examples/xegpu/nanoGPT_payload.py:299-317; fused QKV, causal, tanh-GELU)."""
    dt = elem_name(dtype)
    if dt not in ("f32", "bf16", "f16"):
        raise ValueError("nanoGPT block dtype must be f32, bf16 or f16")
    ws = int(_lib.load().lh_hip_nanogpt_block_workspace_bytes(B, T, C, lh_dtype(dt), None))
    args = [
        ArgSpec((B * T, C), "f32", writable=True), ArgSpec((B * T, C), "f32"),
        ArgSpec((C,), "f32"), ArgSpec((C,), "f32"),
        ArgSpec((C, 3 * C), dt), ArgSpec((3 * C,), dt),
        ArgSpec((C, C), dt), ArgSpec((C,), dt),
        ArgSpec((C,), "f32"), ArgSpec((C,), "f32"),
        ArgSpec((C, 4 * C), dt), ArgSpec((4 * C,), dt),
        ArgSpec((4 * C, C), dt), ArgSpec((C,), dt),
        ArgSpec((ws,), "i8", writable=False),
    ]
    attrs = _lib.NanoGPTBlockAttrs(lh_dtype(dt), int(n_head), int(B), int(T), float(eps))
    rows, hs = B * T, C // n_head
    flops = 2 * rows * C * 3 * C + 2 * B * n_head * T * T * hs + 2 * rows * C * C + 4 * rows * C * 4 * C
    return _single(PayloadFunction(func_name, "nanogpt_block", attrs, args, flops, 0))


def build_gpt_fused_payload(
    func_name: str, T: int, C: int, hidden: int, vocab: int, n_layer: int, H: int, eps: float = 1e-5,
    dtype: str = "f16", causal: bool = False,
) -> PayloadModule:
    """The reference's full nanoGPT forward, ``build_gpt_fused_payload``
    examples/xegpu/nanoGPT_payload.py:318-407, with its argument list: ``payload(out, x, per layer
    [g1, b1n, wq, wk, wv, wp, bp, g2, b2n, w1, bb1, w2, bb2], gf_g, gf_b, lmw, lmb)`` plus a trailing
    workspace (the reference allocates and frees its intermediates inside the payload, :407-408;
    here the caller's memory manager owns them).  Weights are 16-bit (``dtype``), LayerNorm
    parameters and biases f32, attention non-causal, MLP activation ReLU."""
    dt = elem_name(dtype)
    if dt not in ("f32", "bf16", "f16"):
        raise ValueError("nanoGPT dtype must be f32, bf16 or f16")
    opts = _lib.NanoGPTBlockOpts(1 if causal else 0, _lib.ACT_RELU, _lib.F32, int(hidden))
    ws = int(_lib.load().lh_hip_nanogpt_forward_workspace_bytes(1, T, C, vocab, lh_dtype(dt), ctypes.byref(opts)))
    per_layer = [ArgSpec((C,), "f32"), ArgSpec((C,), "f32"), ArgSpec((C, C), dt), ArgSpec((C, C), dt), ArgSpec((C, C), dt),
                 ArgSpec((C, C), dt), ArgSpec((C,), "f32"), ArgSpec((C,), "f32"), ArgSpec((C,), "f32"),
                 ArgSpec((C, hidden), dt), ArgSpec((hidden,), "f32"), ArgSpec((hidden, C), dt), ArgSpec((C,), "f32")]
    args = [ArgSpec((T, vocab), "f32", writable=True), ArgSpec((T, C), "f32")]
    for _ in range(n_layer):
        args += [ArgSpec(a.shape, a.elem) for a in per_layer]
    args += [ArgSpec((C,), "f32"), ArgSpec((C,), "f32"), ArgSpec((C, vocab), dt), ArgSpec((vocab,), "f32"),
             ArgSpec((ws,), "i8")]
    attrs = _lib.GptFusedAttrs(lh_dtype(dt), int(H), int(n_layer), 1 if causal else 0, float(eps))
    hs = C // H
    flops = n_layer * (2 * T * C * 3 * C + 4 * H * T * T * hs + 2 * T * C * C + 4 * T * C * hidden) + 2 * T * C * vocab
    return _single(PayloadFunction(func_name, "gpt_fused", attrs, args, flops, 0))


def _size(elem: str) -> int:
    return {"f32": 4, "bf16": 2, "f16": 2, "f8E4M3FN": 1, "f64": 8, "i8": 1}[elem]


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


# ---- payload modules by name --------------------------------------------------------------
# The reference's command line runs whatever MLIR module it is given (lighthouse/lh_run.py:103-127);
# for the payloads it ships no MLIR text of (attention, LayerNorm, softmax, the elementwise
# kernels, the nanoGPT block: its examples build them with the generators above), this target's
# command line accepts the generator call itself as the module: ``gen:KIND{key=value ...}`` with
# the generator's own keyword names, the descriptor grammar's option syntax.
_GENERATORS = {
    "matmul": (generate_gpu_matmul_payload, {"M", "N", "K", "ab_type", "c_type"},
               {"transpose_a", "transpose_b", "has_bias", "has_relu", "accumulate_c", "result_type", "has_gelu"}),
    "attention": (generate_gpu_attention_payload, {"Z", "H", "n_ctx", "n_head", "dtype"}, {"causal"}),
    "layer_norm": (generate_gpu_layer_norm_payload, {"M", "N", "dtype"}, {"eps", "result_type"}),
    "softmax": (generate_gpu_softmax_payload, {"M", "N", "dtype"}, set()),
    "elementwise": (generate_gpu_elementwise_payload, {"kind", "M", "N", "dtype"}, {"dst_dtype"}),
    "nanogpt_block": (generate_nanogpt_block_payload, {"B", "T", "C", "n_head", "dtype"}, {"eps"}),
}


def is_generated_module(spec: str) -> bool:
    return spec.startswith("gen:")


def generate_payload_module(spec: str, func_name: str) -> PayloadModule:
    """``gen:attention{Z=4 H=16 n_ctx=2048 n_head=64 dtype=bf16 causal}`` -> the module that
    ``generate_gpu_attention_payload(func_name, Z=4, ...)`` builds.  Unknown kinds, unknown or
    missing keys are errors."""
    from ..pipeline.descriptor import Descriptor

    desc = Descriptor(spec[len("gen:"):])
    kind, params = desc.basename, {**desc.args, **desc.opts}
    if kind not in _GENERATORS:
        raise ValueError(f"no payload generator named '{kind}'; known: {sorted(_GENERATORS)}")
    fn, required, optional = _GENERATORS[kind]
    unknown = sorted(set(params) - required - optional)
    missing = sorted(required - set(params))
    if unknown or missing:
        raise ValueError(f"gen:{kind}: " + "; ".join(
            ([f"unknown key(s) {unknown}"] if unknown else []) + ([f"missing key(s) {missing}"] if missing else []))
            + f" (it takes {sorted(required)} and optionally {sorted(optional)})")
    return fn(func_name, **params)


def default_input_shapes(fn: PayloadFunction) -> str:
    """The ``--input-shape`` string for a generated function when the caller gives none: every
    argument in order, outputs zero-filled, inputs uniform random (``rnd``), byte workspaces zero."""
    parts = []
    for a in fn.args:
        init = "0" if a.writable or a.elem == "i8" else "rnd"
        parts.append("x".join(str(d) for d in a.shape) + f"x{a.elem}x{init}")
    return ",".join(parts)
