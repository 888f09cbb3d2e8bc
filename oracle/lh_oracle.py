"""CPU oracle for the Lighthouse GPU payloads (TEST INFRASTRUCTURE, never shipped).

This module restates, in plain numpy, the arithmetic that Lighthouse's payload
generators describe and that its example checkers verify.  It exists only to
check the HIP kernels: nothing under ``lighthouse_amd/`` may import it; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do.

Every function cites the reference file:line it follows (paths relative to the
Lighthouse source tree).  Functions accumulate in float64 and round once to
float32 unless the reference defines an explicit narrower rounding point; the
float64 result is the arbiter for tolerance checks because the summation order
of a GPU kernel differs from LLVM's scalar loop nest.

Parity status of each function (what pins it, see tests/test_oracle_*.py):
  matmul / lh-run input protocol : pinned by the reference's golden vector
      test/run/pipeline-check.mlir:1,16-31 and by library routines (torch.addmm).
  bf16 / e4m3 rounding            : pinned by torch.bfloat16 / torch.float8_e4m3fn
      casts and exhaustive code tables.
  attention, attention_online     : pinned by torch SDPA (float64), closed-form
      special cases and tile-size independence.
  layer_norm, softmax, gelu_tanh  : pinned by torch.nn.functional routines.
  nanogpt_block                   : pinned by an independent torch nn.Module
      restating the block of the benchmark configuration.
  nanogpt_forward                 : pinned by the same module stacked n times, then
      torch LayerNorm and Linear with non-trivial final gamma / beta / bias.
  ref_block_fused, ref_gpt_fused  : the reference's own checker restated
      (examples/xegpu/nanoGPT.py:84-135); pinned by an independent torch module
      (separate q/k/v projections, non-causal SDPA, ReLU MLP) in float64.
"""

from __future__ import annotations

import math

import numpy as np

# ----------------------------------------------------------------------------
# Narrow float formats
# ----------------------------------------------------------------------------


def f32_to_bf16_bits(x) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round-to-nearest-even.

    This is ``arith.truncf`` f32->bf16 as emitted by ``convert_float_type``
    (lighthouse/ingress/mlir_gen/generic.py:179-188).  NaN maps to a quiet NaN.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        sign = ((u >> 16) & 0x8000).astype(np.uint16)
        r = np.where(nan, sign | np.uint16(0x7FC0), r)
    return r.reshape(x.shape)


def bf16_bits_to_f32(bits) -> np.ndarray:
    """bfloat16 bit patterns (uint16) -> float32 (exact, ``arith.extf``)."""
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def round_bf16(x) -> np.ndarray:
    """Round float32 values through bfloat16 and back (f32 -> bf16 -> f32)."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def round_f16(x) -> np.ndarray:
    """Round through float16; mirrors ``_f16`` in examples/xegpu/nanoGPT.py:91-93."""
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x, elt: str) -> np.ndarray:
    """Round a float array to the named element type and return it as float32."""
    if elt == "f32":
        return np.asarray(x, dtype=np.float32)
    if elt == "bf16":
        return round_bf16(np.asarray(x, dtype=np.float32))
    if elt == "f16":
        return round_f16(x)
    raise ValueError(f"unsupported element type {elt}")


E4M3_MAX = 448.0


def e4m3_decode_table() -> np.ndarray:
    """All 256 OCP float8 e4m3fn codes as float32.

    Format: 1 sign, 4 exponent (bias 7), 3 mantissa; no infinities; the only
    NaN codes are 0x7f and 0xff; largest finite magnitude 448.
    """
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        s = -1.0 if code & 0x80 else 1.0
        e = (code >> 3) & 0xF
        m = code & 0x7
        if e == 0xF and m == 0x7:
            v = float("nan")
        elif e == 0:
            v = s * (m / 8.0) * 2.0 ** (-6)
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[code] = v
    return out


def e4m3_dequant(codes) -> np.ndarray:
    """uint8 e4m3fn codes -> float32."""
    return e4m3_decode_table()[np.asarray(codes, dtype=np.uint8)]


def e4m3_quant(x) -> np.ndarray:
    """float32 -> e4m3fn codes (uint8), saturating to +-448, round-to-nearest-even.

    Brute-force nearest search over the 127 non-negative finite codes with an
    explicit ties-to-even rule, so that the definition does not share any bit
    manipulation with the kernels it checks.
    """
    x = np.asarray(x, dtype=np.float32)
    table = e4m3_decode_table()
    pos = table[:127].astype(np.float64)  # codes 0..126 are finite and increasing
    a = np.minimum(np.abs(x.astype(np.float64)), E4M3_MAX)
    hi = np.searchsorted(pos, a, side="left")
    hi = np.clip(hi, 0, 126)
    lo = np.clip(hi - 1, 0, 126)
    d_hi = np.abs(pos[hi] - a)
    d_lo = np.abs(a - pos[lo])
    pick_lo = (d_lo < d_hi) | ((d_lo == d_hi) & (lo % 2 == 0))
    code = np.where(pick_lo, lo, hi).astype(np.uint8)
    code = np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)
    code = np.where(np.isnan(x), np.uint8(0x7F), code)
    return code


def quantize_per_tensor_e4m3(x):
    """Per-tensor quantisation of the benchmark's fp8 configuration.

    scale = amax(|x|)/448 ; q = e4m3(x/scale).  Returns (codes uint8, scale f32).
    """
    x = np.asarray(x, dtype=np.float32)
    scale = np.float32(np.max(np.abs(x)) / np.float32(E4M3_MAX))
    if scale == 0:
        scale = np.float32(1.0)
    return e4m3_quant(x / scale), scale


# ----------------------------------------------------------------------------
# lh-run input protocol
# ----------------------------------------------------------------------------


def lh_run_inputs(spec: str, seed: int) -> list[np.ndarray]:
    """Buffers ``lh-run --input-shape SPEC --seed SEED`` would create (float types only).

    Follows lighthouse/lh_run.py:82-85,116 and lighthouse/execution/init.py:53-80,
    93-118: legacy ``np.random.seed``, arguments generated in order, ``rnd`` is
    ``np.random.rand(*shape).astype(t)``, ``id`` is ``np.eye``.
    """
    np.random.seed(seed)
    dts = {"f32": np.float32, "f64": np.float64, "f16": np.float16}
    out = []
    for item in spec.split(","):
        parts = item.split("x")
        dims = [int(p) for p in parts[:-2]]
        dt = dts[parts[-2]]
        init = parts[-1]
        if init == "0":
            out.append(np.zeros(dims, dtype=dt))
        elif init == "1":
            out.append(np.ones(dims, dtype=dt))
        elif init == "rnd":
            out.append(np.random.rand(*dims).astype(dt))
        elif init == "id":
            out.append(np.eye(dims[0], dtype=dt))
        else:
            raise ValueError(init)
    return out


# ----------------------------------------------------------------------------
# GEMM payload
# ----------------------------------------------------------------------------


def matmul(
    a,
    b,
    c=None,
    bias=None,
    *,
    relu: bool = False,
    accumulate_c: bool = False,
    transpose_a: bool = False,
    transpose_b: bool = False,
    result_type: str = "f32",
    gelu: bool = False,
) -> np.ndarray:
    """``payload(out, A, B[, bias])`` of the matmul/MLP-layer generator.

    Follows ``emit_mlp_layer`` lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:110-156:
    accumulator starts from 0 or from C extended to the accumulator type
    (:121-130); optional logical transposes (:131-140); ``linalg.matmul``
    (named.py:5-7); bias extended to the accumulator type and broadcast over
    rows (:142-146, named.py:20-25); THEN conversion to ``result_type``
    (:147-149); THEN ReLU in the result type (:150-151, named.py:28-32).

    Inputs are float32 arrays holding values already representable in the A/B
    element type.  The result is float32 holding values of ``result_type``.
    ``gelu`` replaces ReLU by tanh-GELU computed on the accumulator-type value
    before the conversion (the activation of the benchmark's nanoGPT block; not
    part of the reference generator).
    """
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if transpose_a:
        a = a.T
    if transpose_b:
        b = b.T
    acc = a @ b
    if accumulate_c:
        acc = acc + np.asarray(c, dtype=np.float64)
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.float64)[None, :]
    if gelu:
        acc = gelu_tanh(acc, keep_f64=True)
    out = round_to(acc.astype(np.float32), result_type)
    if relu:
        out = np.maximum(out, np.float32(0.0))
    return out


def mlp(x, weights, biases=None, *, has_relu=False, relu_on_final_layer=False, transpose_a=False, transpose_b=False,
        accumulate_c=None, ab_type: str = "f32", result_type: str = "f32") -> np.ndarray:
    """``payload(out, in, W_0.., [b_0..])`` of ``generate_gpu_mlp_payload``
    lighthouse/ingress/mlir_gen/gpu_mlp_payload.py:66-105: every layer is the matmul payload's
    ``emit_mlp_layer``; hidden layers produce ``ab_type`` and get the ReLU, the last layer produces
    ``result_type`` (ReLU only with ``relu_on_final_layer``), ``transpose_a`` is applied to the
    first layer only, and only the last layer accumulates into the passed output
    (``accumulate_c`` = that initial output).  The example's checker
    examples/xegpu/mlp.py:47-88 chains the same steps in float32."""
    act = np.asarray(x, dtype=np.float32)
    n = len(weights)
    for i, w in enumerate(weights):
        last = i == n - 1
        act = matmul(
            act, w, c=accumulate_c if last else None, bias=None if biases is None else biases[i],
            relu=has_relu and (not last or relu_on_final_layer), accumulate_c=last and accumulate_c is not None,
            transpose_a=transpose_a and i == 0, transpose_b=transpose_b,
            result_type=result_type if last else ab_type)
    return act


def matmul_check_reference(c, a, b, bias, *, accumulate_c, has_bias, has_relu, truncate_to=None):
    """The example's own float32 checker, restated.

    Follows ``check_results`` examples/xegpu/matmul.py:252-261: everything in
    float32, C accumulated, bias added, ReLU, optional truncation.
    """
    f32 = np.float32
    d = a.astype(f32) @ b.astype(f32)
    if accumulate_c:
        d += c.astype(f32)
    if has_bias:
        d += bias.astype(f32)
    if has_relu:
        d = np.maximum(d, 0)
    if truncate_to is not None:
        d = round_to(d, truncate_to)
    return d


def matmul_fp8(a_codes, b_codes, scale_a, scale_b, result_type: str = "bf16") -> np.ndarray:
    """fp8 GEMM of the benchmark configuration: bf16((Aq.Bq)_f32 * (sa*sb)).

    Aq is [M,K] and Bq is [K,N] as e4m3fn codes.  Products of two e4m3 values are
    exact in float32; the float64 sum is rounded once to float32, multiplied by the
    float32 product of the two scales, then rounded to ``result_type``.
    """
    a = e4m3_dequant(a_codes).astype(np.float64)
    b = e4m3_dequant(b_codes).astype(np.float64)
    acc = (a @ b).astype(np.float32)
    s = np.float32(scale_a) * np.float32(scale_b)
    return round_to(acc * s, result_type)


# ----------------------------------------------------------------------------
# Attention payload
# ----------------------------------------------------------------------------


def attention(q, k, v, *, scale: float | None = None, causal: bool = False, result_type: str = "f32"):
    """``payload(out, Q, K, V)``: softmax(Q K^T * scale) V per (batch, head).

    Follows ``generate_gpu_attention_payload``
    lighthouse/ingress/mlir_gen/gpu_attention_payload.py:78-125 and the numpy
    checker examples/xegpu/fused_attention.py:61-95 (scale = 1/sqrt(head_dim),
    row max subtracted, exp, row sum, divide).  The causal variant adds -inf to
    the strictly upper triangle after scaling, as in examples/xegpu/nanoGPT.py:102-109.
    Computed in float64; returns float32 values rounded to ``result_type``.
    Shapes: [..., T, d] with any leading batch dims.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    s = np.einsum("...id,...jd->...ij", q, k) * scale
    if causal:
        tq, tk = s.shape[-2:]
        s = s + np.triu(np.full((tq, tk), -np.inf), k=1)
    s = s - s.max(axis=-1, keepdims=True)
    e = np.exp(s)
    w = e / e.sum(axis=-1, keepdims=True)
    o = np.einsum("...ij,...jd->...id", w, v)
    return round_to(o.astype(np.float32), result_type)


def attention_online(q, k, v, *, tile: int, scale: float | None = None, causal: bool = False, elt: str = "bf16"):
    """The fused (flash) form with its float32 state and rounding points.

    Follows ``ReplaceWithFusedAttentionOp``
    lighthouse/dialects/transform/transform_ext/ops/replace_with_fused_attention.py:
    init m=-inf, l=0, acc=0 in f32 (:337-344); per K/V tile: S = Q K_j^T in f32
    (:366-385), S *= scale (:386), m_new = max(m, rowmax S) (:389-398),
    P = exp(S - m_new) and l_j = rowsum(P) over the f32 P (:95-127),
    alpha = exp(m - m_new) (:411-412), l = l*alpha + l_j (:415-416),
    acc *= alpha (:419-421), acc += trunc_elt(P) V_j (:424-439); finally
    O = trunc_elt(acc / l) (:449-455).  A fully masked causal tile is skipped,
    which leaves the state unchanged (alpha = 1, P = 0).
    Single (T, d) problem; float32 arithmetic throughout.
    """
    f32 = np.float32
    q = np.asarray(q, dtype=f32)
    k = np.asarray(k, dtype=f32)
    v = np.asarray(v, dtype=f32)
    t, d = q.shape
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    scale = f32(scale)
    m = np.full((t,), -np.inf, dtype=f32)
    l = np.zeros((t,), dtype=f32)
    acc = np.zeros((t, d), dtype=f32)
    rows = np.arange(t)[:, None]
    for j0 in range(0, k.shape[0], tile):
        kj = k[j0 : j0 + tile]
        vj = v[j0 : j0 + tile]
        s = (q @ kj.T).astype(f32) * scale
        if causal:
            cols = np.arange(j0, j0 + kj.shape[0])[None, :]
            s = np.where(cols > rows, f32(-np.inf), s)
        m_new = np.maximum(m, s.max(axis=1))
        safe = np.where(np.isinf(m_new), f32(0), m_new)  # rows with nothing visible yet
        p = np.exp(s - safe[:, None]).astype(f32)
        l_j = p.sum(axis=1, dtype=f32)
        alpha = np.exp(np.where(np.isinf(m), f32(-np.inf), m - safe)).astype(f32)
        l = l * alpha + l_j
        acc = acc * alpha[:, None]
        acc = acc + (round_to(p, elt) @ vj).astype(f32)
        m = m_new
    return round_to(acc / l[:, None], elt)


# ----------------------------------------------------------------------------
# Row-wise payloads
# ----------------------------------------------------------------------------


def layer_norm(x, gamma, beta, eps: float = 1e-5, result_type: str = "f32") -> np.ndarray:
    """``payload(out, x, gamma, beta)``: two-pass row LayerNorm with biased variance.

    Follows ``emit_layer_norm_generics``
    lighthouse/ingress/mlir_gen/gpu_layer_norm_payload.py:15-87: sum, mean =
    sum * (1/N), sum of squared centred values, var = that * (1/N),
    (x-mean) * rsqrt(var+eps) * gamma + beta.  Same formula as the checker
    examples/xegpu/layer_norm.py:51-57.  float64 arithmetic, one rounding.
    """
    x = np.asarray(x, dtype=np.float64)
    n = x.shape[-1]
    mean = x.sum(axis=-1, keepdims=True) * (1.0 / n)
    c = x - mean
    var = (c * c).sum(axis=-1, keepdims=True) * (1.0 / n)
    y = c / np.sqrt(var + eps) * np.asarray(gamma, dtype=np.float64) + np.asarray(beta, dtype=np.float64)
    return round_to(y.astype(np.float32), result_type)


def softmax(x, result_type: str = "f32") -> np.ndarray:
    """``payload(out, x)``: row softmax (lighthouse/ingress/mlir_gen/gpu_softmax_payload.py:46-55;
    checker examples/xegpu/softmax.py:45-51)."""
    x = np.asarray(x, dtype=np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return round_to((e / e.sum(axis=-1, keepdims=True)).astype(np.float32), result_type)


def gelu_tanh(x, result_type: str = "f32", keep_f64: bool = False):
    """tanh-GELU: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).

    Not present in the reference; defined by the benchmark configuration
    (``torch.nn.functional.gelu(x, approximate="tanh")``).
    """
    x = np.asarray(x, dtype=np.float64)
    y = 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x**3)))
    if keep_f64:
        return y
    return round_to(y.astype(np.float32), result_type)


def bias_act(x, bias, relu: bool = False, result_type: str = "f32"):
    """Elementwise bias (+ReLU): examples/xegpu/nanoGPT_payload.py:141-163."""
    y = np.asarray(x, dtype=np.float32) + np.asarray(bias, dtype=np.float32)[None, :]
    if relu:
        y = np.maximum(y, np.float32(0))
    return round_to(y, result_type)


def residual_add(a, b, result_type: str = "f32"):
    """Elementwise residual add: examples/xegpu/nanoGPT_payload.py:166-181."""
    return round_to(np.asarray(a, dtype=np.float32) + np.asarray(b, dtype=np.float32), result_type)


# ----------------------------------------------------------------------------
# nanoGPT transformer block (benchmark configuration)
# ----------------------------------------------------------------------------


def nanogpt_block(x, p: dict, n_head: int, *, mode: str = "f32", eps: float = 1e-5, causal: bool = True,
                  activation: str = "gelu_tanh", bias_f32: bool = False):
    """Forward of one pre-LayerNorm GPT-2 block.

    Op order follows ``_emit_block_fused`` examples/xegpu/nanoGPT_payload.py:299-317
    and its numpy mirror examples/xegpu/nanoGPT.py:112-126, with the differences
    the benchmark configuration asks for: one fused QKV Linear (C -> 3C, with
    bias), causal attention, tanh-GELU MLP, batch dimension kept.

      ln1 = LN(x) ; qkv = ln1 Wqkv + bqkv ; att = causal MHA(q,k,v)
      a   = x + att Wo + bo
      ln2 = LN(a) ; h = gelu(ln2 W1 + b1) ; y = a + h W2 + b2

    ``mode="f32"``: every tensor float32 (float64 arithmetic here as arbiter).
    ``mode="bf16"`` / ``"f16"``: residual stream, LayerNorm statistics and all accumulators
    in float32; every matmul input (ln1, ln2, weights, q, k, v, attention
    probabilities, attention output, MLP hidden activations) rounded to the 16-bit type, i.e. the
    rounding points of examples/xegpu/nanoGPT.py:114-126.

    The reference's own block is reached with ``causal=False, activation="relu", bias_f32=True``
    and separate projections ``w_q / w_k / w_v`` in place of ``w_qkv`` (any bias may be None).

    x: [B, T, C].  p keys: ln1_g ln1_b w_qkv b_qkv w_o b_o ln2_g ln2_b w_fc b_fc w_proj b_proj,
    weights stored [in, out].  Returns float32 [B, T, C].
    """
    elt = mode
    r = lambda t: round_to(np.asarray(t, dtype=np.float32), elt)
    rb = (lambda t: None if t is None else np.asarray(t, dtype=np.float32)) if bias_f32 else (
        lambda t: None if t is None else r(t))
    gelu, relu = activation == "gelu_tanh", activation == "relu"
    if not (gelu or relu):
        raise ValueError(f"unknown activation {activation}")
    x = np.asarray(x, dtype=np.float32)
    bsz, t, c = x.shape
    hs = c // n_head
    x2 = x.reshape(bsz * t, c)
    ln1 = layer_norm(x2, p["ln1_g"], p["ln1_b"], eps, elt)
    if "w_qkv" in p:
        qkv = matmul(ln1, r(p["w_qkv"]), bias=rb(p.get("b_qkv")), result_type=elt)
    else:
        qkv = np.concatenate([matmul(ln1, r(p[k]), bias=rb(p.get("b" + k[1:])), result_type=elt)
                              for k in ("w_q", "w_k", "w_v")], axis=1)
    qkv = qkv.reshape(bsz, t, 3, n_head, hs)
    q = qkv[:, :, 0].transpose(0, 2, 1, 3)
    k = qkv[:, :, 1].transpose(0, 2, 1, 3)
    v = qkv[:, :, 2].transpose(0, 2, 1, 3)
    if elt == "f32":
        att = attention(q, k, v, causal=causal)
    else:
        att = _attention_rounded_p(q, k, v, causal=causal, elt=elt)
    att = att.transpose(0, 2, 1, 3).reshape(bsz * t, c)
    proj = matmul(att, r(p["w_o"]), bias=rb(p.get("b_o")), result_type="f32")
    a = x2 + proj
    ln2 = layer_norm(a, p["ln2_g"], p["ln2_b"], eps, elt)
    h = matmul(ln2, r(p["w_fc"]), bias=rb(p.get("b_fc")), gelu=gelu, relu=relu, result_type=elt)
    o = matmul(h, r(p["w_proj"]), bias=rb(p.get("b_proj")), result_type="f32")
    return (a + o).astype(np.float32).reshape(bsz, t, c)


def nanogpt_forward(x, layers, lnf_g, lnf_b, lm_w, lm_b, n_head: int, *, mode: str = "f32", eps: float = 1e-5,
                    causal: bool = True, activation: str = "gelu_tanh", bias_f32: bool = False):
    """n blocks, final LayerNorm, lm_head with bias: the tail of ``build_gpt_fused_payload``
    examples/xegpu/nanoGPT_payload.py:401-407 (``hf = LN(h)``, cast to the matmul input type,
    ``logits = hf W + b`` in float32) after ``nanogpt_block`` applied per layer (:399-400)."""
    elt = mode
    h = np.asarray(x, dtype=np.float32)
    for p in layers:
        h = nanogpt_block(h, p, n_head, mode=mode, eps=eps, causal=causal, activation=activation, bias_f32=bias_f32)
    bsz, t, c = h.shape
    hf = layer_norm(h.reshape(bsz * t, c), lnf_g, lnf_b, eps, elt)
    lm_bias = None if lm_b is None else (np.asarray(lm_b, dtype=np.float32) if bias_f32 else round_to(lm_b, elt))
    logits = matmul(hf, round_to(lm_w, elt), bias=lm_bias, result_type="f32")
    return logits.reshape(bsz, t, -1)


def ref_block_fused(x, w: dict, n_head: int, eps: float = 1e-5, causal: bool = False, elt: str = "f16"):
    """The reference's own block checker, ``numpy_ref_block_fused`` examples/xegpu/nanoGPT.py:112-126,
    for the block of ``_emit_block_fused`` examples/xegpu/nanoGPT_payload.py:299-317: separate
    ``wq/wk/wv`` projections without bias, non-causal attention by default, ReLU MLP, float32 biases
    and LayerNorm parameters, 16-bit weights.  x: [T, C] float32.  ``w`` keys as in the reference:
    g1 b1n wq wk wv wp bp g2 b2n w1 bb1 w2 bb2.

    Rounding points (``_f16`` there, ``elt`` here): ln1, q, k, v, the normalised attention weights
    (``_mha`` :95-109), the attention output, ln2, the MLP hidden activations; everything else float32
    (float64 sums here)."""
    r = lambda t: round_to(np.asarray(t, dtype=np.float32), elt)
    f64 = lambda t: np.asarray(t, dtype=np.float64)
    x = np.asarray(x, dtype=np.float32)
    t, c = x.shape
    hs = c // n_head

    def ln(v, g, b):  # _ln :85-88: population variance, division by sqrt
        v = f64(v)
        mu = v.mean(-1, keepdims=True)
        var = ((v - mu) ** 2).mean(-1, keepdims=True)
        return ((v - mu) / np.sqrt(var + eps) * f64(g) + f64(b)).astype(np.float32)

    ln1 = r(ln(x, w["g1"], w["b1n"]))
    q = r((f64(ln1) @ f64(w["wq"])).astype(np.float32))
    k = r((f64(ln1) @ f64(w["wk"])).astype(np.float32))
    v = r((f64(ln1) @ f64(w["wv"])).astype(np.float32))
    attn = np.zeros((t, c), np.float32)
    mask = np.triu(np.full((t, t), -np.inf), k=1) if causal else 0.0
    for h in range(n_head):  # _mha :95-109
        sl = slice(h * hs, (h + 1) * hs)
        s = (f64(q[:, sl]) @ f64(k[:, sl]).T) * (1.0 / hs**0.5) + mask
        e = np.exp(s - s.max(-1, keepdims=True))
        p = r((e / e.sum(-1, keepdims=True)).astype(np.float32))
        attn[:, sl] = (f64(p) @ f64(v[:, sl])).astype(np.float32)
    proj = (f64(r(attn)) @ f64(w["wp"]) + f64(w["bp"])).astype(np.float32)
    a = x + proj
    ln2 = r(ln(a, w["g2"], w["b2n"]))
    hh = np.maximum((f64(ln2) @ f64(w["w1"]) + f64(w["bb1"])).astype(np.float32), np.float32(0))
    o = (f64(r(hh)) @ f64(w["w2"]) + f64(w["bb2"])).astype(np.float32)
    return a + o


def ref_gpt_fused(x, layer_w, gf_g, gf_b, lmw, lmb, n_head: int, eps: float = 1e-5, elt: str = "f16"):
    """``numpy_ref_gpt_fused`` examples/xegpu/nanoGPT.py:128-135: the blocks above, the final
    LayerNorm rounded to the 16-bit type, ``logits = hf W + b`` in float32."""
    h = np.asarray(x, dtype=np.float32)
    for w in layer_w:
        h = ref_block_fused(h, w, n_head, eps, elt=elt)
    hf = layer_norm(h, gf_g, gf_b, eps, elt)
    return (hf.astype(np.float64) @ np.asarray(lmw, dtype=np.float64) + np.asarray(lmb, dtype=np.float64)).astype(np.float32)


def _attention_rounded_p(q, k, v, *, causal: bool, elt: str):
    """Attention with the probabilities rounded to ``elt`` before P.V and the row sum
    taken over the unrounded probabilities (the fused kernel's rounding points,
    replace_with_fused_attention.py:95-127,424-455), evaluated one-shot in float64."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    d = q.shape[-1]
    s = np.einsum("...id,...jd->...ij", q, k) * (1.0 / math.sqrt(d))
    if causal:
        tq, tk = s.shape[-2:]
        s = s + np.triu(np.full((tq, tk), -np.inf), k=1)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    l = e.sum(axis=-1, keepdims=True)
    o = np.einsum("...ij,...jd->...id", round_to(e.astype(np.float32), elt).astype(np.float64), v) / l
    return round_to(o.astype(np.float32), elt)


# ----------------------------------------------------------------------------
# Work counting (the numerators of every throughput figure)
# ----------------------------------------------------------------------------


def matmul_complexity(M, N, K, bias, relu, accumulate_c, nbytes_ab, nbytes_c):
    """examples/xegpu/matmul.py:41-64."""
    flops = 2 * M * N * K + (M * N if bias else 0) + (M * N if relu else 0)
    reads = (M * K + K * N) * nbytes_ab + (N * nbytes_c if bias else 0) + (M * N * nbytes_c if accumulate_c else 0)
    writes = M * N * nbytes_c
    return flops, reads, writes


def fused_attention_complexity(Z, H, n_ctx, n_head, nbytes):
    """examples/xegpu/fused_attention.py:26-43."""
    return Z * H * 4 * n_ctx * n_ctx * n_head, 3 * Z * H * n_ctx * n_head * nbytes, Z * H * n_ctx * n_head * nbytes


def layer_norm_complexity(M, N, nbytes):
    """examples/xegpu/layer_norm.py:27-40."""
    return 8 * M * N, (M * N + 2 * N) * nbytes, M * N * nbytes
