"""The torch front end rejects mismatched calls before any device work (host side; no GPU needed).

The C ABI sees pointers and sizes only: a wrong extent, dtype or layout that got through would read
or write outside a buffer.  Every rejection below is raised on CPU tensors; a well-formed call on CPU
tensors gets as far as the device check ("expected tensors on the GPU"), which shows that the shape
checks come first and pass.
"""

import ctypes

import pytest
import torch

from lighthouse_amd import _lib, ops
from lighthouse_amd.ingress import build_gpt_fused_payload

bf16, f32, f16 = torch.bfloat16, torch.float32, torch.float16
ON_GPU = "expected tensors on the GPU"


def z(*shape, dtype=f32):
    return torch.zeros(*shape, dtype=dtype)


def test_gemm_rejections():
    a, b = z(8, 16, dtype=bf16), z(16, 24, dtype=bf16)
    with pytest.raises(ValueError, match=ON_GPU):
        ops.gemm(a, b)
    with pytest.raises(ValueError, match="rows of K"):
        ops.gemm(a, z(17, 24, dtype=bf16))
    with pytest.raises(ValueError, match="rows of K"):
        ops.gemm(a, z(24, 17, dtype=bf16), transpose_b=True)
    with pytest.raises(ValueError, match="same dtype"):
        ops.gemm(a, z(16, 24))
    with pytest.raises(ValueError, match="out must have shape"):
        ops.gemm(a, b, out=z(8, 25, dtype=bf16))
    with pytest.raises(ValueError, match="float32 or have the A/B dtype"):
        ops.gemm(a, b, out=z(8, 24, dtype=f16))
    with pytest.raises(ValueError, match="innermost stride"):
        ops.gemm(a, b, out=z(24, 8, dtype=bf16).t())
    with pytest.raises(ValueError, match="innermost stride"):
        ops.gemm(a.t().contiguous().t(), b)
    with pytest.raises(ValueError, match=r"bias must have shape \[24\]"):
        ops.gemm(a, b, z(23, dtype=bf16))
    with pytest.raises(ValueError, match="bias must have the output dtype"):
        ops.gemm(a, b, z(24))
    with pytest.raises(ValueError, match="bias must be contiguous"):
        ops.gemm(a, b, z(48, dtype=bf16)[::2])
    with pytest.raises(ValueError, match="residual must be"):
        ops.gemm(a, b, residual=z(8, 23, dtype=bf16))
    with pytest.raises(ValueError, match="unsupported A/B dtype"):
        ops.gemm(z(8, 16, dtype=torch.float64), z(16, 24, dtype=torch.float64))
    with pytest.raises(ValueError, match="workspace must be"):
        ops.gemm(a, b, workspace=z(16))


def test_gemm_fp8_rejections():
    e4 = torch.float8_e4m3fn
    a, b = z(16, 128).to(e4), z(128, 256).to(e4)
    with pytest.raises(ValueError, match=ON_GPU):
        ops.gemm_fp8(a, b, 1.0, 1.0)
    with pytest.raises(ValueError, match="float8_e4m3fn"):
        ops.gemm_fp8(z(16, 128, dtype=bf16), b, 1.0, 1.0)
    with pytest.raises(ValueError, match="B has 127 rows"):
        ops.gemm_fp8(a, z(127, 256).to(e4), 1.0, 1.0)
    with pytest.raises(ValueError, match="out must have shape"):
        ops.gemm_fp8(a, b, 1.0, 1.0, out=z(16, 255, dtype=bf16))
    with pytest.raises(ValueError, match="bfloat16 or float32"):
        ops.gemm_fp8(a, b, 1.0, 1.0, out=z(16, 256, dtype=f16))
    with pytest.raises(ValueError, match="innermost stride"):
        ops.gemm_fp8(a, z(256, 128).to(e4).t(), 1.0, 1.0)


def test_row_and_elementwise_rejections():
    x = z(4, 64)
    with pytest.raises(ValueError, match=ON_GPU):
        ops.layer_norm(x, z(64), z(64))
    with pytest.raises(ValueError, match=r"gamma must have shape \[64\]"):
        ops.layer_norm(x, z(63), z(64))
    with pytest.raises(ValueError, match=r"beta must have shape \[64\]"):
        ops.layer_norm(x, z(64), z(65))
    with pytest.raises(ValueError, match="float32"):
        ops.layer_norm(x, z(64, dtype=bf16), z(64))
    with pytest.raises(ValueError, match="contiguous"):
        ops.layer_norm(z(64, 4).t(), z(64), z(64))
    with pytest.raises(ValueError, match="out must have shape"):
        ops.layer_norm(x, z(64), z(64), out=z(4, 32))
    with pytest.raises(ValueError, match="contiguous"):
        ops.softmax(z(64, 4).t())
    with pytest.raises(ValueError, match="shape and dtype"):
        ops.softmax(x, out=z(4, 64, dtype=bf16))
    with pytest.raises(ValueError, match="shape and dtype"):
        ops.gelu_tanh(x, out=z(4, 63))
    with pytest.raises(ValueError, match="contiguous"):
        ops.gelu_tanh(z(8, 64)[::2])
    with pytest.raises(ValueError, match=r"bias must have shape \[64\]"):
        ops.bias_act(x, z(4))
    with pytest.raises(ValueError, match="bias must be"):
        ops.bias_act(x, z(64, dtype=bf16))
    with pytest.raises(ValueError, match="second operand"):
        ops.add(x, z(4, 32))
    with pytest.raises(ValueError, match="second operand"):
        ops.add(x, z(4, 64, dtype=bf16))
    with pytest.raises(ValueError, match="cast: out"):
        ops.cast(x, bf16, out=z(4, 64))
    for fn in (lambda: ops.softmax(x), lambda: ops.gelu_tanh(x), lambda: ops.bias_act(x, z(64)), lambda: ops.add(x, x),
               lambda: ops.cast(x, bf16)):
        with pytest.raises(ValueError, match=ON_GPU):
            fn()


def test_attention_rejections():
    q = z(1, 2, 16, 64, dtype=bf16)
    with pytest.raises(ValueError, match=ON_GPU):
        ops.attention(q, q, q)
    with pytest.raises(ValueError, match="equal 4-D shape"):
        ops.attention(q, z(1, 2, 15, 64, dtype=bf16), q)
    with pytest.raises(ValueError, match="one dtype"):
        ops.attention(q, q.float(), q)
    with pytest.raises(ValueError, match="out must have the shape"):
        ops.attention(q, q, q, out=z(1, 2, 16, 32, dtype=bf16))
    with pytest.raises(ValueError, match="out must have the shape"):
        ops.attention(q, q, q, out=z(1, 2, 16, 64))
    with pytest.raises(ValueError, match="innermost stride"):
        ops.attention(q, q, z(1, 2, 64, 16, dtype=bf16).transpose(2, 3))


def _block(C=32, hidden=128, dtype=bf16, bias=bf16):
    return {"ln1_g": z(C), "ln1_b": z(C), "w_qkv": z(C, 3 * C, dtype=dtype), "b_qkv": z(3 * C, dtype=bias),
            "w_o": z(C, C, dtype=dtype), "b_o": z(C, dtype=bias), "ln2_g": z(C), "ln2_b": z(C),
            "w_fc": z(C, hidden, dtype=dtype), "b_fc": z(hidden, dtype=bias), "w_proj": z(hidden, C, dtype=dtype),
            "b_proj": z(C, dtype=bias)}


def test_nanogpt_rejections():
    x = z(2, 8, 32)
    with pytest.raises(ValueError, match=ON_GPU):
        ops.nanogpt_block(x, _block(), 4)
    with pytest.raises(ValueError, match="float32"):
        ops.nanogpt_block(x.to(bf16), _block(), 4)
    with pytest.raises(ValueError, match="contiguous"):
        ops.nanogpt_block(z(2, 32, 8).transpose(1, 2), _block(), 4)
    with pytest.raises(ValueError, match="multiple of n_head"):
        ops.nanogpt_block(x, _block(), 5)
    for name, bad in (("w_qkv", z(32, 95, dtype=bf16)), ("w_o", z(32, 32)), ("w_proj", z(128, 33, dtype=bf16)),
                      ("w_fc", z(128, 32, dtype=bf16).t())):
        p = _block()
        p[name] = bad
        with pytest.raises(ValueError, match=name):
            ops.nanogpt_block(x, p, 4)
    for name, bad in (("ln1_g", z(31)), ("ln2_b", z(32, dtype=bf16)), ("b_qkv", z(95, dtype=bf16)), ("b_fc", z(128, dtype=f16)),
                      ("b_proj", z(32))):  # the last: bias dtypes must agree within a block
        p = _block()
        p[name] = bad
        with pytest.raises(ValueError, match=name):
            ops.nanogpt_block(x, p, 4)
    p = _block()
    del p["w_qkv"]
    with pytest.raises(ValueError, match="w_qkv or all of"):
        ops.nanogpt_block(x, p, 4)
    with pytest.raises(ValueError, match="activation"):
        ops.nanogpt_block(x, _block(), 4, activation="silu")
    # separate projections, float32 biases, no qkv bias: the reference's layout is accepted
    p = _block(dtype=f16, bias=f32)
    del p["w_qkv"], p["b_qkv"]
    p.update(w_q=z(32, 32, dtype=f16), w_k=z(32, 32, dtype=f16), w_v=z(32, 32, dtype=f16))
    with pytest.raises(ValueError, match=ON_GPU):
        ops.nanogpt_block(x, p, 4, causal=False, activation="relu")
    # forward
    with pytest.raises(ValueError, match="lm_w"):
        ops.nanogpt_forward(x, [_block()], z(32), z(32), z(31, 50, dtype=bf16), None, 4)
    with pytest.raises(ValueError, match="lm_b"):
        ops.nanogpt_forward(x, [_block()], z(32), z(32), z(32, 50, dtype=bf16), z(49, dtype=bf16), 4)
    with pytest.raises(ValueError, match="every block must have lm_w's dtype"):
        ops.nanogpt_forward(x, [_block()], z(32), z(32), z(32, 50), None, 4)
    with pytest.raises(ValueError, match="same MLP width"):
        ops.nanogpt_forward(x, [_block(), _block(hidden=64)], z(32), z(32), z(32, 50, dtype=bf16), None, 4)
    with pytest.raises(ValueError, match="lnf_g"):
        ops.nanogpt_forward(x, [_block()], z(31), z(32), z(32, 50, dtype=bf16), None, 4)
    with pytest.raises(ValueError, match="out must be"):
        ops.nanogpt_forward(x, [_block()], z(32), z(32), z(32, 50, dtype=bf16), None, 4, out=z(2, 8, 49))
    with pytest.raises(ValueError, match=ON_GPU):
        ops.nanogpt_forward(x, [_block()], z(32), z(32), z(32, 50, dtype=bf16), z(50, dtype=bf16), 4)


def test_workspace_queries_run_without_a_gpu():
    """The size queries run the dispatch code with launches and allocations switched off."""
    lib = _lib.load()
    assert ops.gemm_workspace_bytes(4096, 4096, 4096, bf16) == 0
    # decode shape: eight f32 blocks of the K cut
    assert ops.gemm_workspace_bytes(16, 8192, 8192, bf16) == 8 * 16 * 8192 * 4
    # ragged N: padded copies of B and of the result
    assert ops.gemm_workspace_bytes(4096, 4100, 4096, bf16) >= (4096 * 4104 * 2) * 2
    assert ops.gemm_workspace_bytes(4096, 4096, 4096, bf16, transpose_a=True) == 4096 * 4096 * 2
    assert ops.gemm_workspace_bytes(1024, 1024, 1024, f32) == 0
    # a requested cut along K needs its own blocks, whatever the library would have chosen (four here)
    assert ops.gemm_workspace_bytes(128, 8192, 8192, bf16) == 4 * 128 * 8192 * 4
    assert ops.gemm_workspace_bytes(128, 8192, 8192, bf16, split_k=8) == 8 * 128 * 8192 * 4
    assert ops.gemm_workspace_bytes(128, 8192, 8192, bf16, split_k=1) == 0
    assert ops.gemm_workspace_bytes(16, 8192, 8192, bf16, tile=(128, 128)) == 0  # a tile request switches the cut off
    # the pointer-aware query counts the padded copy of an operand that is not 16-byte aligned
    fake = 1 << 20
    args = (1024, 1024, 1024, 1024, 1024, 1024, _lib.BF16, _lib.BF16, 0)
    assert lib.lh_hip_gemm_workspace_bytes_for(fake, fake, fake, None, *args) == 0
    assert lib.lh_hip_gemm_workspace_bytes_for(fake, fake + 2, fake, None, *args) >= 1024 * 1024 * 2
    assert ops.gemm_fp8_workspace_bytes(8192, 8192, 8192) == 0
    # attention: only a key range split between workgroups takes temporary memory
    assert ops.attention_workspace_bytes(4, 16, 2048, 64, bf16) == 0
    assert ops.attention_workspace_bytes(4, 16, 2048, 64, bf16, causal=True) == 0
    assert ops.attention_workspace_bytes(1, 1, 8192, 64, bf16) > 0
    assert ops.attention_workspace_bytes(1, 1, 8192, 64, bf16, kv_split=1) == 0
    assert ops.attention_workspace_bytes(1, 1, 8192, 64, f32) == 0
    assert ops.attention_workspace_bytes(1, 1, 8192, 128, bf16) == 0
    assert ops.gemm_fp8_workspace_bytes(16, 8192, 8192) > 0
    base = ops.nanogpt_block_workspace_bytes(8, 1024, 768, bf16)
    rows = 8 * 1024
    fixed = rows * 768 * (2 + 6 + 2 + 4) + rows * 3072 * 2
    assert fixed <= base <= fixed + (1 << 20)
    # a two-row batch runs its projections cut along K: the workspace carries those blocks too
    small = ops.nanogpt_block_workspace_bytes(1, 2, 768, bf16)
    assert small > 2 * 768 * (2 + 6 + 2 + 4) + 2 * 3072 * 2 + 4096
    o = _lib.NanoGPTBlockOpts(0, _lib.ACT_RELU, _lib.F32, 1024)
    fwd = lib.lh_hip_nanogpt_forward_workspace_bytes(1, 256, 256, 256, _lib.F16, ctypes.byref(o))
    blk = lib.lh_hip_nanogpt_block_workspace_bytes(1, 256, 256, _lib.F16, ctypes.byref(o))
    assert fwd >= blk + 2 * 256 * 256 * 4
    assert lib.lh_hip_nanogpt_block_workspace_bytes(1, 256, 256, _lib.F64, None) == 0  # unsupported type


def test_gpt_fused_payload_signature():
    """The argument list of build_gpt_fused_payload, examples/xegpu/nanoGPT_payload.py:333-351."""
    T, C, hidden, vocab, L = 256, 256, 1024, 256, 2
    fn = build_gpt_fused_payload("payload", T, C, hidden, vocab, L, 4).lookup("payload")
    assert fn.entry == "gpt_fused" and fn.outputs == [0]
    assert len(fn.args) == 2 + 13 * L + 4 + 1
    assert (fn.args[0].shape, fn.args[0].elem) == ((T, vocab), "f32")
    layer = [(a.shape, a.elem) for a in fn.args[2:15]]
    assert layer == [((C,), "f32"), ((C,), "f32"), ((C, C), "f16"), ((C, C), "f16"), ((C, C), "f16"), ((C, C), "f16"),
                     ((C,), "f32"), ((C,), "f32"), ((C,), "f32"), ((C, hidden), "f16"), ((hidden,), "f32"),
                     ((hidden, C), "f16"), ((C,), "f32")]
    assert [(a.shape, a.elem) for a in fn.args[-5:-1]] == [((C,), "f32"), ((C,), "f32"), ((C, vocab), "f16"), ((vocab,), "f32")]
    assert fn.args[-1].elem == "i8" and fn.args[-1].shape[0] > 0
    assert (fn.attrs.n_layer, fn.attrs.n_head, fn.attrs.causal, fn.attrs.dtype) == (L, 4, 0, _lib.F16)
