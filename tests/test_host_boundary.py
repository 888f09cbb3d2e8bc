"""Host-side behaviour of the drop-in boundary (no GPU needed): descriptor discovery, target
overrides, argument parsing, memref packing, C ABI symbols and error paths."""

import ctypes
import os
import re
from pathlib import Path
from unittest import mock

import numpy as np
import pytest

from lighthouse_amd import _lib, pipeline
from lighthouse_amd.execution import (GPUMemoryManager, InitType, KernelArgument, KernelArgumentParser, Runner,
                                      TargetInfo, TorchMemoryManager)
from lighthouse_amd.execution.memory_manager import ExternalMemoryManager
from lighthouse_amd.ingress import (generate_gpu_attention_payload, generate_gpu_layer_norm_payload,
                                    generate_gpu_matmul_fp8_payload, generate_gpu_matmul_payload,
                                    generate_gpu_softmax_payload)
from lighthouse_amd.pipeline import Descriptor, PipelineDescriptor, string_to_type
from lighthouse_amd.utils import memref as mr
from lighthouse_amd.utils import numpy as lnp

ROOT = Path(__file__).resolve().parent.parent
FIXTURES = Path(__file__).parent / "fixtures" / "pipeline"
INTERNAL, EXTERNAL = str(FIXTURES / "internal"), str(FIXTURES / "external")


def _norm(path):
    if path is None:
        return None
    for tag, root in (("EXTERNAL", EXTERNAL), ("INTERNAL", INTERNAL)):
        if path.startswith(root):
            return f"{tag}/{os.path.relpath(path, root)}"
    return path


def test_find_pipeline_discovery_paths():
    """The scenarios of the reference's test/pipeline/find_pipeline.py:38-108."""
    x86 = lambda feats: TargetInfo(arch="x86_64", features=feats)
    with mock.patch.object(pipeline.finder, "DESCRIPTORS_REPO", INTERNAL):
        f, feat = pipeline.find_pipeline_file(x86(["amx_bf16"]), "matmul", "bf16")
        assert (_norm(f), feat) == ("INTERNAL/x86_64/amx_bf16/matmul/bf16.yaml", "amx_bf16")
        f, feat = pipeline.find_pipeline_file(x86([]), "matmul", "f32")
        assert (_norm(f), feat) == ("INTERNAL/x86_64/matmul/f32.yaml", None)
        f, feat = pipeline.find_pipeline_file(x86([]), "matmul", "f32", base_path=EXTERNAL)
        assert (_norm(f), feat) == ("EXTERNAL/x86_64/matmul/f32.yaml", None)
        f, feat = pipeline.find_pipeline_file(x86([]), "matvec", "f32", base_path=EXTERNAL)
        assert (_norm(f), feat) == ("INTERNAL/x86_64/matvec/f32.yaml", None)
        f, feat = pipeline.find_pipeline_file(x86([]), "matmul", "f32", base_path="/lh/does/not/exist")
        assert (_norm(f), feat) == ("INTERNAL/x86_64/matmul/f32.yaml", None)
        assert pipeline.find_pipeline_file(x86([]), "no_such_pipeline", "f32") == (None, None)
        assert pipeline.find_pipeline_file(x86([]), "", "f32") == (None, None)
        assert pipeline.find_pipeline_file(None, "matmul", "f32") == (None, None)


def test_packaged_gfx950_descriptors():
    t = TargetInfo(arch="gfx950")
    assert t.is_gpu() and t.is_supported("mfma")
    for pipe, dtypes in {"matmul": ["f32", "bf16", "f16", "f8E4M3FN"], "attention": ["bf16", "f16", "f32"],
                         "layer_norm": ["f32", "bf16"], "softmax": ["f32"], "nanogpt_block": ["f32", "bf16"]}.items():
        for dt in dtypes:
            path, feat = pipeline.find_pipeline_file(t, pipe, dt)
            assert path is not None and feat is None, (pipe, dt)
            stages = PipelineDescriptor(Descriptor(path)).kernel_stages()
            assert len(stages) == 1 and hasattr(_lib.load(), f"lh_hip_payload_{stages[0].entry}")
    # Every packaged file name is kebab/identifier case like the reference's check_yaml_filenames hook expects.
    for f in (Path(pipeline.finder.DESCRIPTORS_REPO)).rglob("*.yaml"):
        assert re.fullmatch(r"[A-Za-z0-9_-]+\.yaml", f.name)
    assert pipeline.find_pipeline_file(TargetInfo(arch="x86_64", features=[]), "matmul", "bf16") == (None, None)


def test_target_info_override_semantics():
    """The scenarios of the reference's test/execution/target_info_host_override.py:6-69."""
    TargetInfo.reset_host_cache()
    before = TargetInfo.host()
    feats = ["amx_tile"]
    with TargetInfo.override(features=feats, arch="x86_64"):
        feats.append("unexpected")
        a, b = TargetInfo.host(), TargetInfo.host()
        assert (a.arch, a.features, a is b) == ("x86_64", ["amx_tile"], False)
        with TargetInfo.override(features=["avx2"], arch="aarch64"):
            n = TargetInfo.host()
            assert (n.arch, n.features) == ("aarch64", ["avx2"])
        r = TargetInfo.host()
        assert (r.arch, r.features) == ("x86_64", ["amx_tile"])
    with TargetInfo.override(features=["sse4_2"], arch="x86_64"):
        assert TargetInfo.host().features == ["sse4_2"]
    with TargetInfo.override(features=["avx512f"]):
        h = TargetInfo.host()
        assert h.arch == before.arch and h.features == ["avx512f"] and h.vector_register_width_bits == 512
    with TargetInfo.override(arch="x86_64"):
        h = TargetInfo.host()
        assert h.arch == "x86_64" and h.features == before.features
    after = TargetInfo.host()
    assert (after.arch, after.features) == (before.arch, before.features)
    assert TargetInfo.host() is TargetInfo.host()


def test_descriptor_grammar():
    d = Descriptor("sched.py[gen=f,seq=s]{k=4 flag tiles=[8,16] name=abc}")
    assert d.basename == "sched.py" and d.args == {"gen": "f", "seq": "s"}
    assert d.opts == {"k": 4, "flag": True, "tiles": [8, 16], "name": "abc"}
    assert d.is_transform() and not d.is_pass()
    assert str(Descriptor("x.mlir", args={"a": 1}, opts={"b": True, "c": 2})) == "x.mlir[a=1]{b c=2}"
    assert Descriptor("convert-linalg-to-loops").is_pass()
    assert string_to_type("None") is None and string_to_type("TRUE") is True and string_to_type("1.5") == 1.5
    assert string_to_type("(1,a)") == (1, "a") and string_to_type("[]") == [] and string_to_type("") == ""
    with pytest.raises(ValueError):
        Descriptor("no_such_file.yaml", type="include", base_path=str(FIXTURES))


def test_pipeline_descriptor_include_and_variables(tmp_path):
    (tmp_path / "inner.yaml").write_text("Pipeline:\n  - kernel: \"elementwise{kind=$kind dtype=f32}\"\n")
    (tmp_path / "outer.yaml").write_text(
        "Pipeline:\n  - pass: canonicalize\n  - include: \"inner.yaml{kind=$k}\"\n  - kernel: matmul{tile_m=$tm}\n")
    pd = PipelineDescriptor(Descriptor(str(tmp_path / "outer.yaml"), opts={"k": "gelu", "tm": 128}))
    kinds = [(s.type, s.basename) for s in pd.get_stages()]
    assert kinds == [("pass", "canonicalize"), ("kernel", "elementwise"), ("kernel", "matmul")]
    ks = pd.kernel_stages()
    assert ks[0].params == {"kind": "gelu", "dtype": "f32"} and ks[1].params == {"tile_m": 128}
    assert [s.basename for s in pd.unsupported_stages()] == ["canonicalize"]
    (tmp_path / "empty.yaml").write_text("Pipeline: []\n")
    with pytest.raises(ValueError):
        PipelineDescriptor(Descriptor(str(tmp_path / "empty.yaml"), type="include"))
    (tmp_path / "bad.yaml").write_text("Pipeline:\n  - frobnicate: x\n")
    with pytest.raises(ValueError):
        PipelineDescriptor(Descriptor(str(tmp_path / "bad.yaml"), type="include"))


def test_kernel_argument_parser():
    """lighthouse/execution/init.py:26-118: grammar, errors and the random protocol."""
    np.random.seed(123)
    a, b, c = KernelArgumentParser.parse_all("16x64xf32xrnd,64x32xf32x1,16x32xf32x0")
    np.random.seed(123)
    np.testing.assert_array_equal(a.arg, np.random.rand(16, 64).astype(np.float32))
    assert b.arg.dtype == np.float32 and (b.arg == 1).all() and (c.arg == 0).all() and c.dims == [16, 32]
    ident = KernelArgumentParser.parse("4x4xf64xid")
    np.testing.assert_array_equal(ident.arg, np.eye(4))
    bf = KernelArgumentParser.parse("8x8xbf16x1").arg
    assert lnp.elem_name(bf.dtype) == "bf16" and (lnp.bf16_to_f32(bf) == 1).all()
    np.random.seed(5)
    r = KernelArgumentParser.parse("3x3xbf16xrnd").arg
    np.random.seed(5)
    np.testing.assert_array_equal(np.asarray(r).view(np.uint16), np.asarray(lnp.f32_to_bf16(np.random.rand(3, 3))).view(np.uint16))
    for bad in ("4x4xf32xwhat", "4xqx f32x0", "4x4xq99x0", "4x5xf32xid", "0x4xf32x0"):
        with pytest.raises(ValueError):
            KernelArgumentParser.parse(bad)
    with pytest.raises(ValueError):
        KernelArgument([], np.float32, InitType.ZERO)


def test_memref_descriptors_and_packed_args():
    a = np.zeros((4, 6), np.float32)[:, ::2]
    d = mr.get_ranked_memref_descriptor(a)
    assert list(d.shape) == [4, 3] and list(d.strides) == [6, 2] and d.offset == 0 and d.aligned == a.ctypes.data
    packed = mr.to_packed_args([d, 7])
    assert len(packed) == 2
    back = ctypes.cast(packed[0], ctypes.POINTER(ctypes.POINTER(type(d)))).contents.contents
    assert list(back.shape) == [4, 3] and back.aligned == a.ctypes.data
    assert ctypes.cast(packed[1], ctypes.POINTER(ctypes.c_int64)).contents.value == 7
    m = mr.make_memref(1024, (2, 3, 4))
    assert list(m.strides) == [12, 4, 1] and mr.memref_num_elements(m) == 24
    import torch

    t = torch.zeros(5, 8)[:, 2:6]
    td = mr.torch_to_memref(t)
    assert list(td.shape) == [5, 4] and list(td.strides) == [8, 1] and td.aligned == t.data_ptr()
    assert mr.make_nd_memref_descriptor(2) is mr.make_nd_memref_descriptor(2)


def test_dtype_tables():
    assert lnp.mlir_to_numpy_dtype("f32") == np.float32 and lnp.numpy_to_mlir_type(np.dtype(np.float16)) == "f16"
    assert lnp.elem_name(lnp.bfloat16) == "bf16" and lnp.elem_name(lnp.float8_e4m3fn) == "f8E4M3FN"
    with pytest.raises(ValueError):
        lnp.mlir_to_numpy_dtype("f128")
    with pytest.raises(ValueError):
        lnp.elem_name(np.dtype(np.uint16))
    x = np.array([1.0, -2.5, 3.0e-3, 1e30], np.float32)
    import torch

    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(np.asarray(lnp.f32_to_bf16(x)).view(np.uint16), ref)
    q = lnp.astype(np.array([1.0, 500.0, -0.3], np.float32), "f8E4M3FN")
    np.testing.assert_array_equal(lnp.to_float32(q), [1.0, 448.0, -0.3125])


def test_c_abi_exports_every_declared_symbol():
    header = (ROOT / "include" / "lighthouse_hip.h").read_text()
    declared = set(re.findall(r"\b(lh_hip_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    assert declared == set(_lib.PROTOTYPES), declared ^ set(_lib.PROTOTYPES)
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.lh_hip_last_error() is not None
    n = ctypes.c_int32(-1)
    assert lib.lh_hip_device_count(ctypes.byref(n)) == 0 and n.value >= 0


def test_c_abi_argument_validation_without_gpu():
    """Validation happens before any device work, so it is observable on a machine with no GPU."""
    lib = _lib.load()
    z = _lib.Strides3(0, 0, 0)
    assert lib.lh_hip_gemm(None, None, None, None, 4, 4, 4, 4, 4, 4, _lib.F32, _lib.F32, 0, None) == _lib.LH_ERR_INVALID
    assert b"null" in lib.lh_hip_last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.lh_hip_gemm(p, p, p, None, 0, 4, 4, 4, 4, 4, _lib.F32, _lib.F32, 0, None) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_gemm(p, p, p, None, 4, 4, 4, 2, 4, 4, _lib.F32, _lib.F32, 0, None) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_gemm(p, p, p, None, 4, 4, 4, 4, 4, 4, _lib.F32, _lib.F32, 1, None) == _lib.LH_ERR_INVALID  # bias flag, no bias
    assert lib.lh_hip_gemm(p, p, p, None, 4, 4, 4, 4, 4, 4, _lib.F64, _lib.F64, 0, None) == _lib.LH_ERR_UNSUPPORTED
    assert lib.lh_hip_gemm(p, p, p, None, 4, 4, 4, 4, 4, 4, _lib.BF16, _lib.F16, 0, None) == _lib.LH_ERR_UNSUPPORTED
    assert lib.lh_hip_gemm(p, p, p, None, 4, 4, 4, 4, 4, 4, _lib.F32, _lib.F32, 1 << 9, None) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_attention(p, p, p, p, 1, 1, 128, 512, z, z, z, z, 1.0, 0, _lib.BF16, None) == _lib.LH_ERR_UNSUPPORTED
    assert lib.lh_hip_attention(p, p, p, p, 1, 1, 100, 64, z, z, z, z, 1.0, 0, _lib.BF16, None) == _lib.LH_ERR_INVALID  # row stride 0
    assert lib.lh_hip_attention(p, p, p, p, 0, 1, 100, 64, z, z, z, z, 1.0, 0, _lib.BF16, None) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_layer_norm(p, p, p, p, 0, 8, 1e-5, _lib.F32, _lib.F32, None) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_nanogpt_block(p, p, None, 1, 1, 8, 2, 1e-5, _lib.F32, None, p, 0, None) == _lib.LH_ERR_INVALID
    with pytest.raises(ValueError):
        _lib.check(_lib.LH_ERR_INVALID, "x")
    with pytest.raises(RuntimeError):
        _lib.check(_lib.LH_ERR_RUNTIME, "x")
    attrs = _lib.MatmulAttrs(_lib.F32, _lib.F32, 0)
    assert lib.lh_hip_payload_matmul(None, 3, ctypes.byref(attrs)) == _lib.LH_ERR_INVALID
    d = mr.make_memref(p.value, (4, 4))
    bad = mr.make_memref(p.value, (5, 4))
    assert lib.lh_hip_payload_matmul(mr.to_packed_args([d, d]), 2, ctypes.byref(attrs)) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_payload_matmul(mr.to_packed_args([d, bad, d]), 3, ctypes.byref(attrs)) == _lib.LH_ERR_INVALID
    assert lib.lh_hip_payload_benchmark(b"nope", mr.to_packed_args([d, d, d]), 3, ctypes.cast(ctypes.byref(attrs), ctypes.c_void_p),
                                        None, 0, 0) == _lib.LH_ERR_INVALID


def test_payload_generators_and_runner_errors():
    m = generate_gpu_matmul_payload("payload", 64, 32, 16, "bf16", "f32", has_bias=True, has_relu=True,
                                    result_type="bf16", transpose_b=True)
    fn = m.lookup("payload")
    assert [a.shape for a in fn.args] == [(64, 32), (64, 16), (32, 16), (32,)] and fn.outputs == [0]
    assert [a.elem for a in fn.args] == ["bf16"] * 4
    assert fn.attrs.flags == _lib.GEMM_HAS_BIAS | _lib.GEMM_HAS_RELU | _lib.GEMM_TRANSPOSE_B
    assert fn.flops == 2 * 64 * 32 * 16 + 2 * 64 * 32
    assert "lh_hip_payload_matmul" in str(m)
    with pytest.raises(ValueError):
        generate_gpu_matmul_payload("p", 8, 8, 8, "bf16", "bf16")  # accumulator must be f32
    with pytest.raises(ValueError):
        generate_gpu_matmul_payload("p", 8, 8, 8, "i8", "f32")
    with pytest.raises(ValueError):
        m.lookup("other")
    att = generate_gpu_attention_payload("payload", 4, 16, 2048, 64, "bf16", causal=True).lookup("payload")
    assert att.flops == 34359738368 and abs(att.attrs.scale - 0.125) < 1e-7 and att.attrs.causal == 1
    ln = generate_gpu_layer_norm_payload("payload", 8192, 768, "f32").lookup("payload")
    assert ln.bytes_moved == (8192 * 768 + 2 * 768) * 4 + 8192 * 768 * 4
    assert generate_gpu_softmax_payload("payload", 4, 8, "f32").lookup("payload").entry == "elementwise"
    assert generate_gpu_matmul_fp8_payload("p", 16, 8, 32, 0.5, 0.25).lookup("p").args[1].elem == "f8E4M3FN"

    with pytest.raises(ValueError):
        Runner("not a module")
    with pytest.raises(ValueError):
        Runner(m, shared_libs=["libdoes_not_exist.so"])
    r = Runner(m, mem_manager_cls=dict)
    bufs = [lnp.f32_to_bf16(np.zeros(a.shape)) for a in fn.args]
    with pytest.raises(ValueError, match="Unsupported mem_manager_cls"):
        r.execute("payload", bufs)
    with pytest.raises(ValueError):
        Runner(m).execute("payload", None)
    with pytest.raises(ValueError):
        Runner(m).execute("payload", bufs[:3])
    with pytest.raises(ValueError):
        Runner(m).execute("payload", [np.zeros(a.shape, np.float32) for a in fn.args])  # wrong element type
    with pytest.raises(ValueError):
        Runner(m).execute("payload", ["x"] * 4)
    with pytest.raises(NotImplementedError):
        TorchMemoryManager().alloc()
    assert issubclass(TorchMemoryManager, ExternalMemoryManager) and Runner.payload_benchmark_function_name == "__benchmark"
    assert Runner.get_bench_wrapper_schedule("payload") == "payload"
    Runner.make_function_callable(m, "payload")


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("LIGHTHOUSE_HIP_LIBRARY", "/nonexistent/liblighthouse_hip.so")
    with pytest.raises(ValueError, match="Could not find shared library"):
        _lib.load()


def test_schedule_parameters_container(tmp_path):
    """lighthouse/schedule/parameters.py: a verified list of per-layer dictionaries with a JSON round trip."""
    from lighthouse_amd.schedule import ScheduleParameters

    params = ScheduleParameters([{"layer_kind": "matmul", "m": 4096, "n": 4096, "k": 4096}])
    params[0].update({"wg_m": 256, "wg_n": 256})
    params.append({"layer_kind": "matmul", "wg_tile": [128, 128], "relu": True})
    assert len(params) == 2 and [p["layer_kind"] for p in params] == ["matmul", "matmul"]
    for bad, match in (("matmul", "must be a dictionary"), ({"wg_m": 1}, "layer_kind"), ({"layer_kind": 3}, "must be a string"),
                       ({"layer_kind": "matmul", "x": object()}, "values must be"), ({"layer_kind": "matmul", 1: 2}, "keys must be")):
        with pytest.raises(ValueError, match=match):
            params.append(bad)
        with pytest.raises(ValueError, match=match):
            ScheduleParameters([bad])
    with pytest.raises(ValueError, match="list of dictionaries"):
        ScheduleParameters({"layer_kind": "matmul"})
    path = tmp_path / "p.json"
    params.to_json(path)
    with pytest.raises(FileExistsError):
        params.to_json(path)
    params.to_json(path, overwrite=True)
    again = ScheduleParameters.from_json(str(path))
    assert list(again) == list(params)
    del again[1]
    again.insert(0, {"layer_kind": "attention"})
    assert [p["layer_kind"] for p in again] == ["attention", "matmul"] and len(ScheduleParameters(None)) == 0


def test_parameter_selector_database_then_cost_model(tmp_path):
    """lighthouse/schedule/xegpu/xegpu_parameter_selector.py:26-85: a shape in the database gets its
    entry, any other the cost model's first configuration; the result feeds the torch ingress."""
    from lighthouse_amd.ingress.torch import with_schedule_parameters
    from lighthouse_amd.schedule import HipParameterSelector, ScheduleParameters
    from lighthouse_amd.tuning import TileDB

    db = TileDB(str(tmp_path / "db.json"))
    db.record("bf16", 16, 8192, 8192, None, 25.0, 86.0, split_k=4)
    db.record("bf16", 8192, 768, 768, (256, 128), 20.0, 480.0)
    db.save()
    sel = HipParameterSelector(str(tmp_path / "db.json"))
    assert sel.get_parameters_dict((16, 8192, 8192)) == {
        "layer_kind": "matmul", "m": 16, "n": 8192, "k": 8192, "transpose_a": False, "transpose_b": False,
        "source": "database", "split_k": 4}
    hit = sel.get_parameters((8192, 768, 768))
    assert isinstance(hit, ScheduleParameters) and (hit[0]["wg_m"], hit[0]["wg_n"], hit[0]["source"]) == (256, 128, "database")
    miss = sel.get_parameters_dict((4096, 4096, 4096))
    assert (miss["wg_m"], miss["wg_n"], miss["source"]) == (256, 256, "cost model")
    assert sel.get_parameters_dict((8192, 768, 768), transpose_b=True)["source"] == "cost model"
    assert sel.get_parameters_dict((1024, 1024, 1024), dtype="f32")["wg_m"] in (128, 64)
    # a decode shape the library would cut along K: no tile request (it would switch the cut off)
    decode = sel.get_parameters_dict((128, 8192, 8192))
    assert decode["source"] == "library" and "wg_m" not in decode and "split_k" not in decode
    with pytest.raises(ValueError, match="did not return any valid"):
        sel.get_parameters_dict((100, 100, 100))
    layers = sel.get_parameters_for_layers([{"shape": (8192, 2304, 768)}, {"shape": (8192, 768, 3072)}])
    assert len(layers) == 2 and all(p["layer_kind"] == "matmul" for p in layers)
    with_schedule_parameters(layers)      # every key the selector writes is one the ingress accepts
    # the packaged database loads by default
    assert HipParameterSelector().get_parameters_dict((2048, 2048, 2048))["layer_kind"] == "matmul"


def test_torch_tensors_as_packed_arguments():
    """lighthouse/utils/torch.py:41-83: element strides of views, rank 0, integers among the tensors."""
    import torch

    from lighthouse_amd.utils.torch import to_memref, to_packed_args

    base = torch.arange(24, dtype=torch.float32).reshape(4, 6)
    view = base[:, 1:5].t()
    d = to_memref(view)
    assert d.aligned == view.data_ptr() and tuple(d.shape) == (4, 4) and tuple(d.strides) == (1, 6) and d.offset == 0
    scalar = to_memref(torch.tensor(3.0))
    assert not hasattr(scalar, "shape") and scalar.offset == 0
    packed = to_packed_args([base, 7, view])
    assert len(packed) == 3
    second = ctypes.cast(packed[1], ctypes.POINTER(ctypes.c_int64))
    assert second[0] == 7
    inner = ctypes.cast(packed[2], ctypes.POINTER(ctypes.POINTER(type(d))))
    assert tuple(inner[0][0].strides) == (1, 6)
