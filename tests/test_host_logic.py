"""Host-side mirror of the reference's op surface: argument rules that need no GPU."""
import numpy as np
import pytest
import torch

from conftest import load_package


def _cpu_args(B=4, N=6, L=5, K=3):
    x = torch.zeros(B, N)
    lookup = torch.zeros(L, K, dtype=torch.int32)
    w = torch.zeros(L, K)
    return x, lookup, w


def test_same_names_as_the_reference_binding():
    # sparse/ops/fixed_fan_in_ops.py:15-28
    pkg = load_package()
    for name in ("fan_in_sparse_matmul", "fan_in_sparse_matmul_tp", "fan_in_sparse_matmul_grad",
                 "fan_in_sparse_matmul_grad_tp"):
        assert callable(getattr(pkg, name))
    import ecml23_sparse_amd        # alias registered by the package itself
    assert ecml23_sparse_amd is pkg


def test_no_cpu_fallback():
    pkg = load_package()
    x, lookup, w = _cpu_args()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.fan_in_sparse_matmul(x, lookup, w)


def test_shape_rules_of_the_op_shape_functions():
    # tfsparse/cc/ops/fixed_fan_in_ops.cpp:14-53: rank 2 everywhere, lookup.shape == weights.shape,
    # out_grad.shape == [B, L]
    pkg = load_package()
    ops = pkg.fixed_fan_in_ops
    x, lookup, w = _cpu_args()
    with pytest.raises(ValueError, match="rank 2"):
        ops._check_inputs(x[0], lookup, w, False)
    with pytest.raises(ValueError, match="equal shapes"):
        ops._check_inputs(x, lookup[:, :2], w, False)
    with pytest.raises(TypeError):
        ops._check_inputs(x.double(), lookup, w, False)
    with pytest.raises(TypeError):
        ops._check_inputs(x, lookup.long(), w, False)


def test_synthetic_lookup_laws():
    pkg = load_package()
    from ecml23_sparse_amd import synth
    g = torch.Generator().manual_seed(1)
    idx = synth.make_lookup(500, 32, 768, generator=g)
    assert idx.dtype == torch.int32 and idx.shape == (500, 32)
    assert int(idx.min()) >= 0 and int(idx.max()) < 768
    srt = np.sort(idx.numpy(), axis=1)
    assert (srt[:, 1:] != srt[:, :-1]).all()                      # distinct inside each row
    wide = synth.make_lookup(300, 72, 65536, generator=g, sorted_rows=True).numpy()
    assert (wide[:, 1:] > wide[:, :-1]).all()
    rep = synth.make_lookup(200, 16, 8, distinct=False, generator=g).numpy()
    assert (np.sort(rep, axis=1)[:, 1:] == np.sort(rep, axis=1)[:, :-1]).any()


def test_synthetic_inputs_shapes_and_bytes():
    load_package()
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS["c2"]
    t = synth.make_inputs(cfg, seed=42, num_units=1000)
    assert t["features"].shape == (128, 768) and float(t["features"].min()) == 0.0
    assert t["lookup"].shape == (1000, 32) and t["weights"].shape == (1000, 32) and t["out_grad"].shape == (128, 1000)
    assert abs(float(t["weights"].std()) - 32 ** -0.5) < 0.01
    tt = synth.make_inputs(cfg, seed=42, num_units=1000, transposed=True)
    assert torch.equal(tt["features"].t(), t["features"])
    b = synth.algorithmic_bytes(cfg)
    # 515.0 MB per pass at 670,091 labels x fan-in 32 x 768 inputs x batch 128
    assert b["forward"] == b["input_grad"] == b["weight_grad"] == 515_023_104
    c3 = synth.make_inputs(synth.CONFIGS["c3"], num_units=10)["features"]
    assert torch.allclose(c3.norm(dim=1), torch.ones(256), atol=1e-5) and float(c3.min()) >= 0


def test_layer_constructor_arithmetic():
    """connections from sparsity (sparse/layer.py:173-177), fan-in = connections // units
    (sparse/custom_layer.py:46), argument errors; no kernel runs."""
    pkg = load_package()
    L = pkg.custom_layer.StratifiedRewireLayerV2
    layer = L(100, 64, sparsity=0.75, device="cpu")
    assert layer.connections == int(100 * 64 * 0.25) == 1600 and layer.fan_in == 16
    assert layer.kernel_weights.shape == (1600,) and layer.kernel_indices.shape == (1600,)
    assert int(layer.kernel_indices.min()) >= 0 and int(layer.kernel_indices.max()) < 64
    limit = (6.0 / (2 * 1600)) ** 0.5
    assert float(layer.kernel_weights.detach().abs().max()) <= limit
    assert layer.bias.shape == (100,) and float(layer.bias.detach().abs().sum()) == 0.0
    assert L(10, 8, connections=40, use_bias=False, device="cpu").bias is None
    with pytest.raises(ValueError):
        L(10, 8, connections=40, sparsity=0.5, device="cpu")
    with pytest.raises(ValueError):
        L(10, 8, connections=45, device="cpu")
    with pytest.raises(ValueError):
        L(10, 8, sparsity=1.5, device="cpu")
    with pytest.raises(RuntimeError):          # the product path needs the GPU: no CPU fallback
        layer(torch.zeros(2, 64))


def test_tensorflow_shim_declares_the_reference_ops():
    # The op library a maintainer builds against ROCm TensorFlow (csrc/tf/ffi_tf_ops.cc) must declare the four ops
    # exactly as tfsparse/cc/ops/fixed_fan_in_ops.cpp:55-93 does (names, attrs, inputs, outputs: the Python binding
    # sparse/ops/fixed_fan_in_ops.py:9-40 is generated from them) and register the sixteen kernels of
    # tfsparse/cc/kernels/register.cpp:79-109 (eight GPU, eight CPU).  TensorFlow is not in this image: the files are checked as text.
    import os
    import re

    from conftest import ROOT
    src = open(os.path.join(ROOT, "ecml23-sparse_amd", "csrc", "tf", "ffi_tf_ops.cc")).read()
    code = re.sub(r"//[^\n]*", "", src)
    fwd = re.search(r"#define FFI_DECLARE_FORWARD_OP\(NAME, TRANSPOSED\)(.*?)\n#define", code, re.S).group(1)
    grad = re.search(r"#define FFI_DECLARE_GRAD_OP\(NAME, TRANSPOSED\)(.*?)\n\n", code, re.S).group(1)

    def parts(text):
        return (re.findall(r'\.Attr\("([^"]+)"\)', text), re.findall(r'\.Input\("([^"]+)"\)', text),
                re.findall(r'\.Output\("([^"]+)"\)', text))

    assert parts(fwd) == (["T: type", "I: type"], ["features: T", "lookup: I", "weights: T"], ["result: T"])
    assert parts(grad) == (["T: type", "I: type"], ["features: T", "lookup: I", "weights: T", "output: T"],
                           ["feature_grad: T", "weight_grad: T"])
    declared = re.findall(r'FFI_DECLARE_(FORWARD|GRAD)_OP\("(\w+)", (true|false)\);', code)
    assert declared == [("FORWARD", "FanInSparseMatmul", "false"), ("FORWARD", "FanInSparseMatmulTp", "true"),
                        ("GRAD", "FanInSparseMatmulGrad", "false"), ("GRAD", "FanInSparseMatmulGradTp", "true")]
    kernels = re.findall(r'FFI_REGISTER_GPU\("(\w+)", (\w+), (\w+), (true|false)\);', code)
    assert len(kernels) == 8
    # ... and the eight CPU kernels of register.cpp:79-80,88-89,97-98,106-107, in the second source of the same target
    cpu_src = open(os.path.join(ROOT, "ecml23-sparse_amd", "csrc", "tf", "ffi_tf_cpu_ops.cc")).read()
    cpu_code = re.sub(r"//[^\n]*", "", cpu_src)
    cpu_kernels = re.findall(r'FFI_REGISTER_CPU\("(\w+)", (\w+), (\w+), (true|false)\);', cpu_code)
    assert len(cpu_kernels) == 8 and len(set(kernels)) + len(set(cpu_kernels)) == 16
    for op, transposed in (("FanInSparseMatmul", "false"), ("FanInSparseMatmulTp", "true"),
                           ("FanInSparseMatmulGrad", "false"), ("FanInSparseMatmulGradTp", "true")):
        for ids in ("int32", "uint32"):
            assert (op, "FanInSparseMatmulGradGpuOp" if "Grad" in op else "FanInSparseMatmulGpuOp", ids, transposed) in kernels
            assert (op, "FanInSparseMatmulGradCpuOp" if "Grad" in op else "FanInSparseMatmulCpuOp", ids, transposed) in cpu_kernels
    # the compute stream is taken as the reference takes it (forward.cu:50, backward.cu:63: the Eigen GPU device's stream,
    # present in every TensorFlow 2.x), not through an accessor of recent releases only
    assert "eigen_device<Eigen::GpuDevice>().stream()" in code
    assert "platform_specific_handle" not in code and "op_device_context" not in code
    # both sources are in the CMake target
    cmake = open(os.path.join(ROOT, "ecml23-sparse_amd", "csrc", "CMakeLists.txt")).read()
    assert re.search(r"add_library\(sparseops SHARED tf/ffi_tf_ops\.cc tf/ffi_tf_cpu_ops\.cc\)", cmake)
    assert "host/ffi_host_kernels.cc" in cmake
    assert "DEVICE_GPU" in code and 'TypeConstraint<float>("T")' in code
    # no arithmetic in the shim: its Compute bodies end in exactly one C-ABI call each
    assert code.count("ffi_forward_f32(") == 1 and code.count("ffi_backward_f32(") == 1
    # and the default CMake build does not depend on TensorFlow
    cm = open(os.path.join(ROOT, "ecml23-sparse_amd", "csrc", "CMakeLists.txt")).read()
    assert "if(FFI_TF_INCLUDE_DIR AND FFI_TF_LIBRARY)" in cm and "tf/ffi_tf_ops.cc" in cm


def test_host_kernels_match_the_oracle():
    # the product's own CPU implementation behind the DEVICE_CPU kernels (csrc/host/ffi_host_kernels.cc, host pointers,
    # no GPU): the reference's shape grid (testing/test.cpp:50-59), both layouts, work split into ranges the way an op's
    # thread pool would split it; gates as for the GPU kernels (1e-5 forward, 1e-4 gradients)
    import ctypes

    import numpy as np

    import oracle
    from conftest import REFERENCE_SHAPES, load_package, reference_law_inputs, rel_err
    lib = load_package()._lib.lib()
    ptr = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    for (B, N, L, K) in [s for s in REFERENCE_SHAPES if s[2] <= 20000] + [(5, 7, 11, 3)]:
        x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=L + K)
        for tp in (0, 1):
            xin = np.ascontiguousarray(x.T) if tp else x
            out = np.full((B, L), np.nan, dtype=np.float32)
            gx = np.full(xin.shape, np.nan, dtype=np.float32)
            gw = np.full((L, K), np.nan, dtype=np.float32)
            cuts = [0, L // 3, L]
            for a, b in zip(cuts[:-1], cuts[1:]):
                assert lib.ffi_host_forward_f32(ptr(xin), ptr(lookup), ptr(w), ptr(out), B, N, L, K, tp, a, b) == 0
                assert lib.ffi_host_backward_f32(ptr(xin), ptr(lookup), ptr(w), ptr(g), None, ptr(gw), B, N, L, K, tp, a, b, 0, 0) == 0
            bcuts = [0, B // 2, B]
            for a, b in zip(bcuts[:-1], bcuts[1:]):
                assert lib.ffi_host_backward_f32(ptr(xin), ptr(lookup), ptr(w), ptr(g), ptr(gx), None, B, N, L, K, tp, 0, 0, a, b) == 0
            assert rel_err(out, oracle.forward(xin, lookup, w, transposed=bool(tp))) <= 1e-5
            o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=bool(tp))
            assert rel_err(gw, o_gw) <= 1e-4 and rel_err(gx, o_gx) <= 1e-4
    # argument checks
    one = ctypes.c_void_p(16)
    assert lib.ffi_host_forward_f32(None, one, one, one, 1, 1, 1, 1, 0, 0, 1) == -1
    assert lib.ffi_host_forward_f32(one, one, one, one, 1, 1, 1, 1, 0, 0, 2) == -8
    bad = np.array([[3]], dtype=np.int32); f1 = np.ones((1, 1), dtype=np.float32)
    assert lib.ffi_host_forward_f32(ptr(f1), ptr(bad), ptr(f1), ptr(f1.copy()), 1, 1, 1, 1, 0, 0, 1) == -6
