"""Host logic of the drop-in boundary, without a GPU: the C++ registry / dispatch / declare mirror
(compiled test program modelled on the reference's tests/cpp/test_op_dialect.cc) and the Python
operator front end's error behaviour."""
import subprocess
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def test_cpp_registry_dispatch_declare(native_libs, tmp_path):
    exe = tmp_path / "test_hip_dialect"
    d = ROOT / "raf_amd" / "csrc" / "dialect"
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", f"-I{d}", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "cpp" / "test_hip_dialect.cc"),
                    str(d / "registry.cc"), str(d / "hip_dialect.cc"), str(d / "device_api.cc"),
                    str(d / "memory_pool.cc"),
                    f"-L{native_libs.LIB_DIR}", "-lraf_hip_optim", f"-Wl,-rpath,{native_libs.LIB_DIR}",
                    "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ALL OK" in r.stdout


def test_cpp_ir_patterns_fuse_dialect_pass(native_libs, tmp_path):
    """Graph IR, dataflow patterns, the fuse-pattern registry, the FuseDialect pass on the traced SGD
    update and the dispatch of fused functions (tests/cpp/test_fuse_dialect.cc)."""
    exe = tmp_path / "test_fuse_dialect"
    d = ROOT / "raf_amd" / "csrc" / "dialect"
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", f"-I{d}", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "cpp" / "test_fuse_dialect.cc"),
                    str(d / "registry.cc"), str(d / "raf_ir.cc"), str(d / "hip_fusion.cc"),
                    str(d / "hip_dialect.cc"), str(d / "device_api.cc"), str(d / "memory_pool.cc"),
                    f"-L{native_libs.LIB_DIR}", "-lraf_hip_optim", f"-Wl,-rpath,{native_libs.LIB_DIR}",
                    "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ALL OK" in r.stdout


def test_cpp_graph_rewrites_multi_tensor_sgd_and_mixed_lans(native_libs, tmp_path):
    """The hip dialect's whole-graph rewrites on the traced SGD and LANS optimizers: expected graphs,
    variants that must stay as they are (tests/cpp/test_graph_rewrites.cc)."""
    exe = tmp_path / "test_graph_rewrites"
    d = ROOT / "raf_amd" / "csrc" / "dialect"
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", f"-I{d}", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "cpp" / "test_graph_rewrites.cc"),
                    str(d / "registry.cc"), str(d / "raf_ir.cc"), str(d / "hip_fusion.cc"),
                    str(d / "hip_dialect.cc"), str(d / "device_api.cc"), str(d / "memory_pool.cc"),
                    f"-L{native_libs.LIB_DIR}", "-lraf_hip_optim", f"-Wl,-rpath,{native_libs.LIB_DIR}",
                    "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ALL OK" in r.stdout


def test_traced_update_needs_a_rocm_device(native_libs):
    import torch
    from raf_amd import op
    from raf_amd._lib import RafError

    w = torch.zeros(8)
    with pytest.raises(RafError, match="no fuse pattern matched on device type cpu"):
        op.traced_sgd_update(w, torch.ones(8), torch.zeros(8), 0.1, 0.9)


def test_dispatch_lists_seen_from_python(native_libs):
    from raf_amd import op

    assert op.dispatch_list("raf.op.lans") == [("hip", "raf.op.hip.lans", 30)]
    assert op.dispatch_list("raf.op.sgd") == [("hip", "raf.op.hip.sgd", 30)]
    assert op.dispatch_list("raf.op.lans_mixed") == [("hip", "raf.op.hip.lans_mixed", 30)]
    for name in ("l2norm", "fuse_tensor", "defuse_tensor", "sgd_multi", "sgd_multi_mixed"):
        assert op.dispatch_list(f"raf.op.{name}") == [("hip", f"raf.op.hip.{name}", 30)]
    assert op.dispatch_list("raf.op.lans", op.DEV_CPU) == []
    with op.with_dialect("tvm"):
        assert op.dispatch_list("raf.op.sgd") == []
    assert op.dispatch_list("raf.op.sgd") == [("hip", "raf.op.hip.sgd", 30)]


def test_cpu_tensors_find_no_backend(native_libs):
    """No fallback: CPU tensors have no dialect to go to and the call fails like the reference's
    dispatcher does (src/impl/op.cc:173-179)."""
    from raf_amd import _lib, op

    x = torch.zeros(4, 4)
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.sgd"):
        op.sgd(x, x, x, 0.1, 0.9)
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.lans"):
        op.lans([x] * 4, torch.tensor(1.0), 1e-3, .9, .999, 1e-6, True, 0.01, True, True, True)


def test_declare_errors_reach_python(native_libs):
    from raf_amd import _lib, op

    x = torch.zeros(4, 4)
    with pytest.raises(_lib.RafError, match="differ in shape"):
        op.sgd(x, torch.zeros(4, 5), x, 0.1, 0.9)
    with pytest.raises(_lib.RafError, match="4n tensors"):
        op.lans([x] * 3, torch.tensor(1.0), 1e-3, .9, .999, 1e-6, True, 0.01, True, True, True)
    with pytest.raises(_lib.RafError, match="3n tensors"):
        op.sgd_multi([x] * 4, 0.1, 0.9)
    with pytest.raises(_lib.RafError, match="differ in shape"):
        op.sgd_multi([x, torch.zeros(4, 5), x], 0.1, 0.9)
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.sgd_multi"):
        op.sgd_multi([x] * 3, 0.1, 0.9)
    with pytest.raises(_lib.RafError, match="5n tensors"):
        op.lans_mixed([x] * 4, torch.tensor(1.0), 1e-3, .9, .999, 1e-6, True, 0.01, True, True, True)


def test_tensor_op_declares_reach_python(native_libs):
    """Declare-time behaviour of l2norm / fuse_tensor / defuse_tensor without a GPU: size check,
    the empty list, and no backend for CPU tensors."""
    from raf_amd import _lib, op

    x = torch.zeros(6)
    with pytest.raises(_lib.RafError, match="Input tensor size should be 7, got 6"):
        op.defuse_tensor(x, [3, 4], [3, 4], [1, 2])
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.defuse_tensor"):
        op.defuse_tensor(x, [2, 4], [2, 2, 2], [1, 3])
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.l2norm"):
        op.l2norm(x)
    with pytest.raises(_lib.RafError, match="Cannot find a valid dispatch for op raf.op.fuse_tensor"):
        op.fuse_tensor([x, x])
    assert op.fuse_tensor([]) is None  # declared as a no-op (src/op/declare/memory.cc:54-55)


def test_optimizer_front_end_argument_checks():
    from raf_amd import optim

    with pytest.raises(ValueError, match="Invalid learning rate"):
        optim.SGD([torch.zeros(2)], -0.1)
    with pytest.raises(ValueError, match="Invalid momentum"):
        optim.SGD([torch.zeros(2)], 0.1, -1)
    o = optim.LANS([torch.zeros(2)])
    assert (o.lr, o.beta1, o.beta2, o.eps, o.weight_decay) == (1e-3, 0.9, 0.999, 1e-6, 0.01)
    assert o._step == 1 and o.bias_correction and o.grad_averaging and o.mode and o.normalize_grad
    o.step()  # no gradients anywhere: nothing is dispatched, the step counter still advances
    assert o._step == 2


def test_shape_lists():
    from raf_amd import shapes

    base, large, gpt2 = (shapes.numels(f()) for f in (shapes.bert_base_shapes, shapes.bert_large_shapes,
                                                       shapes.gpt2_shapes))
    assert (len(base), sum(base)) == (199, 109_482_240)
    assert (len(large), sum(large), max(large)) == (391, 335_141_888, 31_254_528)
    assert (len(gpt2), sum(gpt2), max(gpt2)) == (580, 1_557_611_200, 80_411_200)
    c4 = shapes.log_uniform_numels()
    assert len(c4) == 2000 and min(c4) >= 1 and max(c4) <= 65536
    assert c4 == shapes.log_uniform_numels()  # seeded
