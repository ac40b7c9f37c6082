"""The C-ABI libraries load and export exactly what include/*.h declares; argument validation and
host-only arithmetic work without a GPU.  No kernel is launched here."""
import ctypes
import re
from ctypes import c_int64, c_void_p
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent


def _declared(header: str):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rafhip_[a-z0-9_]+)\s*\(", text)))


def test_optim_header_symbols_all_exported_and_bound(native_libs):
    lib = native_libs.optim()
    names = _declared("rafhip_optim.h")
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in rafhip_optim.h but not exported"
    assert sorted(native_libs.OPTIM_SYMBOLS) == names, "ctypes table and header disagree"


def test_device_header_symbols_all_exported_and_bound(native_libs):
    lib = native_libs.optim()
    names = _declared("rafhip_device.h")
    assert len(names) == 18
    for n in names:
        assert hasattr(lib, n), f"{n} declared in rafhip_device.h but not exported"
    assert sorted(native_libs.DEVICE_SYMBOLS) == names


def test_dialect_header_symbols_all_exported_and_bound(native_libs):
    lib = native_libs.dialect()
    names = _declared("rafhip_dialect.h")
    for n in names:
        assert hasattr(lib, n), f"{n} declared in rafhip_dialect.h but not exported"
    assert sorted(native_libs.DIALECT_SYMBOLS) == names


def test_built_libraries_are_not_older_than_their_sources(native_libs):
    """GPU runs load the in-tree libraries as they are: a source edited after the last build would be
    tested and measured in its old form."""
    from raf_amd import build

    assert build.stale() == []


def test_status_and_dtype_codes_match_the_header(native_libs):
    text = (ROOT / "include" / "rafhip_optim.h").read_text()
    codes = dict(re.findall(r"\b(RAFHIP_(?:OK|ERR_[A-Z_]+|F16|F32|F64|BF16))\s*=\s*(\d+)", text))
    assert len([k for k in codes if k.startswith("RAFHIP_ERR_")]) == 6
    for name, value in codes.items():
        assert getattr(native_libs, name) == int(value), name
    slots = re.search(r"#define\s+RAFHIP_TABLE_SLOTS\s+(\d+)", text)
    assert slots and native_libs.RAFHIP_TABLE_SLOTS == int(slots.group(1))


def test_abi_version_and_struct_layout(native_libs):
    lib = native_libs.optim()
    assert lib.rafhip_abi_version() == 1
    assert ctypes.sizeof(native_libs.LansHParams) == 40
    hp = native_libs.LansHParams()
    lib.rafhip_lans_default_hparams(ctypes.byref(hp))
    # defaults of raf.optim.LANS, python/raf/optim/lans.py:44-55
    assert (hp.learning_rate, hp.beta1, hp.beta2, hp.eps) == tuple(
        float(np.float32(x)) for x in (1e-3, 0.9, 0.999, 1e-6))
    assert (hp.bias_correction, hp.grad_averaging, hp.mode, hp.normalize_grad) == (1, 1, 1, 1)
    assert hp.weight_decay == float(np.float32(0.01)) and hp.grad_unscale == 1.0


def test_sgd_argument_validation(native_libs):
    lib = native_libs.optim()
    assert lib.rafhip_sgd_f32(None, None, None, None, None, 0, 0.1, 0.9, None) == 0  # n == 0: no-op
    assert lib.rafhip_sgd_f32(None, None, None, None, None, -1, 0.1, 0.9, None) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert b"n = -1" in lib.rafhip_last_error()
    assert lib.rafhip_sgd_f32(None, None, None, None, None, 8, 0.1, 0.9, None) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert b"null" in lib.rafhip_last_error()


def test_lans_layout_query_is_host_arithmetic(native_libs):
    from raf_amd import kernels, shapes

    per_tensor = native_libs.optim().rafhip_lans_chunk_elements
    chunk = per_tensor(1)
    assert chunk % 1024 == 0 and per_tensor(1 << 22) % chunk == 0
    sizes = [0, 1, chunk - 1, chunk, chunk + 1, 10 * chunk + 3]
    chunks, ws = kernels.query_layout(sizes)
    assert chunks == sum(-(-n // chunk) for n in sizes) == 0 + 1 + 1 + 1 + 2 + 11
    assert ws % 256 == 0 and ws >= 32 * chunks + 64 * len(sizes)
    big = shapes.numels(shapes.bert_large_shapes())
    chunks, ws = kernels.query_layout(big)
    assert chunks == sum(-(-n // per_tensor(n)) for n in big)
    assert ws < 2 << 20  # no per-element scratch: under two megabytes for 335M elements
    assert kernels.query_layout([])[0] == 0
    lib = native_libs.optim()
    bad = (c_int64 * 2)(5, -3)
    assert lib.rafhip_lans_query_layout(2, bad, None, None) == native_libs.RAFHIP_ERR_INVALID_ARG


def test_lans_plan_argument_validation(native_libs):
    lib = native_libs.optim()
    h = c_void_p(None)
    one = (c_int64 * 1)(8)
    assert lib.rafhip_lans_plan_create(1, one, 7, ctypes.byref(h)) == native_libs.RAFHIP_ERR_UNSUPPORTED
    assert lib.rafhip_lans_plan_create(-1, one, 0, ctypes.byref(h)) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert lib.rafhip_lans_plan_create(1, None, 0, ctypes.byref(h)) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert lib.rafhip_lans_plan_create(1, one, 0, None) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert lib.rafhip_lans_workspace_bytes(None) < 0
    assert lib.rafhip_lans_step(None, None, None, None, None, None, 1, None, None, 0, None) == native_libs.RAFHIP_ERR_INVALID_ARG
    assert lib.rafhip_lans_plan_destroy(None) == 0


def test_product_fails_loudly_without_gpu(native_libs):
    """No CPU fallback: on a host without a GPU plan creation reports NO_DEVICE."""
    lib = native_libs.optim()
    if lib.rafhip_device_count() > 0:
        pytest.skip("a GPU is visible")
    h = c_void_p(None)
    one = (c_int64 * 1)(8)
    assert lib.rafhip_lans_plan_create(1, one, 0, ctypes.byref(h)) == native_libs.RAFHIP_ERR_NO_DEVICE
    assert not h.value


def test_package_has_no_oracle_or_cpu_fallback():
    """The product never imports the oracle."""
    for py in (ROOT / "raf_amd").rglob("*.py"):
        assert "oracle" not in py.read_text(), py
    for src in (ROOT / "raf_amd" / "csrc").rglob("*.*"):
        assert "oracle" not in src.read_text(), src


def test_sgd_kernel_isa_has_no_fused_multiply_add(tmp_path):
    """Bit-exactness of SGD hinges on four separate roundings: the compiled gfx950 code of sgd.hip
    must contain no FMA/MAC instruction of any width and no packed fp32 instruction (the 16-bit
    variant of the op may use packed half multiplies and adds: each is one correctly rounded
    operation per element)."""
    import shutil
    import subprocess

    from raf_amd import build

    if not shutil.which("hipcc") and not Path("/opt/rocm/bin/hipcc").exists():
        pytest.skip("hipcc not available")
    out = tmp_path / "sgd.s"
    subprocess.run([build.hipcc(), *build.HIP_FLAGS, f"-I{build.INCLUDE}", f"-I{build.CSRC}", "-S",
                    "--cuda-device-only", str(build.CSRC / "sgd.hip"), "-o", str(out)],
                   check=True, capture_output=True)
    asm = out.read_text()
    assert "sgd_vec4_kernel" in asm and "v_mul_f32" in asm
    assert not re.search(r"\bv_(fma|mac|fmac|mad|pk_fma|pk_mad)_", asm)
    assert not re.search(r"\bv_pk_(add|mul|fma)_f32", asm)
