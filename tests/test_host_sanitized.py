"""The host C++ layer (interface mirror, registries, memory pools, graph IR and passes, the `hip`
dialect's OpEnvs and the C window) built with AddressSanitizer and UndefinedBehaviorSanitizer and
exercised by the C++ test programs, on the CPU.  The kernel library is replaced by a stub of every
entry point its headers declare (each reports "no device"), so nothing here needs a GPU or HIP; the
reference builds its own library this way with RAF_USE_SANITIZER (cmake/modules/Sanitizer.cmake)."""
import os
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
DIALECT = ROOT / "raf_amd" / "csrc" / "dialect"
SAN_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer",
             "-static-libasan", "-g", "-O1"]

_DECL = re.compile(r"^(int|int32_t|int64_t|const char\*|void\*|void)\s+(rafhip_\w+)\s*\(([^;{]*?)\)\s*;", re.M | re.S)


def write_stub(path: Path, leave_out=()) -> int:
    """A definition for every function include/rafhip_optim.h and include/rafhip_device.h declare:
    status functions return RAFHIP_ERR_NO_DEVICE, counts 0, sizes -1, pointers NULL.  `leave_out`
    names functions a test program defines itself."""
    out = ['#include "rafhip_optim.h"', '#include "rafhip_device.h"', 'extern "C" {']
    n = 0
    for header in ("rafhip_optim.h", "rafhip_device.h"):
        text = re.sub(r"/\*.*?\*/", "", (ROOT / "include" / header).read_text(), flags=re.S)
        for ret, name, params in _DECL.findall(text):
            if name in leave_out:
                continue
            if name == "rafhip_device_count":
                body = "return 0;"
            elif name == "rafhip_abi_version":
                body = "return RAFHIP_ABI_VERSION;"
            elif ret == "int":
                body = "return RAFHIP_ERR_NO_DEVICE;"
            elif ret in ("int32_t", "int64_t"):
                body = "return -1;"
            elif ret == "const char*":
                body = 'return "stub of the kernel library: no device";'
            elif ret == "void*":
                body = "return 0;"
            else:
                body = ""
            out.append(f"{ret} {name}({' '.join(params.split())}) {{ {body} }}")
            n += 1
    out.append("}")
    path.write_text("\n".join(out) + "\n")
    from raf_amd import _lib

    declared = {line.split("(")[0].split()[-1] for line in out if "rafhip_" in line and "(" in line}
    assert declared | set(leave_out) == set(_lib.OPTIM_SYMBOLS) | set(_lib.DEVICE_SYMBOLS), \
        "the stub must cover the whole C ABI"
    return n


SOURCES = ["registry.cc", "raf_ir.cc", "hip_fusion.cc", "hip_dialect.cc", "device_api.cc", "memory_pool.cc",
           "c_api.cc"]


@pytest.fixture(scope="module")
def sanitized_objects(tmp_path_factory):
    """Every source of the host layer and the stub compiled once, instrumented; the test programs
    link what they need."""
    from concurrent.futures import ThreadPoolExecutor

    out = tmp_path_factory.mktemp("sanitized")
    stub = out / "rafhip_stub.cc"
    assert write_stub(stub) >= 50  # every entry point of the two headers

    def compile_one(src: Path) -> Path:
        obj = out / (src.stem + ".o")
        subprocess.run(["g++", "-std=c++17", "-Wall", *SAN_FLAGS, f"-I{DIALECT}", f"-I{ROOT / 'include'}", "-c",
                        str(src), "-o", str(obj)], check=True)
        return obj

    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(compile_one, [DIALECT / s for s in SOURCES] + [stub]))
    return {o.stem: o for o in objs}, out


def _build_and_run(sanitized_objects, program: str, sources):
    objs, out = sanitized_objects
    exe = out / program
    cmd = ["g++", "-std=c++17", "-Wall", *SAN_FLAGS, f"-I{DIALECT}", f"-I{ROOT / 'include'}",
           str(ROOT / "tests" / "cpp" / f"{program}.cc"), *[str(objs[Path(s).stem]) for s in sources],
           str(objs["rafhip_stub"]), "-o", str(exe)]
    subprocess.run(cmd, check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    r = subprocess.run([str(exe)], capture_output=True, text=True, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ALL OK" in r.stdout
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr and "LeakSanitizer" not in r.stderr


def test_registry_dispatch_declare_under_sanitizers(sanitized_objects):
    _build_and_run(sanitized_objects, "test_hip_dialect",
                   ["registry.cc", "hip_dialect.cc", "device_api.cc", "memory_pool.cc"])


def test_ir_patterns_and_fuse_pass_under_sanitizers(sanitized_objects):
    _build_and_run(sanitized_objects, "test_fuse_dialect",
                   ["registry.cc", "raf_ir.cc", "hip_fusion.cc", "hip_dialect.cc", "device_api.cc", "memory_pool.cc"])


def test_graph_rewrites_under_sanitizers(sanitized_objects):
    _build_and_run(sanitized_objects, "test_graph_rewrites",
                   ["registry.cc", "raf_ir.cc", "hip_fusion.cc", "hip_dialect.cc", "device_api.cc", "memory_pool.cc"])


def test_c_window_under_sanitizers(sanitized_objects):
    """The C entry points of rafhip_dialect.h driven from a small C++ program: makes that fail for
    want of a device, traced graphs that are built, fused and printed, pools on the cpu device."""
    _build_and_run(sanitized_objects, "test_c_window", SOURCES)


def test_op_envs_rebind_when_an_address_moves(sanitized_objects):
    """LansHipEnv / SgdMultiHipEnv against a kernel library that records its calls: the same
    tuple, a new tuple over the same tensors (the VM's pattern), a replaced field, moved storage,
    alternating gradient allocations (tests/cpp/test_lans_env_binding.cc)."""
    objs, out = sanitized_objects
    program = (ROOT / "tests" / "cpp" / "test_lans_env_binding.cc").read_text()
    own = set(re.findall(r"^(?:int|int64_t|void|const char\*)\s+(rafhip_\w+)\s*\(", program, re.M))
    assert {"rafhip_lans_plan_bind", "rafhip_lans_step_bound", "rafhip_sgd_multi_step"} <= own
    stub = out / "rafhip_stub_partial.cc"
    write_stub(stub, leave_out=own)
    exe = out / "test_lans_env_binding"
    subprocess.run(["g++", "-std=c++17", "-Wall", *SAN_FLAGS, f"-I{DIALECT}", f"-I{ROOT / 'include'}",
                    str(ROOT / "tests" / "cpp" / "test_lans_env_binding.cc"), str(stub),
                    *[str(objs[n]) for n in ("registry", "hip_dialect", "device_api", "memory_pool")],
                    "-o", str(exe)], check=True)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    r = subprocess.run([str(exe)], capture_output=True, text=True, env=env)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-6000:]
    assert "ALL OK" in r.stdout
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr and "LeakSanitizer" not in r.stderr
