"""The C++ layer as a C++ caller sees it: tests/cpp/call_sites.cpp is compiled against fuser_amd/csrc/nvf_cutlass.h
and callers.h, linked against the built fuser_amd/_C.so + libnvf_hip.so and run (CPU only: signature checks at
compile time, the validators' failure path at run time)."""
import os
import subprocess
import sys
import sysconfig

import torch
import torch.utils.cpp_extension as ce

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reference_style_call_sites_compile_link_and_run(tmp_path):
    pkg = os.path.join(ROOT, "fuser_amd")
    assert os.path.exists(os.path.join(pkg, "_C.so")), "build the extension first (__graft_entry__.build())"
    exe = str(tmp_path / "call_sites")
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-std=c++17", "-O0", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__",
           os.path.join(ROOT, "tests", "cpp", "call_sites.cpp"), "-o", exe, "-I" + os.path.join(pkg, "csrc"),
           "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"]]
    cmd += ["-I" + p for p in ce.include_paths()]
    pylib = sysconfig.get_config_var("LDLIBRARY")
    cmd += ["-L" + pkg, "-l:_C.so", "-lnvf_hip", "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_python",
            "-L" + (sysconfig.get_config_var("LIBDIR") or "/usr/lib"), "-l:" + pylib if pylib else "-lpython3.10",
            "-Wl,-rpath," + pkg, "-Wl,-rpath," + torch_lib, "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "call sites ok" in r.stdout, r.stdout + r.stderr


def test_host_layer_compiles_against_the_reference_exception_header(tmp_path):
    """With the reference's csrc/ on the include path the host layer takes nvfuser::nvfError, NVF_CHECK and NVF_THROW
    from the reference's own exceptions.h (one definition of the class in a program that links both): the two
    translation units must compile that way and then call the reference's nvfCheckFail instead of throwing the
    stand-in class.  Compile only: the reference's library that defines nvfCheckFail is not built here."""
    import pytest

    ref_csrc = "/root/reference/csrc"
    if not os.path.exists(os.path.join(ref_csrc, "exceptions.h")):
        pytest.skip("the reference tree is not present")
    pkg = os.path.join(ROOT, "fuser_amd")
    for unit in ("nvf_cutlass", "callers"):
        obj = str(tmp_path / (unit + ".o"))
        cmd = ["g++", "-std=c++20", "-O0", "-fPIC", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-DUSE_ROCM",
               "-D__HIP_PLATFORM_AMD__", "-c", os.path.join(pkg, "csrc", unit + ".cpp"), "-o", obj, "-I" + os.path.join(pkg, "csrc"),
               "-I" + os.path.join(ROOT, "include"), "-I" + ref_csrc, "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"]]
        cmd += ["-I" + p for p in ce.include_paths()]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
        assert r.returncode == 0, r.stderr[-3000:]
        syms = subprocess.run(["nm", "-C", obj], capture_output=True, text=True).stdout
        assert "nvfuser::nvfCheckFail" in syms, unit
