"""The ATen-level C++ boundary keeps the reference's signatures: a translation unit written the
way a user of tc::aten writes it (metadata-owning DLTensors from inferOutputTensorInfo, a tuner
subclass that reads tc_, BackendType / MappingOptionsType) must compile against the headers with
tc::HipBackend as the backend.  Compile only: nothing runs on a device."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reference_call_shapes_compile_against_the_hip_backend():
    import torch
    tdir = os.path.dirname(torch.__file__)
    src = os.path.join(ROOT, "tests", "cpp", "aten_signatures.cc")
    cmd = ["g++", "-std=c++17", "-O0", "-c", "-o", os.devnull, "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I", os.path.join(tdir, "include"), "-I", os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I", "/opt/rocm/include", "-I", os.path.join(ROOT, "tensorcomprehensions_amd", "csrc"),
           "-I", os.path.join(ROOT, "include"), src]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
