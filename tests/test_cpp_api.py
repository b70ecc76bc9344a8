"""include/morello_amd.hpp (the C++ mirror of the reference's Spec surface) compiles and its
host-side answers match the reference's expectations.  No GPU needed."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_header_host_surface(tmp_path):
    exe = tmp_path / "cpp_api_check"
    lib_dir = os.path.join(ROOT, "morello_amd")
    cmd = ["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp_api_check.cpp"), "-o", str(exe), "-L", lib_dir, "-lmorello_amd",
           f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0 and "cpp api ok" in run.stdout, run.stdout + run.stderr


def test_common_strided_view_of_two_layouts(tmp_path):
    """morello_amd/csrc/layout_factor.h: the strided view the Move kernels use for Packed / OddEven
    layouts sends every element where the layouts' index expressions send it (named pairs,
    the reference's own layout.rs:1537 example, 300 seeded random pairs)."""
    exe = tmp_path / "layout_view_check"
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "layout_view_check.cpp"), "-o", str(exe)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0 and "layout view ok" in run.stdout, run.stdout[-2000:] + run.stderr
